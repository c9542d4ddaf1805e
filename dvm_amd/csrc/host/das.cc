// Text forms of a kernel: operator graph dump and bytecode disassembly.
// Role in the reference: VKernel::DumpGraph and Code::Das (src/code.cc:27-1498).
// The disassembly is one instruction per line, "<mnemonic>.<type> operands";
// tests pin fusion decisions by counting these mnemonics.
#include <cstdio>
#include <functional>
#include <sstream>

#include "ir.h"
#include "system.h"

namespace dvm {

namespace {

const char *DTypeName(DataType t) {
  switch (t) {
    case kBool: return "bool";
    case kFloat16: return "fp16";
    case kBFloat16: return "bf16";
    case kFloat32: return "fp32";
    case kInt32: return "int32";
    case kInt64: return "int64";
    default: return "?";
  }
}

const char *kUnaryNames[] = {"Sqrt", "Abs", "Log", "Exp", "Reciprocal", "IsFinite", "LogicalNot", "Round", "Floor", "Ceil", "Trunc"};
const char *kBinaryNames[] = {"Equal", "NotEqual", "Greater", "GreaterEqual", "Less", "LessEqual", "Add", "Sub",
                              "Mul", "Div", "Pow", "Maximum", "Minimum", "LogicalAnd", "LogicalOr"};
const char *kReduceNames[] = {"Sum", "Max", "Min"};

void PrintShape(std::ostringstream &os, const NDObject *o) {
  os << "[";
  for (int i = 0; i < o->rank(); ++i) os << (i ? "," : "") << o->dim(i);
  os << "]";
}

const char *kMemTypes[] = {"bool", "fp16", "bf16", "fp32", "int32", "positions"};
const char *kBinF[] = {"Add", "Sub", "RSub", "Mul", "Div", "RDiv", "Min", "Max", "And", "Or", "Pow", "RPow", "Div~", "RDiv~"};
const char *kBinI[] = {"Add", "Sub", "RSub", "Mul", "Min", "Max", "WrapIndex"};
const char *kUn[] = {"Sqrt", "Abs", "Log", "Exp", "IsFinite", "Round", "Floor", "Ceil", "Trunc", "Abs", "Exp", "Exp~", "Exp~", "Log~", "Sqrt~", "SiLU~", "Sigmoid~"};
const char *kCmp[] = {"Eq", "Ne", "Gt", "Ge", "Lt", "Le"};
const char *kRnd[] = {"fp32", "fp16", "bf16", "?"};
const char *kRed[] = {"sum", "max", "min"};
const char *kFmt[] = {"fp32", "fp16", "bf16", "?"};

void PrintSrc(std::ostringstream &os, uint64_t w) {
  char buf[64];
  switch (VI_KIND(w)) {
    case VK_REG: os << "v" << VI_A(w) << "." << kFmt[(VI_SUB(w) >> 6) & 3]; break;
    case VK_SREG: os << "s" << VI_A(w); break;
    case VK_MEM: os << "m" << VI_A(w); break;
    case VK_ACC: os << "acc"; break;
    default:
      std::snprintf(buf, sizeof(buf), "#0x%08x", VI_IMM(w));
      os << buf;
      break;
  }
}

}  // namespace

std::string &VKernel::DumpGraph(bool ref_shapes) {
  (void)ref_shapes;  // compute shapes and API shapes coincide on this backend
  std::ostringstream os;
  os << "kernel " << (name_.empty() ? "dvm" : name_) << " type=" << static_cast<int>(ktype_) << " flags=" << flags_ << "\n";
  for (const NDObject *o : ops_) {
    os << "%" << o->id << " = ";
    switch (o->kind) {
      case kObjLoad: os << "Load"; break;
      case kObjStore: os << "Store"; break;
      case kObjUnary: os << kUnaryNames[o->op]; break;
      case kObjBinary: os << kBinaryNames[o->op]; break;
      case kObjBinaryS: os << kBinaryNames[o->op] << "S" << (o->scalar_left ? "(scalar-left)" : ""); break;
      case kObjCompare: os << kBinaryNames[o->op]; break;
      case kObjCompareS: os << kBinaryNames[o->op] << "S" << (o->scalar_left ? "(scalar-left)" : ""); break;
      case kObjSelect: os << "Select"; break;
      case kObjCast: os << "Cast"; break;
      case kObjBroadcast: os << "Broadcast"; break;
      case kObjBroadcastS: os << "BroadcastS"; break;
      case kObjReduce: os << "Reduce" << kReduceNames[o->op] << (o->keepdims ? "(keepdims)" : ""); break;
      case kObjReshape: os << "Reshape"; break;
      case kObjPermute: os << "Permute"; break;
      case kObjSlice: os << "Slice"; break;
      case kObjConcatPart: os << "ConcatPart"; break;
      case kObjConcat: os << "Concat"; break;
      case kObjCopy: os << "Copy"; break;
      case kObjMatMul:
        os << (o->gmm_type != 0 ? "GroupedMatMul" : "MatMul") << (o->trans_a ? "T" : "N") << (o->trans_b ? "T" : "N");
        if (o->gmm_type != 0) os << "<group_type=" << (o->gmm_type == 1 ? 0 : 2) << ", group_list_type=" << (o->gmm_sizes ? 1 : 0) << ", list=%" << o->group_list->id << ">";
        break;
      case kObjPack64: os << "Pack"; break;
      case kObjOneHot: os << "OneHot<" << o->slice_dim << ">"; break;
      case kObjGather: os << "GatherLoad<" << o->slice_dim << ", gather_mode(" << static_cast<int>(o->op) << ")>"; break;
      case kObjHalf64: os << (o->op == 0 ? "ExtractLo" : "ExtractHi"); break;
    }
    os << "." << DTypeName(o->type_id_) << "(";
    for (int i = 0; i < o->nin; ++i) {
      if (o->in[i] != nullptr) os << (i ? ", " : "") << "%" << o->in[i]->id;
    }
    os << ") ";
    if (normalized_) PrintShape(os, o);
    os << "\n";
  }
  dump_str_ = os.str();
  return dump_str_;
}

std::string &VKernel::DisAssemble() {
  std::ostringstream os;
  if (!compiled_) {
    dump_str_ = "<not compiled>\n";
    return dump_str_;
  }
  int idx = 0;
  for (const Program &p : programs_) {
    os << "== sub-kernel " << idx++ << " ==\n";
    if (p.skip) {
      os << "idle (empty domain), " << p.fills.size() << " clean fill(s)\n";
      continue;
    }
    auto print_code = [&os](const uint64_t *code, uint32_t n_code, const std::function<uint32_t(uint32_t)> &mem_dtype) {
      for (uint32_t i = 0; i < n_code; ++i) {
        const uint64_t w = code[i];
        const uint32_t sub = VI_SUB(w);
        os << "  ";
        switch (VI_OP(w)) {
          case VOP_END: os << "end"; break;
          case VOP_LDR: os << "mov acc, v" << VI_A(w) << "." << kFmt[sub & 3]; break;
          case VOP_LDS: os << "mov acc, s" << VI_A(w); break;
          case VOP_LDI: {
            char buf[32];
            std::snprintf(buf, sizeof(buf), "#0x%08x", VI_IMM(w));
            os << "broadcast_s acc, " << buf;
            break;
          }
          case VOP_STR: os << "mov v" << VI_A(w) << "." << kFmt[sub & 3] << ", acc"; break;
          case VOP_STS: os << "mov s" << VI_A(w) << ", acc"; break;
          case VOP_ST:
            os << "store." << kMemTypes[mem_dtype(VI_A(w))] << " m" << VI_A(w) << ", acc";
            if (static_cast<uint32_t>(w) & VI_ENDS) os << "  ; endsweep";
            break;
          case VOP_UN:
            if (sub == VU_SILU_APPROX || sub == VU_SIGMOID_APPROX) {
              os << kUn[sub] << "." << kRnd[VI_RND(w)] << (sub == VU_SILU_APPROX ? " acc / (exp(acc * #0x" : " 1 / (exp(acc * #0x") << std::hex << VI_IMM(w) << std::dec << ") + 1)";
              break;
            }
            if (sub == VU_EXP_SCALED || sub == VU_EXP_SCALED_APPROX) {
              os << kUn[sub] << "." << kRnd[VI_RND(w)] << " acc * #0x" << std::hex << VI_IMM(w) << std::dec;
              break;
            }
            os << kUn[sub] << "." << (sub == VU_IABS ? "int32" : kRnd[VI_RND(w)]) << " acc";
            break;
          case VOP_CAST: {
            static const char *names[] = {"cast.f2i", "cast.i2f", "cast.round", "cast.f2b"};
            os << names[sub] << "." << kRnd[VI_RND(w)] << " acc";
            break;
          }
          case VOP_RED:
            os << "reduce_" << kRed[sub & 0xf] << ((sub & VRF_SQUARE) ? ".square" : "") << ((sub & VRF_PAIR) ? " (and its square into r1)" : "") << ((sub & VRF_INT) ? ".int32" : "") << " r" << VI_A(w) << ", acc";
            if (static_cast<uint32_t>(w) & VI_ENDS) os << "  ; endsweep";
            break;
          case VOP_SWEEP: os << ((sub & VSW_REVERSE) ? "sweep (last round first) slots=" : "sweep slots=") << kRed[(VI_IMM(w) & 0xf) < 3 ? (VI_IMM(w) & 0xf) : 0]
                             << ((VI_IMM(w) & 0xf) < 3 ? "" : "(none)");
            break;
          case VOP_ENDSWEEP: os << "endsweep"; break;
          case VOP_FIN: os << "mov" << ((sub & VRF_INT) ? ".int32" : "") << " acc, r" << VI_A(w); break;
          case VOP_UNI_BEGIN: os << "per-output run, " << (VI_IMM(w) - 1) << " instructions on one value per lane (first wave only when the team is the workgroup)"; break;
          case VOP_UNI_END: os << "end of per-output run"; break;
          case VOP_LD:
            os << "load." << kMemTypes[mem_dtype(VI_A(w))] << " acc, m" << VI_A(w);
            if (static_cast<uint32_t>(w) & (VI_LD_KEEP_WR | VI_LD_KEEP_RD)) {
              const bool wr = (static_cast<uint32_t>(w) & VI_LD_KEEP_WR) != 0;
              os << (wr ? "  ; parks its first " : "  ; takes its first ") << (VI_IMM(w) & 0xffffu) << (wr ? " rounds in local memory" : " rounds from local memory");
              if ((VI_IMM(w) >> 16) & 3u) os << " (the value behind the next instruction, as " << kFmt[(VI_IMM(w) >> 20) & 3u] << ")";
            }
            if (static_cast<uint32_t>(w) & VI_LD_PAIR) os << "  ; fetches the next instruction's operand in the same trip";
            if (static_cast<uint32_t>(w) & VI_LD_RED2) os << "  ; fetches several rounds per trip and does the reduce behind it";
            break;
          case VOP_BINF:
            if (VI_KIND(w) == VK_SREG2) {  // two chained operations
              const uint32_t second = VI_IMM(w);
              os << kBinF[sub & 0x3f] << "." << kRnd[VI_RND(w)] << " acc, s" << VI_A(w) << "  ; then " << kBinF[second & 0x3f] << "."
                 << kRnd[(second >> 16) & 3] << " acc, s" << ((second >> 8) & 0xff);
              break;
            }
            if (VI_KIND(w) == VK_MEM && (VI_IMM(w) & VI_PRE_SREG)) {
              os << kBinF[VI_IMM(w) & 0x3f] << "." << kRnd[(VI_IMM(w) >> 16) & 3] << " acc, s" << ((VI_IMM(w) >> 8) & 0xff) << "  ; then ";
            }
            os << kBinF[sub & 0x3f] << "." << kRnd[VI_RND(w)] << " acc, ";
            PrintSrc(os, w);
            break;
          case VOP_BINI: os << kBinI[sub & 0x3f] << ".int32 acc, "; PrintSrc(os, w); break;
          case VOP_CMP: os << "Cmp" << kCmp[sub & 7] << "." << ((sub & VCMP_INT) ? "int32" : "fp32") << " acc, "; PrintSrc(os, w); break;
          case VOP_LDX: os << "gather_load." << kMemTypes[mem_dtype(VI_A(w))] << " acc, m" << VI_A(w) << " + acc"; break;
          case VOP_MSK: os << "mask "; PrintSrc(os, w); break;
          case VOP_MOVM: os << "select acc, "; PrintSrc(os, w); break;
          default: os << "?"; break;
        }
        if (VI_OP(w) > VOP_LD && VI_KIND(w) == VK_MEM && (static_cast<uint32_t>(w) & VI_OFFS_ASIDE)) os << "  ; offsets of its own (those before it stay current)";
        os << "\n";
      }
    };
    const VVecHeader *h = reinterpret_cast<const VVecHeader *>(p.blob.w);
    if (h->entry == VE_VECTOR) {
      static const char *sched[] = {"pointwise", "reduce-x", "reduce-y"};
      os << "entry vector sched=" << sched[h->sched & VS_KIND_MASK] << ((h->sched & VS_WIDE) ? " wide" : "") << ((h->sched & VS_SWEEPS) ? " sweeps" : "") << " blocks=" << p.grid << " threads=" << p.threads
         << " lds=" << p.lds_bytes << " items=" << h->n_items << " kept=" << h->n_kidx << " red=" << h->n_ridx
         << " inner=" << h->inner_extent << " team=" << (h->team_is_block ? p.threads : (1u << h->team_log2))
         << " vslots=" << h->n_vslot;
      if (h->r_chunk != 0 && h->k_per_chunk != 0) os << " shared-reduce parts=" << h->n_kidx / h->k_per_chunk << " x " << h->r_chunk;
      os << "\n";
      os << "  kdims:";
      for (uint32_t i = 0; i < h->n_kdim; ++i) os << " " << h->kdims[i].extent;
      os << "  rdims:";
      for (uint32_t i = 0; i < h->n_rdim; ++i) os << " " << h->rdims[i].extent;
      os << "\n";
      const VMemDesc *mems = reinterpret_cast<const VMemDesc *>(p.blob.w + h->mem_off);
      for (uint32_t i = 0; i < h->n_mem; ++i) {
        char buf[32];
        std::snprintf(buf, sizeof(buf), "0x%llx", static_cast<unsigned long long>(mems[i].addr));
        os << "  m" << i << ": " << kMemTypes[mems[i].dtype] << " @" << buf << ((mems[i].flags & VMF_VEC) ? " vec" : (mems[i].flags & VMF_GATHER) ? " gather" : " bcast")
           << ((mems[i].flags & VMF_ALIGNED) ? " aligned" : "") << " k[";
        for (uint32_t j = 0; j < h->n_kdim; ++j) os << (j ? "," : "") << mems[i].kstride[j];
        os << "] r[";
        for (uint32_t j = 0; j < h->n_rdim; ++j) os << (j ? "," : "") << mems[i].rstride[j];
        os << "]\n";
      }
      print_code(p.blob.w + h->code_off, h->n_code, [&](uint32_t m) { return mems[m].dtype; });
    } else if (h->entry == VE_CUBE) {
      const VCubeHeader *c = reinterpret_cast<const VCubeHeader *>(p.blob.w);
      static const int tile[] = {256, 128, 64, 256};
      os << "entry cube " << kMemTypes[c->dtype] << " m=" << c->m << " n=" << c->n << " k=" << c->k << " trans_a=" << c->trans_a
         << " trans_b=" << c->trans_b << " batch=" << c->nb0 << "x" << c->nb1 << " tile=" << tile[c->tile] << " blocks=" << p.grid
         << " lds=" << p.lds_bytes << (c->fast ? " fast" : " guarded") << (c->tile == 3 ? " eight-waves" : "");
      if (c->epi_flags & VCF_PLAIN_STORE) os << " plain-store";
      else if (c->epi_flags & VCF_SLIM) os << " slim-epilogue";
      if (c->epi_flags & VCF_DUMP16) os << " tile-as-16-bit";
      if (c->epi_flags & VCF_SPLITK_PARTIAL) os << " split-k partials " << c->k_split << " x " << c->k_chunk;
      if (c->epi_flags & VCF_SPLITK_COMBINE) os << " split-k sum of " << c->k_split;
      if (c->group_mode != VCG_NONE) {
        static const char *gm[] = {"", "rows by bounds", "rows by sizes", "k by bounds", "k by sizes"};
        os << " groups=" << c->nb1 << " (" << gm[c->group_mode <= VCG_K_SIZE ? c->group_mode : 0] << ", " << (c->group_i32 ? "int32" : "int64") << " list)";
      }
      os << "\n";
      const VCubeMem *cm = reinterpret_cast<const VCubeMem *>(p.blob.w + c->mem_off);
      for (uint32_t i = 0; i < c->n_mem; ++i) {
        char buf[32];
        std::snprintf(buf, sizeof(buf), "0x%llx", static_cast<unsigned long long>(cm[i].addr));
        os << "  m" << i << ": " << kMemTypes[cm[i].dtype] << " @" << buf << " strides n=" << cm[i].stride_n << " m=" << cm[i].stride_m
           << " b=" << cm[i].stride_b0 << "," << cm[i].stride_b1 << "\n";
      }
      if (c->epi_flags & VCF_SPLITK_PARTIAL) {
        os << "  mmad acc, A, B\n  store.fp32 partials, acc\n";
        continue;
      }
      os << ((c->epi_flags & VCF_SPLITK_COMBINE) ? "  sum acc, partials\n" : "  mmad acc, A, B\n");
      print_code(p.blob.w + c->code_off, c->n_code, [&](uint32_t m) { return cm[m].dtype; });
    } else if (h->entry == VE_ATTN) {
      const VAttnHeader *a = reinterpret_cast<const VAttnHeader *>(p.blob.w);
      os << "entry attention " << kMemTypes[a->dtype] << " batch=" << a->nb << " sq=" << a->sq << " skv=" << a->skv << " d=" << a->d
         << " scale=" << a->scale << " blocks=" << p.grid << " lds=" << p.lds_bytes << "\n";
      {
        static const char *names[4] = {"q", "k", "v", "o"};
        const uint32_t rows[4] = {a->sq, a->skv, a->skv, a->sq};
        for (int i = 0; i < 4; ++i) {  // operands that are not dense [batch][rows][d]
          const bool dense = a->row_stride[i] == a->d && (a->nb_inner == 1 ? a->outer_stride[i] == rows[i] * a->d
                                                                           : (a->inner_stride[i] == rows[i] * a->d && a->outer_stride[i] == rows[i] * a->d * a->nb_inner));
          if (!dense) os << "  " << names[i] << ": view, strides row=" << a->row_stride[i] << " batch=" << a->outer_stride[i] << "," << a->inner_stride[i]
                         << " (inner batch extent " << a->nb_inner << ")\n";
        }
      }
      os << "  mmad s, K, Q^T\n  online_softmax p, s\n  mmad o, V^T, p\n  store o\n";
    } else {
      os << "entry type " << h->entry << " blocks=" << p.grid << " threads=" << p.threads << "\n";
    }
  }
  dump_str_ = os.str();
  return dump_str_;
}

std::string &VKernel::Inspect() {
  std::ostringstream os;
  if (!g_system.HasDevice()) os << "warning: LaunchNone (" << g_system.LoadError() << ")\n";
  if (!compiled_) os << "warning: not compiled\n";
  for (const NDObject *o : ops_) {
    if ((o->kind == kObjLoad || o->kind == kObjStore) && o->addr == nullptr) {
      os << "note: %" << o->id << " has no address yet\n";
    }
  }
  dump_str_ = os.str();
  return dump_str_;
}

}  // namespace dvm
