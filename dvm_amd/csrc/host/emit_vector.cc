// Accumulator-machine code for vector sub-kernels: memory operand descriptors, registers, sections, programs.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "compiler.h"

namespace dvm {

// emission helpers
void Compiler::Emit(uint32_t op, uint32_t sub, uint32_t kind, uint32_t rnd, uint32_t a, uint32_t imm) {
  uint64_t w = VI_MAKE(op, sub, kind, rnd, a, imm);
  if (op == VOP_ENDSWEEP) w |= VI_ENDS;
  if (!cube_mode_) {
    const bool mem = op == VOP_ST || (op >= VOP_SRC_BASE && kind == VK_MEM);
    if (mem) {
      // consecutive memory instructions of one round that walk memory identically share their offsets
      if (last_mem_ >= 0 && std::memcmp(mems_[last_mem_].kstride, mems_[a].kstride, sizeof(mems_[a].kstride)) == 0 &&
          std::memcmp(mems_[last_mem_].rstride, mems_[a].rstride, sizeof(mems_[a].rstride)) == 0) {
        w |= VI_SAME_OFFS;
        last_mem_ = static_cast<int>(a);
      } else if (last_mem_ >= 0 && op != VOP_ST && op != VOP_LD) {
        w |= VI_OFFS_ASIDE;  // an operand on a path of its own: the offsets of the instruction before stay current
      } else {
        last_mem_ = static_cast<int>(a);
      }
    } else if (op == VOP_SWEEP || op == VOP_ENDSWEEP) {
      last_mem_ = -1;
    } else if (uniform_emit_ && (op == VOP_UN || op == VOP_CAST ||
                                 ((op == VOP_BINF || op == VOP_BINI || op == VOP_CMP) && (kind == VK_IMM || kind == VK_SREG || kind == VK_ACC)))) {
      w |= VI_UNIFORM;
    }
  }
  code_.push_back(w);
}

// ---------- emission ----------

int Compiler::MemIndex(int v) {
  ANode &n = nodes_[v];
  if (n.mem_idx >= 0) return n.mem_idx;
  if (cube_mode_) return CubeMemIndex(v);
  if (n_mem_ >= DVM_VEC_MAXMEM) Fail("too many memory operands");
  VMemDesc &m = mems_[n_mem_];
  std::memset(&m, 0, sizeof(m));
  // (a OneHot's own operand: the positions along its new dim, no memory behind them)
  const bool iota = n.kind == AK_OP && n.op->kind == kObjOneHot;
  m.dtype = iota ? VDT_IOTA : MemDType(n.dtype);
  // element stride of every axis the operand has (row-major over its own shape)
  int64_t stride = 1;
  int64_t dim_stride[kMaxAxes];
  bool dim_has[kMaxAxes] = {false};
  for (int d = n.rank - 1; d >= 0; --d) {
    if (n.axis[d] >= 0) {
      const int p = pos_[n.axis[d]];
      const int md = dim_of_axis_[p];
      dim_has[md] = true;
      // the innermost axis of a merged dim carries its stride; a strided view brings its own
      if (p == dims_[md].last_axis) dim_stride[md] = n.view != nullptr ? n.view->vstride_[d] : stride;
    }
    stride *= n.dims[d];
  }
  const int inner = n_dims_ - 1;
  bool aligned = true;
  const int64_t isz = iota ? 4 : static_cast<int64_t>(DTypeSize(n.dtype));
  const int64_t need = isz * E >= 16 ? 16 : isz * E;
  for (int i = 0; i < nk_; ++i) {
    const int md = klist_[i];
    if (!dim_has[md]) continue;
    if (dim_stride[md] >= (1ll << 32)) Fail("stride above 2^32");
    m.kstride[i] = static_cast<uint32_t>(dim_stride[md]);
    if (md != inner && (dim_stride[md] * isz) % need != 0) aligned = false;
  }
  if (split_inner_ && dim_has[inner]) {  // the tiles of 64 along the innermost axis are the outermost kept dim
    if (dim_stride[inner] * 64 >= (1ll << 32)) Fail("stride above 2^32");
    m.kstride[nk_] = static_cast<uint32_t>(dim_stride[inner] * 64);
  }
  for (int i = 0; i < nr_; ++i) {
    const int md = rlist_[i];
    if (!dim_has[md]) continue;
    if (dim_stride[md] >= (1ll << 32)) Fail("stride above 2^32");
    m.rstride[i] = static_cast<uint32_t>(dim_stride[md]);
    if (md != inner && (dim_stride[md] * isz) % need != 0) aligned = false;
  }
  for (int i = 0; i < n_peel_; ++i) {
    const int md = peel_dim_[i];
    peel_stride_[n_mem_][i] = dim_has[md] ? dim_stride[md] * isz : 0;  // in bytes
    if (peel_stride_[n_mem_][i] % need != 0) aligned = false;
  }
  if (dim_has[inner] && dims_[inner].first_axis >= 0) {
    if (dim_stride[inner] == 1) {
      m.flags |= VMF_VEC;
      if (aligned) m.flags |= VMF_ALIGNED;
    } else if (n.view != nullptr && dim_stride[inner] != 0) {
      // a transposing or element-skipping view: element by element (correct, not fast)
      if (dim_stride[inner] >= (1ll << 24) || dim_stride[inner] < 0) Fail("innermost stride above 2^24");
      m.flags |= VMF_GATHER | (static_cast<uint32_t>(dim_stride[inner]) << 8);
    } else if (dim_stride[inner] != 0) {
      Fail("innermost axis is not contiguous");
    }
  }
  if (iota) m.flags &= ~static_cast<uint32_t>(VMF_ALIGNED);  // element by element: the 128-bit paths would read memory
  Program::Patch p;
  p.word = static_cast<uint32_t>(sizeof(VVecHeader) / 8 + n_mem_ * (sizeof(VMemDesc) / 8));
  p.op_id = n.addr_op;
  p.ws_slot = n.ws_slot;
  p.byte_offset = n.view != nullptr ? n.view->view_base_ * isz : 0;
  mem_is_view_[n_mem_] = n.view != nullptr;
  p.role = iota ? Program::kPatchIota : Program::kPatchVecMem;
  prog_->patches.push_back(p);
  n.mem_idx = n_mem_++;
  return n.mem_idx;
}

int Compiler::AllocSReg() {
  for (int i = 0; i < DVM_VEC_NSREG; ++i) {
    if (!((sreg_used_ >> i) & 1u)) {
      sreg_used_ |= 1u << i;
      return i;
    }
  }
  Fail("out of S registers");
  return -1;
}

int Compiler::AllocVSlot(int n) {
  for (int i = 0; i + n <= vslot_limit_; ++i) {
    const uint32_t msk = ((1u << n) - 1u) << i;
    if ((vslot_used_ & msk) == 0) {
      vslot_used_ |= msk;
      max_vslot_ = std::max(max_vslot_, i + n);
      return i;
    }
  }
  Fail("out of V register slots");
  return -1;
}

void Compiler::ReleaseReg(int v) {
  ANode &n = nodes_[v];
  if (n.reg < 0) return;
  if (!n.has_inner) {
    sreg_used_ &= ~(1u << n.reg);
  } else {
    const int cnt = (n.reg_fmt == VF_F32 && !cube_mode_) ? 2 : 1;
    vslot_used_ &= ~(((1u << cnt) - 1u) << n.reg);
  }
  n.reg = -1;
}

void Compiler::SaveAcc(int v) {
  ANode &n = nodes_[v];
  if (n.reg >= 0) return;
  if (!n.has_inner) {
    n.reg = AllocSReg();
    Emit(VOP_STS, 0, 0, 0, n.reg, 0);
  } else if (cube_mode_) {
    // fragment temporaries hold the fp32 container as it is
    n.reg_fmt = VF_F32;
    n.reg = AllocVSlot(1);
    Emit(VOP_STR, 0, 0, 0, n.reg, 0);
  } else {
    n.reg_fmt = n.dtype == kFloat16 ? VF_F16 : (n.dtype == kBFloat16 ? VF_BF16 : VF_F32);
    if (n.dtype == kBool) n.reg_fmt = VF_F16;
    n.reg = AllocVSlot(n.reg_fmt == VF_F32 ? 2 : 1);
    Emit(VOP_STR, n.reg_fmt, 0, 0, n.reg, 0);
  }
}

// Called before an instruction replaces the accumulator by an unrelated value.
void Compiler::BeforeOverwrite() {
  if (acc_node_ < 0) return;
  ANode &n = nodes_[acc_node_];
  if (n.kind == AK_MEM || n.kind == AK_SCALAR) return;  // cheaper to fetch again than to park
  const bool needed_later = n.last_sec > cur_sec_ && (!n.fd || single_round_);
  if (n.kind == AK_REDUCE && n.slot_ready && !needed_later) return;  // still in its slot
  if ((n.uses > 0 || needed_later) && n.reg < 0) SaveAcc(acc_node_);
}

void Compiler::ConsumeUse(int v) {
  ANode &n = nodes_[v];
  if (n.uses > 0) --n.uses;
  const bool needed_later = n.last_sec > cur_sec_ && (!n.fd || single_round_);
  if (n.uses != 0 || needed_later || n.reg < 0) return;
  // A sweep of several rounds runs its instructions again: a value from an earlier section keeps its
  // register until the sweep ends, or a temporary of round one would replace it before round two reads it.
  if ((cur_sec_ & 1) && !single_round_ && n.sec < cur_sec_) {
    bool listed = false;
    for (int i = 0; i < n_held_; ++i) listed |= held_[i] == v;
    if (!listed) held_[n_held_++] = v;
    return;
  }
  ReleaseReg(v);
}

bool Compiler::SimpleOperand(int v) {
  const ANode &n = nodes_[v];
  if (n.reg >= 0) return true;
  if (acc_node_ == v) return false;
  return n.kind == AK_MEM || n.kind == AK_SCALAR;
}

// acc = acc (op) value-of-v, v being a simple operand.
void Compiler::EmitOperandInsn(uint32_t op, uint32_t sub, uint32_t rnd, int v) {
  ANode &n = nodes_[v];
  if (n.reg >= 0) {
    if (!n.has_inner) {
      Emit(op, sub, VK_SREG, rnd, n.reg, 0);
    } else {
      Emit(op, sub | (static_cast<uint32_t>(n.reg_fmt) << 6), VK_REG, rnd, n.reg, 0);
    }
  } else if (n.kind == AK_MEM) {
    Emit(op, sub, VK_MEM, rnd, MemIndex(v), 0);
  } else if (n.kind == AK_SCALAR) {
    Emit(op, sub, VK_IMM, rnd, 0, ScalarToContainer(n.op->scalar.Get(), n.dtype, n.op->half64));
  } else {
    Fail("operand is not addressable");
  }
  ConsumeUse(v);
}

// Puts value v into the accumulator.
void Compiler::EmitValue(int v) {
  v = Resolve(v);
  if (acc_node_ == v) return;
  ANode &n = nodes_[v];
  if (n.reg >= 0) {
    BeforeOverwrite();
    if (!n.has_inner) {
      Emit(VOP_LDS, 0, 0, 0, n.reg, 0);
    } else {
      Emit(VOP_LDR, n.reg_fmt, 0, 0, n.reg, 0);
    }
    acc_node_ = v;
    return;
  }
  if (n.kind == AK_REDUCE && n.slot_ready) {
    BeforeOverwrite();
    Emit(VOP_FIN, n.dtype == kInt32 ? VRF_INT : 0, 0, 0, n.slot, 0);
    acc_node_ = v;
    return;
  }
  ComputeInto(v);
  acc_node_ = v;
}

namespace {
uint32_t BinSubF(int op, bool reversed) {
  switch (op) {
    case kAdd: return VB_ADD;
    case kSub: return reversed ? VB_RSUB : VB_SUB;
    case kMul: return VB_MUL;
    case kDiv: return reversed ? VB_RDIV : VB_DIV;
    case kPow: return reversed ? VB_RPOW : VB_POW;
    case kMaximum: return VB_MAX;
    case kMinimum: return VB_MIN;
    case kLogicalAnd: return VB_AND;
    case kLogicalOr: return VB_OR;
    default: Throw("binary operator without a device form");
  }
}
uint32_t BinSubI(int op, bool reversed) {
  switch (op) {
    case kAdd: return VBI_ADD;
    case kSub: return reversed ? VBI_RSUB : VBI_SUB;
    case kMul: return VBI_MUL;
    case kMaximum: return VBI_MAX;
    case kMinimum: return VBI_MIN;
    default: Throw("binary operator without an int32 form");
  }
}
uint32_t CmpSub(int op, bool reversed, bool is_int) {
  static const uint32_t rev[6] = {VCMP_EQ, VCMP_NE, VCMP_LT, VCMP_LE, VCMP_GT, VCMP_GE};
  uint32_t t = static_cast<uint32_t>(op);  // kEqual..kLessEqual == VCMP_EQ..VCMP_LE
  if (reversed) t = rev[t];
  return t + (is_int ? VCMP_INT : 0);
}
bool NeedsRounding(int op) { return op == kAdd || op == kSub || op == kMul || op == kDiv || op == kPow; }
}  // namespace

// Emits the code that computes v (not in a register, not in the accumulator).
void Compiler::ComputeInto(int v) {
  ANode &n = nodes_[v];
  NDObject *o = n.op;
  // outside the sweeps of a reduce kernel, a value without the innermost axis is one number per lane
  struct UniformScope {
    bool &flag, saved;
    UniformScope(bool &f, bool v) : flag(f), saved(f) { flag = v; }
    ~UniformScope() { flag = saved; }
  } scope(uniform_emit_, !cube_mode_ && nr_ > 0 && (cur_sec_ & 1) == 0 && !n.has_inner && n.kind == AK_OP);
  switch (n.kind) {
    case AK_MEM:
      BeforeOverwrite();
      Emit(VOP_LD, 0, VK_MEM, 0, MemIndex(v), 0);
      return;
    case AK_SCALAR:
      BeforeOverwrite();
      Emit(VOP_LDI, 0, 0, 0, 0, ScalarToContainer(o->scalar.Get(), n.dtype, o->half64));
      return;
    case AK_REDUCE:
      Fail("reduce result used before it is complete");
      return;
    default:
      break;
  }
  const bool is_int = (o->kind == kObjCompare || o->kind == kObjCompareS || o->kind == kObjBinary ||
                       o->kind == kObjBinaryS || o->kind == kObjUnary)
                          ? o->in[0]->type_id_ == kInt32
                          : false;
  switch (o->kind) {
    case kObjUnary: {
      const int x = Resolve(n.in[0]);
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      uint32_t sub;
      bool rnd = false;
      switch (o->op) {
        case kSqrt: sub = VU_SQRT; rnd = true; break;
        case kAbs: sub = is_int ? VU_IABS : VU_ABS; break;
        case kLog: sub = VU_LOG; rnd = true; break;
        case kExp: sub = VU_EXP; rnd = true; break;
        case kIsFinite: sub = VU_ISFINITE; break;
        case kRound: sub = VU_ROUND; break;
        case kFloor: sub = VU_FLOOR; break;
        case kCeil: sub = VU_CEIL; break;
        case kTrunc: sub = VU_TRUNC; break;
        default: Throw("unary operator without a device form");
      }
      Emit(VOP_UN, sub, 0, rnd ? RndOf(n.dtype) : 0, 0, 0);
      return;
    }
    case kObjCast: {
      const int x = Resolve(n.in[0]);
      const DataType s = o->in[0]->type_id_, d = n.dtype;
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      if (d == kInt32) {
        Emit(VOP_CAST, VC_F2I, 0, 0, 0, 0);
      } else if (s == kInt32) {
        Emit(VOP_CAST, VC_I2F, 0, RndOf(d), 0, 0);
      } else if (d == kBool) {
        Emit(VOP_CAST, VC_F2B, 0, 0, 0, 0);
      } else {
        Emit(VOP_CAST, VC_RND, 0, RndOf(d), 0, 0);
      }
      return;
    }
    case kObjBinaryS:
    case kObjCompareS: {
      const int x = Resolve(n.in[0]);
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      const uint32_t imm = ScalarToContainer(o->scalar.Get(), o->in[0]->type_id_);
      if (o->kind == kObjCompareS) {
        Emit(VOP_CMP, CmpSub(o->op, o->scalar_left, is_int), VK_IMM, 0, 0, imm);
      } else if (is_int) {
        Emit(VOP_BINI, BinSubI(o->op, o->scalar_left), VK_IMM, 0, 0, imm);
      } else {
        Emit(VOP_BINF, BinSubF(o->op, o->scalar_left), VK_IMM, NeedsRounding(o->op) ? RndOf(n.dtype) : 0, 0, imm);
      }
      return;
    }
    case kObjBinary:
    case kObjCompare: {
      int a = Resolve(n.in[0]), b = Resolve(n.in[1]);
      bool reversed = false;
      uint32_t opc, sub, rnd = 0;
      auto pick = [&](bool rev) {
        if (o->kind == kObjCompare) {
          opc = VOP_CMP;
          sub = CmpSub(o->op, rev, is_int);
        } else if (is_int) {
          opc = VOP_BINI;
          sub = BinSubI(o->op, rev);
        } else {
          opc = VOP_BINF;
          sub = BinSubF(o->op, rev);
          rnd = NeedsRounding(o->op) ? RndOf(n.dtype) : 0;
        }
      };
      if (a == b) {
        EmitValue(a);
        ConsumeUse(a);
        ConsumeUse(a);
        BeforeOverwrite();
        pick(false);
        Emit(opc, sub, VK_ACC, rnd, 0, 0);
        return;
      }
      if (acc_node_ == b) {
        std::swap(a, b);
        reversed = true;
      }
      if (acc_node_ == a) {
        if (!SimpleOperand(b)) {
          // computing b would clobber a: park a, compute b, then use a as the operand
          SaveAcc(a);
          EmitValue(b);
          std::swap(a, b);
          reversed = !reversed;
        }
      } else if (SimpleOperand(b)) {
        EmitValue(a);
      } else if (SimpleOperand(a)) {
        EmitValue(b);
        std::swap(a, b);
        reversed = true;
      } else {
        EmitValue(b);
        if (SimpleOperand(a)) {
          // a was computed and parked on the way to b (b is a function of a, as in x / (exp(-x) + 1))
          std::swap(a, b);
          reversed = true;
        } else {
          SaveAcc(b);
          EmitValue(a);
        }
      }
      ConsumeUse(a);
      BeforeOverwrite();
      pick(reversed);
      EmitOperandInsn(opc, sub, rnd, b);
      return;
    }
    case kObjSelect: {
      const int c = Resolve(n.in[0]), x = Resolve(n.in[1]), y = Resolve(n.in[2]);
      if (!SimpleOperand(c)) {
        EmitValue(c);
        SaveAcc(c);
      }
      if (!SimpleOperand(x)) {
        EmitValue(x);
        SaveAcc(x);
      }
      EmitValue(y);
      ConsumeUse(y);
      BeforeOverwrite();
      EmitOperandInsn(VOP_MSK, 0, 0, c);
      EmitOperandInsn(VOP_MOVM, 0, 0, x);
      return;
    }
    case kObjOneHot: {
      const int x = Resolve(n.in[0]);
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      // index == position along the new dim ? on : off
      Emit(VOP_CMP, VCMP_EQ + VCMP_INT, VK_MEM, 0, MemIndex(v), 0);
      Emit(VOP_MSK, 0, VK_ACC, 0, 0, 0);
      Emit(VOP_LDI, 0, 0, 0, 0, ScalarToContainer(o->scalar2.Get(), n.dtype));
      Emit(VOP_MOVM, 0, VK_IMM, 0, 0, ScalarToContainer(o->scalar.Get(), n.dtype));
      return;
    }
    case kObjGather: {
      const int x = Resolve(n.in[0]);
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      // the index becomes an offset in elements: wrapped into the gathered dim, times that dim's stride
      Emit(VOP_BINI, VBI_WRAP, VK_IMM, 0, 0, static_cast<uint32_t>(o->gather_extent));
      if (o->gather_stride != 1) Emit(VOP_BINI, VBI_MUL, VK_IMM, 0, 0, static_cast<uint32_t>(o->gather_stride));
      Emit(VOP_LDX, 0, VK_MEM, 0, MemIndex(v), 0);
      return;
    }
    default:
      Fail("operator without a vector form");
  }
}

// Counts, for the section being emitted, how often each value of the cone is read.
void Compiler::CountCone(int v) {
  v = Resolve(v);
  ANode &n = nodes_[v];
  ++n.uses;
  if (n.in_cone) return;
  n.in_cone = true;
  if (n.reg >= 0 || n.kind == AK_MEM || n.kind == AK_SCALAR || n.kind == AK_REDUCE) return;
  for (int j = 0; j < n.nin; ++j)
    if (n.in[j] >= 0) CountCone(n.in[j]);
}

void Compiler::EmitSection(int sec) {
  cur_sec_ = sec;
  last_mem_ = -1;
  const bool sweep = (sec & 1) != 0;
  for (int i = 0; i < nn_; ++i) {
    nodes_[i].uses = 0;
    nodes_[i].in_cone = false;
  }
  if (!sweep && sec > 0) {
    // The previous sweep's reduces have their results in the slots, where this section reads them as often as
    // it likes; a result that a later section needs becomes a register value now (the next sweep reuses the slots).
    for (int i = 0; i < nn_; ++i) {
      ANode &n = nodes_[i];
      if (n.kind != AK_REDUCE || n.sec != sec - 1) continue;
      n.slot_ready = true;
      if (n.last_sec <= sec) continue;
      BeforeOverwrite();
      Emit(VOP_FIN, n.dtype == kInt32 ? VRF_INT : 0, 0, 0, n.slot, 0);
      acc_node_ = i;
      SaveAcc(i);
    }
  }
  // sinks of this section, in node order
  int sinks[kMaxNodes];
  int ns = 0;
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if ((n.kind == AK_REDUCE || n.kind == AK_OUT) && n.sec == sec) sinks[ns++] = i;
  }
  // values computed here that a later section reads from a register
  int keep[kMaxNodes];
  int nkp = 0;
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.sec != sec || n.last_sec <= sec) continue;
    if (n.kind == AK_MEM) {
      // an operand that does not vary inside the sweeps is loaded once per output into an S register
      if (sweep || n.has_inner || n_sec_ == 1) continue;
      if (__builtin_popcount(sreg_used_) >= DVM_VEC_NSREG - 3) continue;
      keep[nkp++] = i;
      continue;
    }
    if (n.kind != AK_OP) continue;
    if (n.fd && !single_round_) continue;  // recomputed by the later sweep
    keep[nkp++] = i;
  }
  if (sweep) {
    uint32_t kinds = 0xff;
    int slot = 0;
    for (int i = 0; i < ns; ++i) {
      ANode &n = nodes_[sinks[i]];
      if (n.kind != AK_REDUCE) continue;
      if (slot >= DVM_VEC_NSLOT) Fail("more than two reduces in one sweep");
      const uint32_t rk = n.op->op == kSum ? VR_SUM : (n.op->op == kMax ? VR_MAX : VR_MIN);
      kinds = (kinds & ~(0xfu << (4 * slot))) | (rk << (4 * slot));
      n.slot = slot;
      ++slot;
    }
    BeforeOverwrite();
    for (int i = 0; i < nn_; ++i) nodes_[i].slot_ready = false;  // the sweep starts its slots afresh
    Emit(VOP_SWEEP, 0, 0, 0, 0, kinds);
    if (!single_round_) acc_node_ = -1;
  }
  for (int i = 0; i < ns; ++i) CountCone(nodes_[sinks[i]].in[0]);
  for (int i = 0; i < nkp; ++i) CountCone(keep[i]);
  for (int i = 0; i < ns; ++i) {
    ANode &n = nodes_[sinks[i]];
    const int x = Resolve(n.in[0]);
    EmitValue(x);
    if (n.kind == AK_REDUCE) {
      const uint32_t rk = n.op->op == kSum ? VR_SUM : (n.op->op == kMax ? VR_MAX : VR_MIN);
      Emit(VOP_RED, rk | (n.dtype == kInt32 ? VRF_INT : 0), 0, 0, n.slot, 0);
    } else {
      Emit(VOP_ST, 0, 0, 0, MemIndex(sinks[i]), 0);
    }
    ConsumeUse(x);
  }
  for (int i = 0; i < nkp; ++i) {
    const int v = keep[i];
    if (nodes_[v].reg < 0) {
      EmitValue(v);
      SaveAcc(v);
    }
    ConsumeUse(v);
  }
  if (sweep) {
    if (!single_round_) BeforeOverwrite();
    Emit(VOP_ENDSWEEP, 0, 0, 0, 0, 0);
    if (!single_round_) acc_node_ = -1;
  }
  for (int i = 0; i < n_held_; ++i)
    if (nodes_[held_[i]].uses == 0) ReleaseReg(held_[i]);
  n_held_ = 0;
}

void Compiler::EmitProgram() {
  const int inner = n_dims_ - 1;
  const int inner_first = dims_[inner].first_axis, inner_last = dims_[inner].last_axis;
  // classify values
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    n.has_inner = false;
    n.fd = false;
    for (int d = 0; d < n.rank; ++d) {
      if (n.axis[d] < 0) continue;
      const int p = pos_[n.axis[d]];
      if (inner_first >= 0 && p >= inner_first && p <= inner_last) n.has_inner = true;
      if (axes_[n.axis[d]].reduced) n.fd = true;
    }
    // Only a value that is the same for every slab of a lane fits an S register: slabs differ in
    // the kept position (pointwise) or in the reduce position (sweeps).
    if (n.fd || nr_ == 0) n.has_inner = true;
  }
  int max_level = 0;
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    n.level = 0;
    for (int j = 0; j < n.nin; ++j) {
      if (n.in[j] < 0) continue;
      const ANode &x = nodes_[n.in[j]];
      n.level = std::max(n.level, x.level + (x.kind == AK_REDUCE ? 1 : 0));
    }
    if (n.kind == AK_REDUCE) {
      // the reduce runs in the sweep of its input's level
      n.sec = 2 * n.level + 1;
    } else if (nr_ == 0) {
      n.sec = 0;
    } else {
      n.sec = 2 * n.level + (n.fd ? 1 : 0);
    }
    max_level = std::max(max_level, n.level);
  }
  // aliases inherit the class of what they resolve to
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    if (n.kind == AK_ALIAS) {
      const ANode &r = nodes_[Resolve(i)];
      n.sec = r.sec;
    }
  }
  // an output's section is that of the value it stores
  n_sec_ = nr_ == 0 ? 1 : 2 * (max_level + 1);
  for (int i = 0; i < nn_; ++i) nodes_[i].last_sec = -1;
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    if (n.kind == AK_ALIAS) continue;
    const int my_sec = n.sec;
    for (int j = 0; j < n.nin; ++j) {
      if (n.in[j] < 0) continue;
      ANode &x = nodes_[Resolve(n.in[j])];
      x.last_sec = std::max(x.last_sec, my_sec);
    }
  }
  // values recomputed by a later sweep pull their own inputs forward
  if (!single_round_) {
    for (int pass = 0; pass < nn_; ++pass) {
      bool changed = false;
      for (int i = nn_ - 1; i >= 0; --i) {
        ANode &n = nodes_[i];
        if (n.kind != AK_OP || !n.fd) continue;
        for (int j = 0; j < n.nin; ++j) {
          if (n.in[j] < 0) continue;
          ANode &x = nodes_[Resolve(n.in[j])];
          if (x.last_sec < n.last_sec) {
            x.last_sec = n.last_sec;
            changed = true;
          }
        }
      }
      if (!changed) break;
    }
  }
  // local memory budget for V registers
  const uint32_t per_slot = static_cast<uint32_t>(u_) * 16u * prog_->threads;
  const uint32_t budget = g_system.lds_per_wg > 80 * 1024 ? 72 * 1024 : g_system.lds_per_wg - 8 * 1024;
  vslot_limit_ = std::min<int>(DVM_VEC_NREG, static_cast<int>(budget / per_slot));
  sreg_used_ = vslot_used_ = 0;
  max_vslot_ = 0;
  acc_node_ = -1;
  n_held_ = 0;  // (a compile that failed half-way may have left entries behind)
  code_.clear();
  n_mem_ = 0;
  for (int s = 0; s < n_sec_; ++s) EmitSection(s);
  Emit(VOP_END, 0, 0, 0, 0, 0);
}
void Compiler::FinishProgram() {
  {
    uint32_t dts[DVM_VEC_MAXMEM];
    for (int i = 0; i < n_mem_; ++i) dts[i] = mems_[i].dtype;
    DropCastBeforeStore(dts);
  }
  DropUnreadSRegStores();
  // tuning switches: DVM_VEC_FUSE=0 keeps the instruction stream as emitted, DVM_VEC_UNIRUN=0 lets every wave
  // execute the per-team runs
  if (k_->tuning_.vec_fuse != 0 && (hdr_.sched & VS_KIND_MASK) != VS_POINTWISE) FuseSweepInstructions();
  if (k_->tuning_.vec_unirun != 0) MarkUniformRuns();
  if (k_->tuning_.vec_pair != 0) PairLoads();
  if (k_->tuning_.vec_sweeps != 0 && FitsSweepBuild()) hdr_.sched |= VS_SWEEPS;
  hdr_.n_mem = n_mem_;
  hdr_.n_code = static_cast<uint32_t>(code_.size());
  hdr_.mem_off = sizeof(VVecHeader) / 8;
  hdr_.code_off = hdr_.mem_off + n_mem_ * (sizeof(VMemDesc) / 8);
  hdr_.n_vslot = max_vslot_;
  if (hdr_.code_off + code_.size() > DVM_PARAM_WORDS) Fail("program larger than 4 KB");
  std::memset(&prog_->blob, 0, sizeof(VmParam));
  std::memcpy(prog_->blob.w, &hdr_, sizeof(hdr_));
  std::memcpy(prog_->blob.w + hdr_.mem_off, mems_, sizeof(VMemDesc) * n_mem_);
  std::memcpy(prog_->blob.w + hdr_.code_off, code_.data(), 8 * code_.size());
  prog_->lds_bytes = DVM_VEC_RED_SCRATCH_DOUBLES(hdr_.sched, prog_->threads) * 8 + static_cast<uint32_t>(max_vslot_) * u_ * 16 * prog_->threads;
  PlanRereads();
  uint64_t gt = (static_cast<uint64_t>(std::min<uint32_t>(hdr_.n_items, g_system.core_num * 4)) << 32) | prog_->threads;
  if (g_system.HasDevice()) {
    gt = g_system.Api().select_block_thread(hdr_.sched, hdr_.n_items, prog_->threads, prog_->lds_bytes);
  }
  prog_->grid = static_cast<uint32_t>(gt >> 32);
  if (prog_->grid == 0) prog_->grid = 1;
}

void Compiler::CompileArea(int a) {
  cur_area_ = a;
  k_->programs_.emplace_back();
  prog_ = &k_->programs_.back();
  cube_mode_ = false;
  if (areas_[a].attn >= 0) {
    CompileAttn(areas_[a].attn);
    return;
  }
  if (areas_[a].cube) {
    CompileCube(a);
    return;
  }
  BuildNodes(a);
  if (nn_ == 0) {  // only stores that other launches have already served
    prog_->skip = true;
    return;
  }
  // an empty domain: nothing to run, outputs that still have elements are zero-filled
  bool empty = false;
  for (int i = 0; i < nn_; ++i) {
    int64_t n = 1;
    for (int d = 0; d < nodes_[i].rank; ++d) n *= nodes_[i].dims[d];
    if (n == 0) empty = true;
  }
  if (empty) {
    prog_->skip = true;
    for (int i = 0; i < nn_; ++i) {
      const ANode &n = nodes_[i];
      if (n.kind != AK_OUT) continue;
      int64_t cnt = 1;
      for (int d = 0; d < n.rank; ++d) cnt *= n.dims[d];
      if (cnt == 0) continue;
      Program::Fill f;
      f.op_id = n.addr_op;
      f.ws_slot = n.ws_slot;
      f.value = 0;
      f.bytes = (static_cast<size_t>(cnt) * DTypeSize(n.dtype) + 3) & ~static_cast<size_t>(3);
      prog_->fills.push_back(f);
    }
    return;
  }
  UnifyAxes();
  OrderAndMerge();
  ChooseSchedule();
  // a stored value must span the index space it is stored from, or it would be written several times. (The axis
  // that numbers the parts of a shared reduce is the exception: a value stored inside the sweep over the reduced space
  // lies in exactly one part, as every element of the reduce's input does.)
  int parts_axis = -1;
  for (int i = 0; i < nn_; ++i)
    if (nodes_[i].kind == AK_REDUCE && nodes_[i].op->part_split != 0 && nodes_[i].axis[0] >= 0) parts_axis = nodes_[i].axis[0];
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.kind != AK_OUT) continue;
    uint32_t have = 0;
    bool fd = false;
    for (int d = 0; d < n.rank; ++d) {
      if (n.axis[d] < 0) continue;
      have |= 1u << n.axis[d];
      if (axes_[n.axis[d]].reduced) fd = true;
    }
    bool all_reduced = true;  // (does the value have every reduced axis? then it is stored once per element of the reduced space)
    for (int ax = 0; ax < n_axes_; ++ax)
      if (axes_[ax].reduced && !((have >> ax) & 1u)) all_reduced = false;
    for (int ax = 0; ax < n_axes_; ++ax) {
      if ((have >> ax) & 1u) continue;
      if (ax == parts_axis && fd && all_reduced) continue;
      if (!axes_[ax].reduced || fd) Fail("output smaller than the kernel domain");
    }
  }
  EmitProgram();
  FinishProgram();
  if (n_peel_ > 0) ReplicatePeeled();
}

// One copy of the finished program per index of the peeled dims; patches are in operand order, one per VMemDesc.
void Compiler::ReplicatePeeled() {
  int64_t count = 1;
  for (int i = 0; i < n_peel_; ++i) count *= dims_[peel_dim_[i]].extent;
  if (count > 4096) Fail("too many kept dims");
  const Program base = *prog_;
  k_->programs_.pop_back();
  for (int64_t c = 0; c < count; ++c) {
    k_->programs_.push_back(base);
    Program &p = k_->programs_.back();
    if (c > 0) p.fills.clear();
    int64_t rest = c;
    for (int i = 0; i < n_peel_; ++i) {
      const int64_t ext = dims_[peel_dim_[i]].extent;
      const int64_t idx = rest % ext;
      rest /= ext;
      for (size_t m = 0; m < p.patches.size(); ++m) {
        p.patches[m].byte_offset += idx * peel_stride_[m][i];
      }
    }
  }
  prog_ = &k_->programs_.back();
}
}  // namespace dvm
