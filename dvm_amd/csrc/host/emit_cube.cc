// Matmul sub-kernels: tile choice, operand descriptors, the epilogue program.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "compiler.h"

namespace dvm {

// ---------- matmul sub-kernels ----------
//
// The matmul's operands are read from memory by the MFMA tile loop; every other operator of the
// sub-kernel has the matmul's output shape and becomes the epilogue program, emitted with the same
// accumulator-machine rules as a pointwise kernel whose accumulator starts out holding the product.

int Compiler::CubeMemIndex(int v) {
  ANode &n = nodes_[v];
  if (n_mem_ >= DVM_CUBE_MAXMEM) Fail("too many memory operands in a matmul epilogue");
  VCubeMem &m = cmems_[n_mem_];
  std::memset(&m, 0, sizeof(m));
  m.dtype = MemDType(n.dtype);
  const int R = cube_out_->rank();
  int64_t stride = 1;
  if (v == gmm_bias_node_) {
    // the bias of a grouped product is [groups, n]: one row per group, and the groups are the kernel's inner batch axis
    if (n.view != nullptr || n.rank != 2) Fail("the bias of a grouped matmul must be a dense [groups, n] tensor");
    m.stride_n = 1;
    m.stride_b1 = static_cast<uint32_t>(n.dims[1]);
  }
  for (int d = n.rank - 1; d >= 0 && v != gmm_bias_node_; --d) {
    const int od = d + R - n.rank;
    if (n.dims[d] != 1) {
      if (od < 0 || n.dims[d] != cube_out_->dim(od)) Fail("epilogue operand does not broadcast to the matmul result");
      const int64_t walk = n.view != nullptr ? n.view->vstride_[d] : stride;
      if (walk >= (1ll << 32) || walk < 0) Fail("stride above 2^32");
      const uint32_t st = static_cast<uint32_t>(walk);
      if (od == R - 1 && st != 1) Throw("DVM EXCEPTION. reason: a strided view whose innermost stride is not 1 is not supported by the gfx950 backend");
      if (od == R - 1) m.stride_n = st;
      else if (od == R - 2) m.stride_m = st;
      else if (od == R - 3) m.stride_b1 = st;
      else m.stride_b0 = st;
    }
    stride *= n.dims[d];
  }
  Program::Patch p;
  p.word = static_cast<uint32_t>(sizeof(VCubeHeader) / 8 + n_mem_ * (sizeof(VCubeMem) / 8));
  p.op_id = n.addr_op;
  p.ws_slot = n.ws_slot;
  p.byte_offset = n.view != nullptr ? n.view->view_base_ * static_cast<int64_t>(DTypeSize(n.dtype)) : 0;
  p.role = Program::kPatchPlain;
  prog_->patches.push_back(p);
  n.mem_idx = n_mem_++;
  return n.mem_idx;
}

// The epilogue interpreter pays a fixed price per instruction and walk (decode, a serial chain of a few hundred
// cycles with one wave per SIMD), so pairs that one arm can compute are joined: a multiply by a constant followed
// by Exp becomes VU_EXP_SCALED (exp(-x), exp(x * c)); the product is still rounded to fp32 on its own.
// Then, when every store writes a 16-bit float and every operator is continuous in its inputs (no compare,
// select, rounding to an integer, conversion to int32, so that an error of one fp32 ulp cannot flip a decision),
// exp, log, sqrt and the divisions are replaced by their hardware approximations and the header says so.
uint32_t Compiler::FuseCubeEpilogue() {
  std::vector<uint64_t> &out = scratch_code_;
  out.clear();
  out.reserve(code_.size());
  for (size_t i = 0; i < code_.size(); ++i) {
    const uint64_t w = code_[i];
    if (i + 1 < code_.size() && VI_OP(w) == VOP_BINF && VI_SUB(w) == VB_MUL && VI_KIND(w) == VK_IMM && VI_RND(w) == 0) {
      const uint64_t nx = code_[i + 1];
      if (VI_OP(nx) == VOP_UN && VI_SUB(nx) == VU_EXP) {
        out.push_back(VI_MAKE(VOP_UN, VU_EXP_SCALED, 0, VI_RND(nx), 0, VI_IMM(w)));
        ++i;
        continue;
      }
    }
    out.push_back(w);
  }
  code_.swap(out);
  if (k_->tuning_.cube_exact == 1) return 0;
  bool any = false;
  for (uint64_t w : code_) {
    switch (VI_OP(w)) {
      case VOP_END:
      case VOP_LD:
      case VOP_LDR:
      case VOP_LDI:
      case VOP_STR:
        break;
      case VOP_ST: {
        const uint32_t dt = cmems_[VI_A(w)].dtype;
        if (dt != VDT_F16 && dt != VDT_BF16) return 0;
        break;
      }
      case VOP_CAST:
        if (VI_SUB(w) != VC_RND) return 0;
        break;
      case VOP_UN: {
        const uint32_t u = VI_SUB(w);
        if (u != VU_SQRT && u != VU_ABS && u != VU_LOG && u != VU_EXP && u != VU_EXP_SCALED) return 0;
        if (u != VU_ABS) any = true;
        break;
      }
      case VOP_BINF: {
        const uint32_t b = VI_SUB(w);
        if (b != VB_ADD && b != VB_SUB && b != VB_RSUB && b != VB_MUL && b != VB_DIV && b != VB_RDIV && b != VB_MIN && b != VB_MAX) return 0;
        if (b == VB_DIV || b == VB_RDIV) any = true;
        break;
      }
      default:
        return 0;
    }
  }
  if (!any) return 0;
  for (uint64_t &w : code_) {
    uint32_t sub = VI_SUB(w);
    if (VI_OP(w) == VOP_UN) {
      sub = sub == VU_EXP ? VU_EXP_APPROX : sub == VU_EXP_SCALED ? VU_EXP_SCALED_APPROX : sub == VU_LOG ? VU_LOG_APPROX : sub == VU_SQRT ? VU_SQRT_APPROX : sub;
    } else if (VI_OP(w) == VOP_BINF) {
      sub = sub == VB_DIV ? VB_DIV_APPROX : sub == VB_RDIV ? VB_RDIV_APPROX : sub;
    } else {
      continue;
    }
    w = (w & ~0xff00ull) | (static_cast<uint64_t>(sub) << 8);
  }
  // x / (exp(x * c) + 1) and 1 / (exp(x * c) + 1), all in fp32: one dispatch instead of four / three (SiLU, sigmoid)
  if (k_->tuning_.cube_fuse_act != 0) {
    std::vector<uint64_t> &out2 = scratch_code_;
    out2.clear();
    auto is_exp = [](uint64_t w) { return VI_OP(w) == VOP_UN && VI_SUB(w) == VU_EXP_SCALED_APPROX && VI_RND(w) == 0; };
    auto is_add1 = [](uint64_t w) { return VI_OP(w) == VOP_BINF && VI_SUB(w) == VB_ADD && VI_KIND(w) == VK_IMM && VI_RND(w) == 0 && VI_IMM(w) == 0x3f800000u; };
    for (size_t i = 0; i < code_.size(); ++i) {
      const uint64_t w = code_[i];
      if (i + 3 < code_.size() && VI_OP(w) == VOP_STR && is_exp(code_[i + 1]) && is_add1(code_[i + 2])) {
        const uint64_t d = code_[i + 3];
        // the parked value must not be read again later (it is only this division's numerator)
        bool reread = false;
        for (size_t j = i + 4; j < code_.size() && !reread; ++j) {
          const uint64_t v = code_[j];
          if (VI_OP(v) == VOP_STR && VI_A(v) == VI_A(w)) break;
          if ((VI_OP(v) == VOP_LDR || (VI_OP(v) >= VOP_SRC_BASE && VI_KIND(v) == VK_REG)) && VI_A(v) == VI_A(w)) reread = true;
        }
        if (!reread && VI_OP(d) == VOP_BINF && VI_SUB(d) == VB_RDIV_APPROX && VI_KIND(d) == VK_REG && VI_A(d) == VI_A(w) && VI_RND(d) == 0) {
          out2.push_back(VI_MAKE(VOP_UN, VU_SILU_APPROX, 0, 0, 0, VI_IMM(code_[i + 1])));
          i += 3;
          continue;
        }
      }
      if (i + 2 < code_.size() && is_exp(w) && is_add1(code_[i + 1])) {
        const uint64_t d = code_[i + 2];
        if (VI_OP(d) == VOP_BINF && VI_SUB(d) == VB_RDIV_APPROX && VI_KIND(d) == VK_IMM && VI_RND(d) == 0 && VI_IMM(d) == 0x3f800000u) {
          out2.push_back(VI_MAKE(VOP_UN, VU_SIGMOID_APPROX, 0, 0, 0, VI_IMM(w)));
          i += 2;
          continue;
        }
      }
      out2.push_back(w);
    }
    code_.swap(out2);
  }
  return VCF_APPROX_MATH;
}

void Compiler::CompileCube(int a) {
  cube_mode_ = true;
  BuildNodes(a);
  int c = -1;
  for (int i = 0; i < nn_; ++i)
    if (nodes_[i].kind == AK_OP && nodes_[i].op->kind == kObjMatMul) c = i;
  if (c < 0) Fail("matmul sub-kernel without a matmul");
  NDObject *mm = nodes_[c].op;
  cube_out_ = mm;
  const ANode &an = nodes_[nodes_[c].in[0]], &bn = nodes_[nodes_[c].in[1]];
  if (an.kind != AK_MEM || bn.kind != AK_MEM) Fail("matmul operands must come from memory");
  if (an.dtype != bn.dtype || (an.dtype != kFloat16 && an.dtype != kBFloat16)) Fail("matmul operands must both be fp16 or both bf16");
  const int R = mm->rank();
  const int br = R - 2;
  if (br > 2) Fail("matmul with more than two batch dimensions");
  const int gmm = mm->gmm_type;  // 0: a plain product; 1: groups of rows; 2: groups along k
  gmm_bias_node_ = -1;
  VCubeHeader h;
  std::memset(&h, 0, sizeof(h));
  h.entry = VE_CUBE;
  h.dtype = MemDType(an.dtype);
  const int64_t M = mm->dim(R - 2), N = mm->dim(R - 1);
  const int64_t K = mm->trans_a ? an.dims[an.rank - 2] : an.dims[an.rank - 1];
  if (M >= (1ll << 31) || N >= (1ll << 31) || K >= (1ll << 31)) Fail("matmul extent above 2^31");
  h.m = static_cast<uint32_t>(M);
  h.n = static_cast<uint32_t>(N);
  h.k = static_cast<uint32_t>(K);
  h.nb0 = br == 2 ? static_cast<uint32_t>(mm->dim(0)) : 1;
  h.nb1 = br >= 1 ? static_cast<uint32_t>(mm->dim(br - 1)) : 1;
  if (gmm != 0) {
    // the groups are the inner batch axis: matrix g of B with the rows of group g (the output has no batch axis
    // then), or the k range of group g into matrix g of the output
    const int64_t groups = mm->group_list->dim(0);
    if (groups > static_cast<int64_t>(DVM_CUBE_MAX_GROUPS)) Throw("DVM EXCEPTION. reason: a grouped matmul of more than 2048 groups is not supported by the gfx950 backend");
    h.nb0 = 1;
    h.nb1 = static_cast<uint32_t>(groups);
    h.group_mode = gmm == 1 ? (mm->gmm_sizes ? VCG_M_SIZE : VCG_M_BOUND) : (mm->gmm_sizes ? VCG_K_SIZE : VCG_K_BOUND);
    h.group_i32 = mm->group_list->type_id_ == kInt32 ? 1 : 0;
  }
  // An operand is a matrix (or a batch of matrices) walked through a leading dimension and up to two batch strides.
  // A dense tensor gives those from its shape; a strided view (a load with strides, a slice, a permute of a stored
  // value: a sliced weight, the heads-first view of a [batch, seq, heads, dim] tensor, a transposed K) gives them
  // from its element strides: with the innermost stride 1 the matrix is read as it lies, with the second-innermost
  // stride 1 it is the transpose of what lies in memory and the operand's transpose flag flips. Nothing is copied.
  // (The reference reads views into its cube unit as well: include/dvm.h:434-479, src/isa.h:1187-1452.)
  auto operand_layout = [&](const ANode &x, bool *flip, uint32_t *ld, uint32_t *s0, uint32_t *s1) {
    *flip = false;
    *s0 = *s1 = 0;
    const int r = x.rank;
    int64_t walk[kMaxAxes];
    int64_t stride = 1;
    for (int d = r - 1; d >= 0; --d) {
      walk[d] = x.view != nullptr ? x.view->vstride_[d] : stride;
      stride *= x.dims[d];
    }
    for (int d = 0; d < r; ++d)
      if (x.dims[d] != 1 && (walk[d] < 0 || walk[d] >= (1ll << 32))) Fail("stride above 2^32");
    const int64_t rows = x.dims[r - 2], cols = x.dims[r - 1];
    if (cols == 1 || walk[r - 1] == 1) {
      *ld = static_cast<uint32_t>(rows == 1 ? std::max<int64_t>(cols, 1) : walk[r - 2]);
    } else if (rows == 1 || walk[r - 2] == 1) {
      *flip = true;
      *ld = static_cast<uint32_t>(cols == 1 ? std::max<int64_t>(rows, 1) : walk[r - 1]);
    } else {
      Throw("DVM EXCEPTION. reason: a matmul operand view with no contiguous axis is not supported by the gfx950 backend (Copy it first)");
    }
    if (*ld == 0) Throw("DVM EXCEPTION. reason: a matmul operand view that repeats its rows is not supported by the gfx950 backend (Copy it first)");
    for (int d = r - 3; d >= 0; --d) {
      const int od = d + R - r;
      if (x.dims[d] == 1) continue;
      if (od == R - 3) *s1 = static_cast<uint32_t>(walk[d]);
      else *s0 = static_cast<uint32_t>(walk[d]);
    }
  };
  if (M == 0 || N == 0 || h.nb0 == 0 || h.nb1 == 0) {  // an empty result: nothing to launch
    prog_->skip = true;
    return;
  }
  if (K == 0 && gmm == 0) {
    Throw("DVM EXCEPTION. reason: a matmul over an empty k axis is not supported by the gfx950 backend (its result is the bias alone)");
  }
  bool flip_a = false, flip_b = false;
  operand_layout(an, &flip_a, &h.lda, &h.a_sb0, &h.a_sb1);
  operand_layout(bn, &flip_b, &h.ldb, &h.b_sb0, &h.b_sb1);
  if (gmm == 1) {  // matrix g of B: its outermost dim, whatever the rank of the output
    int64_t walk = bn.view != nullptr ? bn.view->vstride_[0] : bn.dims[1] * bn.dims[2];
    if (walk < 0 || walk >= (1ll << 32)) Fail("stride above 2^32");
    h.b_sb0 = 0;
    h.b_sb1 = static_cast<uint32_t>(walk);
    h.a_sb0 = h.a_sb1 = 0;
  }
  const bool trans_a = mm->trans_a != flip_a, trans_b = mm->trans_b != flip_b;  // as the operands lie in memory
  h.trans_a = trans_a ? 1 : 0;
  h.trans_b = trans_b ? 1 : 0;
  // A measured choice of tile and split for this product shape (the online tuner, host/tuner.cc) stands in for the
  // two tuning switches for the rest of this function; a switch the user has set wins.
  struct RestoreTuning {
    Tuning &t;
    const int tile, split;
    ~RestoreTuning() {
      t.cube_tile = tile;
      t.cube_splitk = split;
    }
  } restore_tuning{k_->tuning_, k_->tuning_.cube_tile, k_->tuning_.cube_splitk};
  if (!k_->tuning_.in_tuner && k_->tuning_.cube_tile < 0 && k_->tuning_.cube_splitk < 0 && K > 0 && gmm == 0) {
    CubeProblem q;
    q.m = M;
    q.n = N;
    q.k = K;
    q.nb0 = h.nb0;
    q.nb1 = h.nb1;
    q.dtype = mm->type_id_;
    q.trans_a = trans_a;
    q.trans_b = trans_b;
    CubeChoice c;
    if (CubeTunerLookup(q, &c)) {
      k_->tuning_.cube_tile = c.tile;
      k_->tuning_.cube_splitk = c.split <= 1 ? 0 : c.split;
    }
  }
  // block tile: the largest that still gives most compute units a tile
  // (groups of rows: a tile is computed once per group that owns rows of it, so about once: the groups do not multiply the work)
  const uint64_t batch = gmm == 1 ? 1 : static_cast<uint64_t>(h.nb0) * h.nb1;
  auto tiles = [&](int64_t t) { return static_cast<uint64_t>((M + t - 1) / t) * static_cast<uint64_t>((N + t - 1) / t) * batch; };
  const uint64_t cus = g_system.core_num;
  int64_t bt;
  if (tiles(256) * 4 >= cus * 3) {
    h.tile = 0;
    bt = 256;
  } else if (tiles(128) * 2 >= cus) {
    h.tile = 1;
    bt = 128;
  } else {
    h.tile = 2;
    bt = 64;
  }
  // ... unless most of such a tile would lie outside the output (batches of small matrices, an output narrower than
  // the tile): a tile half the size that covers half the area or less wins. Measured on MI355X, fp16 P x V of an
  // unfused attention, [128,1024,1024] x [128,1024,64]: 299 us on the 256 tile, 416 on 128, 88 on 64;
  // [256,2048,2048] x [256,2048,128]: 1976 / 858 / 1186 us; [64,512,512] x [64,512,32]: 82 / 56 / 31 us.
  {
    auto padded = [&](int64_t t) { return static_cast<double>(tiles(t)) * static_cast<double>(t * t); };
    while (bt > 64 && padded(bt) >= 2.0 * padded(bt / 2)) {
      bt /= 2;
      ++h.tile;
    }
  }
  {  // tuning override: 256, 128 or 64
    const int v = k_->tuning_.cube_tile;
    if (v == 256 || v == 128 || v == 64) {
      bt = v;
      h.tile = v == 256 ? 0 : (v == 128 ? 1 : 2);
    }
  }
  // The 256x256 tile runs on eight waves (two per SIMD, 64x128 accumulators each) unless DVM_CUBE_WAVES=4 asks for
  // four (one per SIMD, 128x128): the second wave of a SIMD fills the stalls of the first in the prologue and in
  // the interpreted epilogue. Measured on MI355X, bf16 8192x4096xk, row-major operands, four -> eight waves:
  // k = 64: 60 -> 54 us (with bias + SiLU 106 -> 87 us), k = 512: 82 -> 76 us, k = 4096: 296-301 us either way for
  // the plain product (the sustained rate is set by the power cap there), 338-342 -> 334-339 us with bias + SiLU.
  // Split k: with fewer tiles than compute units and a long k axis, k_split workgroups share a tile's k axis and a
  // second launch adds their fp32 partial tiles in a fixed order and runs the epilogue (the reference splits k into
  // consecutive matmuls accumulating in fp32 when the operands exceed its L2, src/ops_m.cc:240-264,
  // src/xkernel.cc:1511-1547; here the reason is to fill the chip). Every candidate (tile, parts) gets an estimate
  // from figures measured on MI355X (bf16, microseconds): a workgroup's time per 64 k (2.2 for the 256 tile, 1.3 for
  // 128, 0.71 for 64 alone on its compute unit and 0.9 when two share one; the guarded path of ragged or unaligned
  // tiles takes about two and a half times as long), rounds of workgroups over the chip, and for a split the second launch plus
  // the time its one workgroup per tile needs per partial tile (3.2 / 0.8 / 0.2 with the vectors of several parts in
  // flight together: a single workgroup streams at some 80 GB/s), which is what keeps deep splits of big tiles from
  // paying, plus the time the first launch takes to write the partial tiles (some 4 TB/s over the whole chip).
  uint32_t k_split = 1, k_chunk = 0;
  {
    const int forced = gmm != 0 ? 0 : k_->tuning_.cube_splitk;  // (the k axis of a grouped product is never shared)
    const bool user_tile = k_->tuning_.cube_tile == 256 || k_->tuning_.cube_tile == 128 || k_->tuning_.cube_tile == 64;
    auto parts_of = [&](uint32_t want, uint32_t *chunk) -> uint32_t {  // parts actually made when `want` are asked for
      if (want < 2 || K < 128) return 1;
      const int64_t c = ((K + want - 1) / want + 63) / 64 * 64;
      *chunk = static_cast<uint32_t>(c);
      return static_cast<uint32_t>((K + c - 1) / c);
    };
    if (forced >= 2) {
      k_split = parts_of(static_cast<uint32_t>(forced), &k_chunk);
    } else if (forced != 0 && forced != 1) {
      static const int64_t kTiles[3] = {256, 128, 64};
      static const double kStepUs[3] = {2.2, 1.3, 0.71}, kPartUs[3] = {3.2, 0.8, 0.2};
      const bool aligned = K % 64 == 0 && h.lda % 8 == 0 && h.ldb % 8 == 0;
      double best = 0.0;
      int best_tile = -1;
      uint32_t best_split = 1, best_chunk = 0;
      for (int ti = 0; ti < 3; ++ti) {
        const int64_t t = kTiles[ti];
        if (user_tile && t != bt) continue;
        const uint64_t nt = tiles(t);
        const uint64_t slots = ti == 2 ? 2 * cus : cus;  // two 64x64 workgroups fit a compute unit
        const uint32_t max_split = nt >= slots ? 1u : static_cast<uint32_t>(std::min<uint64_t>(slots / nt, 32));
        // (ragged edge tiles of an aligned product are moved back inside the output and stay on the vector path)
        // (and the 64 tile fetches the rows of a short operand with contiguous k through clamped addresses)
        const bool m_fast = M % t == 0 || (M >= t && (!trans_a || M % 8 == 0)) || (t == 64 && !trans_a);
        const bool n_fast = N % t == 0 || (N >= t && N % 8 == 0) || (t == 64 && trans_b);
        const double slow = (aligned && m_fast && n_fast) ? 1.0 : 2.5;
        for (uint32_t want = 1; want <= max_split; want = want < 2 ? 2 : want * 2) {
          uint32_t chunk = 0;
          const uint32_t parts = parts_of(want, &chunk);
          if (want > 1 && (parts < 2 || chunk < 256)) break;
          const double steps = (parts > 1 ? static_cast<double>(chunk) : static_cast<double>(K)) / 64.0;
          const uint64_t wgs = nt * parts;
          const double rounds = std::ceil(static_cast<double>(wgs) / static_cast<double>(slots));
          const double step_us = (ti == 2 && wgs > cus) ? 0.9 : kStepUs[ti];
          double us = rounds * steps * step_us * slow + 3.0;
          if (parts > 1) us += 5.0 + parts * kPartUs[ti] + static_cast<double>(wgs) * static_cast<double>(t * t) * 4.0 / 4.0e6;
          if (parts > 1 && static_cast<double>(wgs) * static_cast<double>(t * t) * 4.0 > 512.0 * 1024 * 1024) continue;
          if (best_tile < 0 || us < best) {
            best = us;
            best_tile = ti;
            best_split = parts;
            best_chunk = chunk;
          }
        }
      }
      // without a split the tile stays the one chosen above
      if (best_tile >= 0 && best_split > 1) {
        bt = kTiles[best_tile];
        h.tile = static_cast<uint32_t>(best_tile);
        k_split = best_split;
        k_chunk = best_chunk;
      }
    }
  }
  if (h.tile == 0 && k_->tuning_.cube_waves != 4) h.tile = 3;
  h.tiles_m = static_cast<uint32_t>((M + bt - 1) / bt);
  h.tiles_n = static_cast<uint32_t>((N + bt - 1) / bt);
  if (tiles(bt) * (gmm == 1 ? h.nb1 : 1) >= (1ull << 31)) Fail("too many matmul tiles");
  // (groups along k: every group's range decides for itself on the device whether it is whole 64-steps from an aligned start)
  h.fast = ((K % 64 == 0 || gmm == 2) && K > 0 && h.lda < (1u << 22) && h.ldb < (1u << 22) && h.lda % 8 == 0 && h.ldb % 8 == 0 && h.a_sb0 % 8 == 0 &&
            h.a_sb1 % 8 == 0 && h.b_sb0 % 8 == 0 && h.b_sb1 % 8 == 0)
               ? 1
               : 0;
  // operand addresses
  for (int which = 0; which < 2; ++which) {
    const ANode &x = which == 0 ? an : bn;
    Program::Patch p;
    p.word = static_cast<uint32_t>((which == 0 ? offsetof(VCubeHeader, a_addr) : offsetof(VCubeHeader, b_addr)) / 8);
    p.op_id = x.addr_op;
    p.ws_slot = x.ws_slot;
    p.byte_offset = x.view != nullptr ? x.view->view_base_ * static_cast<int64_t>(DTypeSize(x.dtype)) : 0;
    p.role = Program::kPatchCubeOperand;
    prog_->patches.push_back(p);
  }
  if (gmm != 0) {
    Program::Patch p;
    p.word = static_cast<uint32_t>(offsetof(VCubeHeader, group_addr) / 8);
    p.op_id = mm->group_list->id;
    p.ws_slot = -1;
    p.role = Program::kPatchPlain;
    prog_->patches.push_back(p);
  }
  // the epilogue: one section over values that all live in fragments
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    n.has_inner = true;
    n.fd = false;
    n.sec = 0;
    n.last_sec = 0;
    n.level = 0;
    n.uses = 0;
    n.in_cone = false;
  }
  // the tile loop reads A and B itself: they are no values of the epilogue
  const int bias = nodes_[c].nin > 2 ? nodes_[c].in[2] : -1;
  if (bias >= 0 && nodes_[bias].kind != AK_MEM) Fail("matmul bias must come from memory");
  if (gmm != 0) gmm_bias_node_ = bias;
  nodes_[c].nin = 0;
  nr_ = 0;
  n_sec_ = 1;
  cur_sec_ = 0;
  single_round_ = true;
  vslot_limit_ = DVM_CUBE_NTEMP;
  sreg_used_ = vslot_used_ = 0;
  max_vslot_ = 0;
  n_held_ = 0;
  code_.clear();
  n_mem_ = 0;
  // the bias row joins the fp32 accumulators, which are then rounded once to the operand type: that
  // is the matmul's value (src/vm_aic.cce:34-470)
  if (bias >= 0) Emit(VOP_BINF, VB_ADD, VK_MEM, 0, MemIndex(bias), 0);
  Emit(VOP_CAST, VC_RND, 0, RndOf(mm->type_id_), 0, 0);
  acc_node_ = c;
  int sinks[kMaxNodes];
  int ns = 0;
  for (int i = 0; i < nn_; ++i)
    if (nodes_[i].kind == AK_OUT) sinks[ns++] = i;
  for (int i = 0; i < ns; ++i) CountCone(nodes_[sinks[i]].in[0]);
  for (int i = 0; i < ns; ++i) {
    const int x = Resolve(nodes_[sinks[i]].in[0]);
    EmitValue(x);
    Emit(VOP_ST, 0, 0, 0, MemIndex(sinks[i]), 0);
    ConsumeUse(x);
  }
  Emit(VOP_END, 0, 0, 0, 0, 0);
  {
    uint32_t dts[DVM_CUBE_MAXMEM];
    for (int i = 0; i < n_mem_; ++i) dts[i] = cmems_[i].dtype;
    DropCastBeforeStore(dts);
  }
  h.epi_flags = FuseCubeEpilogue();
  {  // the slim pass takes programs of activation-like epilogues
    bool slim = true;
    for (uint64_t w : code_) {
      const uint32_t sub = VI_SUB(w);
      switch (VI_OP(w)) {
        case VOP_END:
        case VOP_LD:
        case VOP_LDI:
        case VOP_ST:
          break;
        case VOP_LDR:
        case VOP_STR:
          if (VI_A(w) != 0) slim = false;
          break;
        case VOP_CAST:
          if (sub != VC_RND) slim = false;
          break;
        case VOP_UN:
          if (sub != VU_ABS && sub != VU_EXP_APPROX && sub != VU_EXP_SCALED_APPROX && sub != VU_LOG_APPROX && sub != VU_SQRT_APPROX &&
              sub != VU_SILU_APPROX && sub != VU_SIGMOID_APPROX) slim = false;
          break;
        case VOP_BINF: {
          const uint32_t b = sub & 0x3fu;
          if (b != VB_ADD && b != VB_SUB && b != VB_RSUB && b != VB_MUL && b != VB_DIV && b != VB_RDIV && b != VB_DIV_APPROX &&
              b != VB_RDIV_APPROX && b != VB_MIN && b != VB_MAX) slim = false;
          if (VI_KIND(w) == VK_REG && VI_A(w) != 0) slim = false;
          break;
        }
        default:
          slim = false;
          break;
      }
    }
    if (slim && k_->tuning_.cube_exact != 2) h.epi_flags |= VCF_SLIM;
  }
  {  // [Add mem] [cast.round] store end: done natively by the kernel
    size_t i = 0;
    if (i < code_.size() && VI_OP(code_[i]) == VOP_BINF && VI_SUB(code_[i]) == VB_ADD && VI_KIND(code_[i]) == VK_MEM && VI_RND(code_[i]) == 0) ++i;
    if (i < code_.size() && VI_OP(code_[i]) == VOP_CAST && VI_SUB(code_[i]) == VC_RND) ++i;
    if (i + 2 == code_.size() && VI_OP(code_[i]) == VOP_ST && VI_OP(code_[i + 1]) == VOP_END && k_->tuning_.cube_exact != 2) h.epi_flags |= VCF_PLAIN_STORE;
  }
  {  // [Add of a bias row] cast.round to the operand type in front: the kernel does them where the accumulators are
    size_t i = 0;
    bool ok = k_->tuning_.cube_dump16 != 0;
    if (i < code_.size() && VI_OP(code_[i]) == VOP_BINF) {
      const uint64_t w = code_[i];
      ok = ok && VI_SUB(w) == VB_ADD && VI_KIND(w) == VK_MEM && VI_RND(w) == 0 && VI_A(w) < static_cast<uint32_t>(n_mem_);
      if (ok) {
        const VCubeMem &b = cmems_[VI_A(w)];
        ok = b.stride_n == 1 && b.stride_m == 0 && (b.dtype == VDT_F32 || b.dtype == VDT_F16 || b.dtype == VDT_BF16);
      }
      ++i;
    }
    // (the rounding is an instruction, or what the one store of the program does: it writes the operand type)
    const bool rounds = i < code_.size() && VI_OP(code_[i]) == VOP_CAST && VI_SUB(code_[i]) == VC_RND && VI_RND(code_[i]) == RndOf(mm->type_id_);
    const bool store_rounds = i + 2 == code_.size() && VI_OP(code_[i]) == VOP_ST && VI_OP(code_[i + 1]) == VOP_END &&
                              VI_A(code_[i]) < static_cast<uint32_t>(n_mem_) && cmems_[VI_A(code_[i])].dtype == MemDType(mm->type_id_);
    if (ok && (rounds || store_rounds)) h.epi_flags |= VCF_DUMP16;
  }
  h.n_mem = n_mem_;
  h.n_code = static_cast<uint32_t>(code_.size());
  h.mem_off = sizeof(VCubeHeader) / 8;
  h.code_off = h.mem_off + n_mem_ * (sizeof(VCubeMem) / 8);
  if (h.code_off + code_.size() > DVM_PARAM_WORDS) Fail("program larger than 4 KB");
  std::memset(&prog_->blob, 0, sizeof(VmParam));
  std::memcpy(prog_->blob.w, &h, sizeof(h));
  std::memcpy(prog_->blob.w + h.mem_off, cmems_, sizeof(VCubeMem) * n_mem_);
  std::memcpy(prog_->blob.w + h.code_off, code_.data(), 8 * code_.size());
  prog_->threads = h.tile == 3 ? 512 : 256;
  prog_->lds_bytes = DVM_CUBE_LDS_BYTES(static_cast<uint32_t>(bt)) + (gmm != 0 ? 8u * h.nb1 : 0u);
  prog_->grid = static_cast<uint32_t>(tiles(bt));
  if (gmm == 1) {
    // The work items are the tiles that have rows of a group to store, counted on the device from the list: at most
    // one row of tiles more per group than the matrix has (a tile a bound runs through is computed for both sides).
    // One workgroup per item that can exist; those past the count leave at once.
    const uint64_t rows_max = static_cast<uint64_t>(h.tiles_m) + std::min<uint64_t>(h.nb1, static_cast<uint64_t>(M));
    prog_->grid = static_cast<uint32_t>(std::min<uint64_t>(rows_max * h.tiles_n, 1u << 20));
  }
  // A short k axis (the scores of an attention, an outer product): a 256 tile is then mostly its start-up (program
  // and header into local memory) and its epilogue, and one workgroup per compute unit that walks the tiles pays the
  // start-up once. Measured on MI355X, fp16: [128,1024,64] x [128,1024,64]^T 148 -> 130 us, 8192 x 8192 x 128
  // 72 -> 64 us; at k = 512 and beyond it makes no difference.
  if (k_split <= 1 && bt == 256 && K <= 256 && prog_->grid > cus) prog_->grid = static_cast<uint32_t>(cus);
  if (k_split > 1) {
    // two launches of the same program: partial products per part of the k axis, then their sum and the epilogue
    const int slot = static_cast<int>(k_->ws_sizes_.size());
    k_->ws_sizes_.push_back(static_cast<size_t>(k_split) * tiles(bt) * static_cast<size_t>(bt * bt) * 4);
    Program::Patch pp;
    pp.word = static_cast<uint32_t>(offsetof(VCubeHeader, part_addr) / 8);
    pp.op_id = -1;
    pp.ws_slot = slot;
    pp.role = Program::kPatchPlain;
    prog_->patches.push_back(pp);
    VCubeHeader *ph = reinterpret_cast<VCubeHeader *>(prog_->blob.w);
    ph->k_split = k_split;
    ph->k_chunk = k_chunk;
    const uint32_t flags = ph->epi_flags;
    ph->epi_flags = flags | VCF_SPLITK_PARTIAL;
    prog_->grid = static_cast<uint32_t>(tiles(bt) * k_split);
    const Program first = *prog_;
    k_->programs_.push_back(first);
    prog_ = &k_->programs_.back();
    reinterpret_cast<VCubeHeader *>(prog_->blob.w)->epi_flags = flags | VCF_SPLITK_COMBINE;
    prog_->grid = static_cast<uint32_t>(tiles(bt));
    prog_->fills.clear();
  }
}
}  // namespace dvm
