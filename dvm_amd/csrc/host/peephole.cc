// Passes over the emitted instruction words of a vector program.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "compiler.h"

namespace dvm {

// A value is copied into an S register wherever a later round of a sweep may need it again; when every row fits one
// round nothing reads some of those registers (the maximum of a softmax row stays in the accumulator): the copies go.
// A dispatch each, of the 18 a row of such a softmax takes.
void Compiler::DropUnreadSRegStores() {
  uint32_t read = 0;
  for (uint64_t w : code_) {
    const uint32_t op = VI_OP(w);
    if (op == VOP_LDS) read |= 1u << VI_A(w);
    if (op >= VOP_SRC_BASE && (VI_KIND(w) == VK_SREG || VI_KIND(w) == VK_SREG2)) {
      read |= 1u << VI_A(w);
      if (VI_KIND(w) == VK_SREG2) read |= 1u << ((VI_IMM(w) >> 8) & 0xffu);
    }
  }
  std::vector<uint64_t> &out = scratch_code_;
  out.clear();
  out.reserve(code_.size());
  for (uint64_t w : code_) {
    if (VI_OP(w) == VOP_STS && VI_A(w) < 32 && !((read >> VI_A(w)) & 1u)) continue;
    out.push_back(w);
  }
  code_.swap(out);
}

// A rounding cast to fp16 / bf16 whose only reader is the store right behind it does nothing the store's own
// conversion does not do (same round to nearest even): the cast instruction is dropped. `mem_dtypes[i]` is the
// element type of memory operand i.
void Compiler::DropCastBeforeStore(const uint32_t *mem_dtypes) {
  std::vector<uint64_t> &out = scratch_code_;
  out.clear();
  out.reserve(code_.size());
  for (size_t i = 0; i < code_.size(); ++i) {
    const uint64_t w = code_[i];
    if (VI_OP(w) == VOP_CAST && VI_SUB(w) == VC_RND && !(static_cast<uint32_t>(w) & VI_UNIFORM) && i + 2 < code_.size() + 1 && i + 1 < code_.size()) {
      const uint64_t st = code_[i + 1];
      const uint32_t next = i + 2 < code_.size() ? VI_OP(code_[i + 2]) : static_cast<uint32_t>(VOP_END);
      const bool acc_dead = next == VOP_END || next == VOP_ENDSWEEP || next == VOP_SWEEP || next == VOP_LD || next == VOP_LDR ||
                            next == VOP_LDS || next == VOP_LDI || next == VOP_FIN;
      if (VI_OP(st) == VOP_ST && acc_dead) {
        const uint32_t dt = mem_dtypes[VI_A(st)];
        if ((VI_RND(w) == VRND_F16 && dt == VDT_F16) || (VI_RND(w) == VRND_BF16 && dt == VDT_BF16)) continue;
      }
    }
    out.push_back(w);
  }
  code_.swap(out);
}

// A load followed by a float binary whose memory operand walks memory identically (x + residual, x * mask): the
// load is told that it may take the binary along. The device then has both operands in flight together, one trip
// to memory for the pair instead of two in a row, which is what a wave with little else in flight waits for.
void Compiler::PairLoads() {
  bool in_run = false;
  for (size_t i = 0; i + 1 < code_.size(); ++i) {
    const uint64_t w = code_[i], nx = code_[i + 1];
    if (VI_OP(w) == VOP_UNI_BEGIN) in_run = true;
    if (VI_OP(w) == VOP_UNI_END) in_run = false;
    if (in_run || VI_OP(w) != VOP_LD || (static_cast<uint32_t>(w) & VI_UNIFORM)) continue;
    if (VI_OP(nx) != VOP_BINF || VI_KIND(nx) != VK_MEM || (VI_IMM(nx) & VI_PRE_SREG)) continue;  // (the paired path runs the binary alone)
    if (!(static_cast<uint32_t>(nx) & VI_SAME_OFFS) || (static_cast<uint32_t>(nx) & (VI_UNIFORM | VI_ENDS))) continue;
    code_[i] = w | VI_LD_PAIR;
  }
  // A sweep whose body is one load and one float reduce (the statistics sweep of a normalisation): the load may
  // fetch several rounds per trip and do the reduce itself.
  if ((hdr_.sched & VS_KIND_MASK) != VS_POINTWISE) {
    for (size_t i = 1; i + 1 < code_.size(); ++i) {
      const uint64_t w = code_[i], nx = code_[i + 1];
      if (VI_OP(code_[i - 1]) != VOP_SWEEP || VI_OP(w) != VOP_LD || (static_cast<uint32_t>(w) & (VI_UNIFORM | VI_LD_PAIR))) continue;
      if (VI_OP(nx) != VOP_RED || !(static_cast<uint32_t>(nx) & VI_ENDS) || (VI_SUB(nx) & VRF_INT)) continue;
      // The fused path leaves no particular round in the accumulator. What follows the sweep may read it (an
      // operand that does not vary along the reduced axes is taken from the last round instead of being loaded
      // again): then the load stays an ordinary one.
      bool acc_dead = false;
      for (size_t q = i + 2; q < code_.size(); ++q) {
        const uint32_t qop = VI_OP(code_[q]);
        if (qop == VOP_UNI_BEGIN || qop == VOP_SWEEP || qop == VOP_ENDSWEEP) continue;
        acc_dead = qop == VOP_END || qop == VOP_FIN || qop == VOP_LDS || qop == VOP_LDI || qop == VOP_LD;
        break;
      }
      if (!acc_dead) continue;
      code_[i] = w | VI_LD_RED2;
    }
  }
}

// The interpreter pays a fixed price per instruction, so the short bodies of sweeps are tightened:
//  * sum(x) and sum(x * x) of one value (mean and variance in one pass): the multiply joins the second reduce;
//  * two float binaries in a row with S-register operands (x * scale + shift) become one chained instruction;
//  * the VOP_ENDSWEEP behind a store or a reduce becomes a flag of that instruction.
// Every fused form computes what the separate instructions compute, rounding by rounding.
void Compiler::FuseSweepInstructions() {
  auto defines_acc = [](uint32_t op) {
    return op == VOP_LD || op == VOP_LDR || op == VOP_LDS || op == VOP_LDI || op == VOP_FIN || op == VOP_END;
  };
  std::vector<uint64_t> &out = scratch_code_;
  out.clear();
  out.reserve(code_.size());
  size_t sweep_first = 0;  // index in code_ of the first instruction of the sweep being copied
  for (size_t i = 0; i < code_.size(); ++i) {
    const uint64_t w = code_[i];
    const uint32_t lo = static_cast<uint32_t>(w);
    if (VI_OP(w) == VOP_SWEEP) sweep_first = i + 1;
    // Mul acc, acc ; reduce_sum rB, acc ; endsweep   (acc dead afterwards)  ->  reduce_sum.square rB, acc
    if (VI_OP(w) == VOP_BINF && (VI_SUB(w) & 0x3fu) == VB_MUL && VI_KIND(w) == VK_ACC && VI_RND(w) == VRND_NONE &&
        !(lo & VI_UNIFORM) && i + 2 < code_.size() && VI_OP(code_[i + 1]) == VOP_RED && VI_SUB(code_[i + 1]) == VR_SUM &&
        VI_OP(code_[i + 2]) == VOP_ENDSWEEP && i + 3 < code_.size() && defines_acc(VI_OP(code_[i + 3])) &&
        sweep_first < code_.size() && defines_acc(VI_OP(code_[sweep_first])) && sweep_first <= i) {
      out.push_back(code_[i + 1] | (static_cast<uint64_t>(VRF_SQUARE) << 8));
      ++i;
      continue;
    }
    // two S-register float binaries in a row
    if (VI_OP(w) == VOP_BINF && VI_KIND(w) == VK_SREG && !(lo & VI_UNIFORM) && i + 1 < code_.size()) {
      const uint64_t n = code_[i + 1];
      if (VI_OP(n) == VOP_BINF && VI_KIND(n) == VK_SREG && !(static_cast<uint32_t>(n) & VI_UNIFORM)) {
        const uint32_t second = (VI_SUB(n) & 0x3fu) | (VI_A(n) << 8) | (VI_RND(n) << 16);
        out.push_back(VI_MAKE(VOP_BINF, VI_SUB(w), VK_SREG2, VI_RND(w), VI_A(w), second));
        ++i;
        continue;
      }
      // an S-register float binary in front of one on a memory operand: one instruction (VI_PRE_SREG)
      const uint32_t sub1 = VI_SUB(w) & 0x3fu;
      if (VI_OP(n) == VOP_BINF && VI_KIND(n) == VK_MEM && !(static_cast<uint32_t>(n) & VI_UNIFORM) && VI_IMM(n) == 0 &&
          (sub1 == VB_ADD || sub1 == VB_SUB || sub1 == VB_RSUB || sub1 == VB_MUL)) {
        const uint32_t pre = VI_PRE_SREG | sub1 | (VI_A(w) << 8) | (VI_RND(w) << 16);
        out.push_back((n & 0xffffffffull) | (static_cast<uint64_t>(pre) << 32));
        ++i;
        continue;
      }
    }
    out.push_back(w);
  }
  // store / reduce ; endsweep  ->  one instruction that also closes the round; a sweep with nothing in it goes
  code_.clear();
  for (size_t i = 0; i < out.size(); ++i) {
    uint64_t w = out[i];
    if (VI_OP(w) == VOP_SWEEP && (VI_IMM(w) & 0xffu) == (VR_NONE | (VR_NONE << 4)) && i + 1 < out.size() &&
        VI_OP(out[i + 1]) == VOP_ENDSWEEP) {
      ++i;
      continue;
    }
    // reduce_sum r0 ; reduce_sum.square r1 ; endsweep  ->  one instruction for both slots
    if (VI_OP(w) == VOP_RED && VI_SUB(w) == VR_SUM && VI_A(w) == 0 && i + 2 < out.size() && VI_OP(out[i + 1]) == VOP_RED &&
        VI_SUB(out[i + 1]) == (VR_SUM | VRF_SQUARE) && VI_A(out[i + 1]) == 1 && VI_OP(out[i + 2]) == VOP_ENDSWEEP) {
      code_.push_back(w | (static_cast<uint64_t>(VRF_PAIR) << 8) | VI_ENDS);
      i += 2;
      continue;
    }
    // reduce ; copy to a V register ; endsweep  ->  the copy first (a plain reduce leaves the accumulator as it is), so
    // that the reduce can close the round
    if (VI_OP(w) == VOP_RED && !(VI_SUB(w) & (VRF_SQUARE | VRF_PAIR)) && i + 2 < out.size() && VI_OP(out[i + 1]) == VOP_STR &&
        VI_OP(out[i + 2]) == VOP_ENDSWEEP) {
      code_.push_back(out[i + 1]);
      code_.push_back(w | VI_ENDS);
      i += 2;
      continue;
    }
    if (i + 1 < out.size() && VI_OP(out[i + 1]) == VOP_ENDSWEEP) {
      if (VI_OP(w) == VOP_ST) {
        code_.push_back(w | VI_ENDS);
        ++i;
        continue;
      }
      if (VI_OP(w) == VOP_RED) {
        code_.push_back(w | VI_ENDS);
        ++i;
        continue;
      }
    }
    code_.push_back(w);
  }
}

// Between sweeps a program computes per-output values (a mean, a scale): one number per lane, the same in every
// lane of the team that owns the output. A run of such instructions is bracketed (VOP_UNI_BEGIN / VOP_UNI_END) and
// the interpreter executes it in a small loop of its own, on one float instead of the whole accumulator. When the
// team is the whole workgroup, only its first wave executes the run and hands the S registers and the accumulator
// to the others through local memory: sixteen waves interpreting the same twenty scalar instructions cost more
// than the one barrier.
void Compiler::MarkUniformRuns() {
  if ((hdr_.sched & VS_KIND_MASK) != VS_REDX) return;
  if (k_->tuning_.vec_runs == 1 && !hdr_.team_is_block) return;  // tuning: runs only where one wave stands in for the others
  auto bcast_load = [&](uint64_t w) {
    return VI_OP(w) == VOP_LD && VI_KIND(w) == VK_MEM && !(mems_[VI_A(w)].flags & (VMF_VEC | VMF_GATHER)) && !mem_is_view_[VI_A(w)];
  };
  auto starts = [&](uint64_t w) {
    const uint32_t op = VI_OP(w);
    return op == VOP_FIN || op == VOP_LDS || op == VOP_LDI || bcast_load(w);
  };
  auto inside = [&](uint64_t w) {
    const uint32_t op = VI_OP(w);
    if (starts(w) || op == VOP_STS) return true;
    const bool arith = op == VOP_UN || op == VOP_CAST || op == VOP_BINF || op == VOP_BINI || op == VOP_CMP;
    return arith && (static_cast<uint32_t>(w) & VI_UNIFORM) != 0;
  };
  std::vector<uint64_t> &out = scratch_code_;
  out.clear();
  out.reserve(code_.size() + 8);
  bool in_sweep = false;
  // The waves that skip a run never compute the offsets of its memory operands: the first memory instruction behind
  // the run that would reuse them (VI_SAME_OFFS) computes its own instead.
  bool offsets_stale = false;
  for (size_t i = 0; i < code_.size();) {
    uint64_t w = code_[i];
    const uint32_t op = VI_OP(w);
    if (op == VOP_SWEEP) {
      in_sweep = true;
      offsets_stale = false;  // (a sweep starts from offsets of its own)
    }
    if (static_cast<uint32_t>(w) & VI_ENDS) {
      in_sweep = false;
    }
    if (!in_sweep && starts(w)) {
      size_t j = i;
      while (j < code_.size() && inside(code_[j])) ++j;
      if (j - i >= 4) {
        out.push_back(VI_MAKE(VOP_UNI_BEGIN, 0, 0, 0, 0, static_cast<uint32_t>(j - i + 1)));
        out.insert(out.end(), code_.begin() + i, code_.begin() + j);
        out.push_back(VI_MAKE(VOP_UNI_END, 0, 0, 0, 0, 0));
        for (size_t q = i; q < j; ++q) offsets_stale = offsets_stale || (VI_OP(code_[q]) >= VOP_SRC_BASE && VI_KIND(code_[q]) == VK_MEM);
        i = j;
        continue;
      }
    }
    if (offsets_stale && (op == VOP_ST || (op >= VOP_SRC_BASE && VI_KIND(w) == VK_MEM))) {
      if (static_cast<uint32_t>(w) & VI_SAME_OFFS) {
        w &= ~static_cast<uint64_t>(VI_SAME_OFFS);
        offsets_stale = false;
      } else if (!(static_cast<uint32_t>(w) & VI_OFFS_ASIDE)) {
        offsets_stale = false;  // offsets of its own, current from here on
      }
    }
    out.push_back(w);
    ++i;
  }
  code_.swap(out);
}

// Whether the finished instruction stream fits the sweep build of the device VM (VS_SWEEPS in isa_gfx950.h spells
// out the vocabulary). Everything is decided from the instruction words and the operand descriptors: shapes,
// alignment and ragged ends are the device's business on either build.
bool Compiler::FitsSweepBuild() {
  if ((hdr_.sched & VS_KIND_MASK) != VS_REDX || (hdr_.sched & VS_WIDE)) return false;
  if (hdr_.n_kdim > 2 || hdr_.n_rdim > 2) return false;  // (the build walks index spaces of at most two axes)
  auto plain_mem = [&](uint32_t a) { return (mems_[a].flags & (VMF_VEC | VMF_GATHER)) == 0; };
  const size_t n = code_.size();
  for (size_t i = 0; i < n; ++i) {
    const uint64_t w = code_[i];
    const uint32_t op = VI_OP(w), kind = VI_KIND(w);
    if (op != VOP_SWEEP) {
      // between the sweeps: one value per lane
      switch (op) {
        case VOP_END: case VOP_UNI_BEGIN: case VOP_UNI_END: case VOP_FIN: case VOP_LDS: case VOP_LDI: case VOP_STS:
        case VOP_UN: case VOP_CAST: case VOP_ENDSWEEP:
          break;
        case VOP_ST:
          if (!plain_mem(VI_A(w))) return false;
          break;
        case VOP_LD: case VOP_BINF: case VOP_BINI: case VOP_CMP: case VOP_MSK: case VOP_MOVM:
          if (kind == VK_REG || (kind == VK_MEM && !plain_mem(VI_A(w)))) return false;
          if (kind == VK_SREG2 && op != VOP_BINF) return false;
          if (kind == VK_MEM && op == VOP_BINF && (VI_IMM(w) & VI_PRE_SREG)) return false;
          break;
        default:
          return false;  // V registers
      }
      continue;
    }
    // a sweep: the load that opens it, then the body up to the instruction that closes the round
    if (i + 2 >= n) return false;
    const uint64_t ld = code_[i + 1];
    if (VI_OP(ld) != VOP_LD || VI_KIND(ld) != VK_MEM || (static_cast<uint32_t>(ld) & (VI_UNIFORM | VI_ENDS))) return false;
    const VMemDesc &ma = mems_[VI_A(ld)];
    constexpr uint32_t kWide = VMF_VEC | VMF_ALIGNED;
    if ((ma.flags & (kWide | VMF_GATHER)) != kWide) return false;
    auto walks_like_load = [&](uint32_t a) {
      const VMemDesc &m = mems_[a];
      // contiguous and aligned, or one fp32 element per slab: what the build's interior rounds access without guards
      if ((m.flags & (kWide | VMF_GATHER)) != kWide && !((m.flags & (VMF_VEC | VMF_GATHER)) == 0 && m.dtype == VDT_F32)) return false;
      bool none = true;
      for (int d = 0; d < DVM_VEC_MAXR; ++d) none = none && m.rstride[d] == 0;
      return none || std::memcmp(m.rstride, ma.rstride, sizeof(ma.rstride)) == 0;
    };
    size_t j = i + 2;
    for (;; ++j) {
      if (j >= n || j - (i + 2) >= DVM_VEC_SWEEP_BODY) return false;
      const uint64_t b = code_[j];
      const uint32_t bop = VI_OP(b), bk = VI_KIND(b), bsub = VI_SUB(b);
      if (static_cast<uint32_t>(b) & VI_UNIFORM) return false;
      switch (bop) {
        case VOP_BINF:
          if ((bsub & 0x3fu) > VB_MAX) return false;
          if (bk == VK_MEM) {
            if (!walks_like_load(VI_A(b))) return false;
            if ((VI_IMM(b) & VI_PRE_SREG) && (VI_IMM(b) & 0x3fu) > VB_MAX) return false;
          } else if (bk == VK_SREG2) {
            if ((VI_IMM(b) & 0x3fu) > VB_MAX) return false;
          } else if (bk != VK_IMM && bk != VK_SREG && bk != VK_ACC) {
            return false;
          }
          break;
        case VOP_RED:
          if (bsub & VRF_INT) return false;
          break;
        case VOP_LD:  // another input of the sweep
          if (bk != VK_MEM || !walks_like_load(VI_A(b)) || (static_cast<uint32_t>(b) & (VI_LD_KEEP_WR | VI_LD_KEEP_RD | VI_LD_RED2))) return false;
          break;
        case VOP_ST:
          if (!walks_like_load(VI_A(b)) || !(mems_[VI_A(b)].flags & VMF_VEC)) return false;
          break;
        case VOP_UN:
          if (bsub > VU_TRUNC) return false;
          break;
        case VOP_CAST:
          if (bsub != VC_RND) return false;
          break;
        case VOP_ENDSWEEP:
          break;
        default:
          return false;
      }
      if (static_cast<uint32_t>(b) & VI_ENDS) break;
    }
    i = j;
  }
  return true;
}

// A reduce with consumers reads its input twice: once for the statistics, once to apply them. What the
// second sweep does not have to fetch again from HBM:
//  * the first rounds of the first sweep stay in the workgroup's spare local memory (VI_LD_KEEP_WR/RD);
//  * a later sweep without reduces of its own runs last round first (VSW_REVERSE), starting with the data the
//    L2 cache still holds from the end of the sweep before, and ending with the parked rounds.
// Called with the blob filled in and lds_bytes set; edits the instruction words in the blob.
void Compiler::PlanRereads() {
  // tuning switch DVM_VEC_REREAD: 0 off, 2 parked rounds only, 3 reversed sweeps only (default: both)
  const int mode = k_->tuning_.vec_reread;
  const bool on = mode != 0, park = mode != 3, reverse = mode != 2;
  if (!on || (hdr_.sched & VS_KIND_MASK) != VS_REDX || (hdr_.sched & VS_WIDE)) return;
  uint64_t *cw = prog_->blob.w + hdr_.code_off;
  const size_t n = code_.size();
  const uint32_t team = hdr_.team_is_block ? prog_->threads : (1u << hdr_.team_log2);
  const uint32_t per_round = team * u_;
  const uint32_t n_rounds = (hdr_.n_ridx + per_round - 1) / per_round;
  if (n_rounds < 2) return;
  // sweeps: position of the VOP_SWEEP word and of the load that opens it (or -1)
  struct Sw { size_t at; int ld; bool reduces; };
  std::vector<Sw> sweeps;
  for (size_t i = 0; i < n; ++i) {
    if (VI_OP(cw[i]) != VOP_SWEEP) continue;
    Sw sw{i, -1, (VI_IMM(cw[i]) & 0xffu) != (VR_NONE | (VR_NONE << 4))};
    if (i + 1 < n && VI_OP(cw[i + 1]) == VOP_LD && VI_KIND(cw[i + 1]) == VK_MEM && (mems_[VI_A(cw[i + 1])].flags & VMF_VEC)) {
      sw.ld = static_cast<int>(i + 1);
    }
    sweeps.push_back(sw);
  }
  for (size_t k = 1; k < sweeps.size(); ++k) {
    if (reverse && !sweeps[k].reduces) cw[sweeps[k].at] |= static_cast<uint64_t>(VSW_REVERSE) << 8;
  }
  // local memory left to this workgroup when as many workgroups as the registers allow share the CU
  const uint32_t per_cu = 1024 / std::max<uint32_t>(prog_->threads, 64);
  const uint32_t budget = std::min<uint32_t>(160 * 1024, g_system.lds_per_wg) / per_cu;
  uint32_t fixed = prog_->lds_bytes + DVM_PARAM_BYTES + 1024;
  const uint32_t per_round_bytes = prog_->threads * u_ * 32;  // one round of one operand, as fp32
  // park rounds of the first pair of sweeps that open with a load of the same operand
  if (!park) return;
  for (size_t a = 0; a + 1 < sweeps.size(); ++a) {
    if (sweeps[a].ld < 0) continue;
    for (size_t b = a + 1; b < sweeps.size(); ++b) {
      if (sweeps[b].ld < 0 || VI_A(cw[sweeps[b].ld]) != VI_A(cw[sweeps[a].ld])) continue;
      // When both sweeps go on with the same instruction behind the load (x + residual: a float binary on an
      // immediate or on a memory operand with the load's offsets), its result is what gets parked, and the
      // reading sweep skips it in parked rounds: neither operand is read twice. A result rounded to a 16-bit
      // type is parked in that type, at half the local memory per round.
      uint32_t prefix = 0, fmt = VF_F32;
      const size_t la = static_cast<size_t>(sweeps[a].ld), lb = static_cast<size_t>(sweeps[b].ld);
      if (la + 2 < n && lb + 2 < n && cw[la + 1] == cw[lb + 1]) {
        const uint64_t w = cw[la + 1];
        const uint32_t lo = static_cast<uint32_t>(w);
        const bool operand_ok = VI_KIND(w) == VK_IMM || (VI_KIND(w) == VK_MEM && (lo & VI_SAME_OFFS));
        if (VI_OP(w) == VOP_BINF && operand_ok && !(lo & (VI_UNIFORM | VI_ENDS))) {
          prefix = 1;
          fmt = VI_RND(w) == VRND_F16 ? VF_F16 : (VI_RND(w) == VRND_BF16 ? VF_BF16 : VF_F32);
        }
      }
      const uint32_t round_bytes = fmt == VF_F32 ? per_round_bytes : per_round_bytes / 2;
      if (budget <= fixed + round_bytes) return;
      const uint32_t rounds = std::min<uint32_t>(n_rounds, (budget - fixed) / round_bytes);
      const uint64_t imm = static_cast<uint64_t>(rounds | (prefix << 16) | (fmt << 20)) << 32;
      cw[la] |= VI_LD_KEEP_WR | imm;
      cw[lb] |= VI_LD_KEEP_RD | imm;
      // a third sweep over the same operand (the division of a softmax) takes the parked rounds as well
      for (size_t c = b + 1; c < sweeps.size(); ++c) {
        if (sweeps[c].ld < 0 || VI_A(cw[sweeps[c].ld]) != VI_A(cw[la])) continue;
        const size_t lc = static_cast<size_t>(sweeps[c].ld);
        if (prefix != 0 && (lc + 1 >= n || cw[lc + 1] != cw[la + 1])) continue;
        if (static_cast<uint32_t>(cw[lc]) & (VI_LD_KEEP_WR | VI_LD_KEEP_RD | VI_LD_RED2)) continue;
        cw[lc] |= VI_LD_KEEP_RD | imm;
      }
      prog_->lds_bytes += rounds * round_bytes;
      return;
    }
  }
}

}  // namespace dvm
