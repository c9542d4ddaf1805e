// gfx950 vector VM: persistent interpreter kernels for fused
// load / elementwise / cast / broadcast / reduce / store programs.
//
// Replaces the reference's generic interpreter (src/vm_gpu.cu:1552-1617 and the
// RunOp switch at :941-1548) with a register-resident design for CDNA4:
//  * a lane owns U slabs of E=8 consecutive elements of the innermost axis per
//    instruction; slab u of all lanes is contiguous, so every global access is
//    a coalesced 128-bit access and U of them are in flight per lane;
//  * values stay in an accumulator (U*E VGPRs); local memory holds only the
//    few values that must outlive an instruction chain and the reduce partials
//    that cross waves;
//  * broadcast operands are never materialised: they are stride-0 operands;
//  * a reduce and its consumers run in one launch as consecutive sweeps over
//    the reduce index space of the workgroup's outputs;
//  * decoding is wave-uniform (scalar unit): the cost of one dispatch is spread
//    over U*E*64 elements.
// Numerics follow the reference device functors (src/vm_gpu.cu:198-329): fp16
// and bf16 arithmetic is one fp32 operation rounded once, sums accumulate in
// fp64 (src/vm_gpu.cu:779-866), float->int is C truncation, round is
// half-to-even.
#include "vec_common.h"

namespace {

// the program, copied from the kernel argument once per workgroup
__shared__ uint32_t prog32[DVM_PARAM_BYTES / 4];

// PARTS: the program's reduce is shared between workgroups (VVecHeader::r_chunk); a build of its own, so that the
// programs without one pay nothing for the part bounds.
template <int SCHED, bool PARTS = false>
__device__ __forceinline__ void vm_vector(const VmParam &p) {
#ifdef DVM_VEC_STAMPS
  const uint64_t stamp_base = p.w[DVM_PARAM_WORDS - 1];
  uint32_t stamp_n = 0;
#endif
  STAMP();
  // The blob arrives as a kernel argument; decoding from there would cost a
  // dependent scalar-memory round trip per access, so each workgroup copies it
  // into local memory once and decodes from there.
  {
    // uniform trip count and clamped indices: no per-lane branch (lanes past the end rewrite the last word)
    // only the words the program occupies are read: the argument segment is far away
    const uint32_t *src = reinterpret_cast<const uint32_t *>(p.w);
    const VVecHeader *hp = reinterpret_cast<const VVecHeader *>(p.w);
    uint32_t used = (hp->code_off + hp->n_code) * 2;
    used = used < DVM_PARAM_BYTES / 4 ? used : DVM_PARAM_BYTES / 4;
    const uint32_t trips = (used + blockDim.x - 1) / blockDim.x;
    for (uint32_t t = 0; t < trips; ++t) {
      uint32_t i = t * blockDim.x + threadIdx.x;
      i = i < used ? i : used - 1;
      prog32[i] = src[i];
    }
    __syncthreads();
  }
  STAMP();
  // the scalar fields of the header live in scalar registers; the axis tables stay in local memory
  struct {
    uint32_t n_kdim, n_rdim, team_log2, team_is_block, n_kidx, n_ridx, inner_extent, n_items, mem_off, code_off, n_vslot, r_chunk, k_per_chunk;
    const VDim *kdims, *rdims;
  } h;
  {
    const VVecHeader *hp = reinterpret_cast<const VVecHeader *>(prog32);
    h.n_kdim = uni(hp->n_kdim);
    h.n_rdim = uni(hp->n_rdim);
    h.team_log2 = uni(hp->team_log2);
    h.team_is_block = uni(hp->team_is_block);
    h.n_kidx = uni(hp->n_kidx);
    h.n_ridx = uni(hp->n_ridx);
    h.inner_extent = uni(hp->inner_extent);
    h.n_items = uni(hp->n_items);
    h.mem_off = uni(hp->mem_off);
    h.code_off = uni(hp->code_off);
    h.n_vslot = uni(hp->n_vslot);
    h.r_chunk = uni(hp->r_chunk);
    h.k_per_chunk = uni(hp->k_per_chunk);
    h.kdims = hp->kdims;
    h.rdims = hp->rdims;
  }
  const uint32_t mem_off = h.mem_off;
  const uint32_t *code32 = prog32 + 2 * h.code_off;

  const uint32_t tid = threadIdx.x;
  const uint32_t nthreads = blockDim.x;
  const uint32_t tlog = h.team_log2;
  const bool team_is_block = h.team_is_block != 0;
  // per-team runs (VOP_UNI_BEGIN .. VOP_UNI_END) are computed by the first wave when the team is the workgroup
  const uint32_t skips_runs = (SCHED == VS_REDX && team_is_block && uni(tid >> 6) != 0u) ? 1u : 0u;
  vf4 *planes = reinterpret_cast<vf4 *>(lds + DVM_VEC_RED_SCRATCH_DOUBLES(SCHED, nthreads));  // behind the reduce scratch
  vf4 *keep_lds = planes + h.n_vslot * U * nthreads;      // behind the V registers: rounds parked by VI_LD_KEEP_WR

  // lane -> (kept local index, reduce local index)
  uint32_t k_local, r_local, k_per_wg, r_step;
  if constexpr (SCHED == VS_POINTWISE) {
    k_local = tid; r_local = 0; k_per_wg = nthreads * U; r_step = 1;
  } else if constexpr (SCHED == VS_REDX) {
    if (team_is_block) {
      k_local = 0; r_local = tid; k_per_wg = 1; r_step = nthreads;
    } else {
      k_local = tid >> tlog; r_local = tid & ((1u << tlog) - 1u); k_per_wg = nthreads >> tlog; r_step = 1u << tlog;
    }
  } else {
    k_local = tid & ((1u << tlog) - 1u); r_local = tid >> tlog; k_per_wg = 1u << tlog; r_step = nthreads >> tlog;
  }
  // (a reduce shared between workgroups: a lane walks one part of the reduced index space, r_chunk indices long)
  const uint32_t r_span = PARTS ? h.r_chunk : h.n_ridx;
  const uint32_t n_rounds = SCHED == VS_POINTWISE ? 1u : (r_span + r_step * U - 1) / (r_step * U);
  constexpr bool inner_red = SCHED == VS_REDX;

  SRegs sr;
  sr.s0 = sr.s1 = sr.s2 = sr.s3 = sr.s4 = sr.s5 = sr.s6 = sr.s7 = 0.0f;
  Acc acc;
  FOR_U acc.v[u] = 0.0f;
  uint32_t mask = 0;
  uint32_t park_slot = 0, park_fmt = 0;  // a value waiting to be parked after the instruction behind its load (slot + 1; 0: none)
  RedAcc<SCHED> racc0, racc1;
  red_init<SCHED>(racc0, VR_SUM);
  red_init<SCHED>(racc1, VR_SUM);
  uint32_t red_flip = 0, box_flip = 0;  // which of the two shared buffers the next sweep end / hand-over uses

  for (uint32_t item = blockIdx.x; item < h.n_items; item += gridDim.x) {
    // position of the lane in the kept space (POINTWISE: of slab 0; slab u is nthreads further each)
    const uint32_t kidx = item * k_per_wg + k_local;
    const bool kvalid = kidx < h.n_kidx;
    // first index of the lane's part of the reduced index space, and the index behind its last
    uint32_t r_base = 0, r_lim = h.n_ridx;
    if constexpr (PARTS) {
      r_base = (kidx / h.k_per_chunk) * h.r_chunk;
      r_lim = (r_base + r_span < h.n_ridx) ? r_base + r_span : h.n_ridx;
    }
    uint32_t nvp_out;  // valid counts outside sweeps
    if constexpr (SCHED == VS_POINTWISE) {
      nvp_out = 0;
      FOR_U {
        const uint32_t ku = kidx + u * nthreads;
        // computed for a clamped index and masked afterwards: a select, never a per-lane branch
        const uint32_t in_range = ku < h.n_kidx ? 0xfu : 0u;
        const uint32_t nv = group_valid(ku < h.n_kidx ? ku : 0u, h.kdims, h.n_kdim, h.inner_extent) & in_range;
        nvp_out |= nv << (4 * u);
      }
    } else {
      const uint32_t nv_in = inner_red ? 1u : group_valid(kvalid ? kidx : 0u, h.kdims, h.n_kdim, h.inner_extent);
      const uint32_t nv = nv_in & (kvalid ? 0xfu : 0u);
      nvp_out = nv * kAllOnes;
    }

    const Slabs sl_out = slab_state(nvp_out);
    bool in_sweep = false;
    Slabs sl = sl_out;  // valid counts of the current round's slabs (outside sweeps: of the lane's output)
    uint32_t round = 0, sweep_pc = 0, slot_kinds = 0;
    bool sweep_rev = false;   // the sweep walks its rounds last to first (VSW_REVERSE)
    uint32_t ridx = r_base + r_local;  // reduce-space index of slab 0 in the current round
    Offs last_off;            // element offsets of the last memory instruction (VI_SAME_OFFS reuses them)
    FOR_U last_off.v[u] = 0;

    // The instruction word is read from local memory one instruction ahead: the read of the next word is
    // in flight while the current instruction executes. The next pc is known at decode time, because only
    // the end of a round (VOP_ENDSWEEP, or an instruction flagged to close the round) ever jumps.
    const vu2 *code64 = reinterpret_cast<const vu2 *>(code32);
    uint32_t pc = 0;
    vu2 fetched = code64[0];
    while (true) {
      uint32_t w0 = uni(fetched[0]);
      const uint32_t imm = uni(fetched[1]);
      uint32_t op = w0 & 0x7fu;
      if (op == VOP_END) break;
      uint32_t sub = (w0 >> 8) & 0xffu;  // (w0, op and sub change when a load takes the instruction behind it along)
      const uint32_t a = w0 >> 24;
      // branch-free: the round-closing bit and, for the waves that skip per-team runs, the jump to their end
      const bool ends = SCHED != VS_POINTWISE && (w0 & VI_ENDS) != 0;
      const uint32_t back = (ends ? 1u : 0u) & (round + 1 < n_rounds ? 1u : 0u);
      pc = back ? sweep_pc : pc + 1;
      pc += ((op == VOP_UNI_BEGIN ? 1u : 0u) & skips_runs) * (imm - 1u);
      fetched = code64[pc];
      auto end_round = [&](bool round_done, bool recount) {
        if constexpr (SCHED != VS_POINTWISE) {
          // end of a round: the next one (the decode above has already turned the pc back), or the end of
          // the sweep, where the slots' partials are combined across lanes
          if (round_done) {
            ++round;
            if (round < n_rounds) {
              ridx = sweep_rev ? ridx - r_step * U : ridx + r_step * U;
            } else {
              in_sweep = false;
              STAMP();
              const uint32_t k0 = slot_kinds & 0xfu, k1 = (slot_kinds >> 4) & 0xfu;
              if constexpr (SCHED == VS_REDX) {
                if (k0 <= VR_MIN || k1 <= VR_MIN) {
                  red_finish_x(racc0.v[0], racc1.v[0], k0, k1, tlog, fresh(h.team_is_block) != 0u, tid, nthreads, red_flip, lds);
                }
              } else {
                if (k0 <= VR_MIN) racc0 = red_finish_y<SCHED>(racc0, k0, tlog, nthreads, k_local, r_local, lds);
                if (k1 <= VR_MIN) racc1 = red_finish_y<SCHED>(racc1, k1, tlog, nthreads, k_local, r_local, lds);
              }
              STAMP();
            }
          }

          // valid counts of the round's slabs
          if (recount) {
            if (in_sweep) {
              uint32_t nvp = 0;
              FOR_U {
                const uint32_t ru = ridx + u * r_step;
                const bool ok = kvalid && ru < r_lim;
                uint32_t nv = inner_red ? group_valid(ok ? ru : 0u, h.rdims, h.n_rdim, h.inner_extent) : (nvp_out & 0xfu);
                nv &= ok ? 0xfu : 0u;
                nvp |= nv << (4 * u);
              }
              sl = slab_state(nvp);
            } else {
              sl = sl_out;
            }
          }
        }
      };
      // VOP_LD flagged VI_LD_PAIR: the next instruction is a float binary whose memory operand has the load's
      // element offsets. When both take the wide path the load fetches both operands in one trip to memory and
      // the binary is finished in the same dispatch (true: src holds its operand; w0, op, sub are the binary's).
      auto take_next_along = [&](const VMemDesc &m, const Offs &off, const Slabs &s2, Acc &x, Acc &y) -> bool {
        constexpr uint32_t kFast = VMF_VEC | VMF_ALIGNED;
        if ((w0 & VI_LD_PAIR) != 0 && (m.flags & kFast) == kFast && s2.uniform) {
          const uint32_t wb = uni(fetched[0]);
          const VMemDesc mb = load_desc(prog32, mem_off, wb >> 24);
          if ((mb.flags & kFast) == kFast) {
            mem_load2_wide(m, mb, off, s2.full, x, y);
            w0 = wb;
            op = wb & 0x7fu;
            sub = (wb >> 8) & 0xffu;
            ++pc;
            fetched = code64[pc];
            return true;
          }
        }
        mem_load(m, off, s2, x);
        return false;
      };

      // ---- a run of per-output arithmetic (VOP_UNI_BEGIN .. VOP_UNI_END): every instruction in it works on one
      // value per lane, so the run has a small loop of its own: one float instead of the accumulator's U*E, a
      // switch over the few opcodes a run may hold. (The waves that skip the run are already past it.) ----
      if constexpr (SCHED == VS_REDX) {
        if (op == VOP_UNI_BEGIN && skips_runs == 0u) {
          const uint32_t run_end = pc + imm - 1u;  // index of the VOP_UNI_END
          float x = acc.v[0][0];
          while (pc < run_end) {
            const uint32_t r0 = uni(fetched[0]);
            const uint32_t rimm = uni(fetched[1]);
            ++pc;
            fetched = code64[pc];
            const uint32_t rop = r0 & 0x7fu, rsub = (r0 >> 8) & 0xffu, ra = r0 >> 24, rkind = (r0 >> 16) & 0xfu;
            if (rop >= VOP_SRC_BASE && rop != VOP_LD) {
              const float sv = rkind == VK_IMM ? __uint_as_float(rimm) : (rkind == VK_SREG ? sreg_read(sr, ra) : x);
              x = uniform_binary(rop, rsub, x, sv);
              if (rop == VOP_BINF) {
                const uint32_t rnd = (r0 >> 20) & 0x3u;
                x = rnd == VRND_F16 ? round_f16(x) : (rnd == VRND_BF16 ? round_bf16(x) : x);
              }
              continue;
            }
            switch (rop) {
              case VOP_FIN: {
                const double d = ra == 0 ? racc0.v[0] : racc1.v[0];
                x = (rsub & VRF_INT) ? __int_as_float(static_cast<int32_t>(d)) : static_cast<float>(d);
                break;
              }
              case VOP_LDS: x = sreg_read(sr, ra); break;
              case VOP_LDI: x = __uint_as_float(rimm); break;
              case VOP_STS: sreg_write(sr, ra, x); break;
              case VOP_LD: {  // one element per output (an operand without the reduced axes), any type
                const VMemDesc m = load_desc(prog32, mem_off, ra);
                uint64_t koff = last_off.v[0];
                if (!(r0 & VI_SAME_OFFS)) koff = space_offset(kvalid ? kidx : 0u, h.kdims, h.n_kdim, m.kstride, false);
                FOR_U last_off.v[u] = koff;
                const float v = elem_load(m.addr, m.dtype, kvalid ? koff : 0u);
                x = kvalid ? v : 0.0f;
                break;
              }
              case VOP_UN: {
                x = uniform_unary(rsub, x);
                const uint32_t rnd = (r0 >> 20) & 0x3u;
                x = rnd == VRND_F16 ? round_f16(x) : (rnd == VRND_BF16 ? round_bf16(x) : x);
                break;
              }
              default: {  // VOP_CAST
                x = uniform_cast(rsub, x);
                if (rsub == VC_I2F || rsub == VC_RND) {
                  const uint32_t rnd = (r0 >> 20) & 0x3u;
                  x = rnd == VRND_F16 ? round_f16(x) : (rnd == VRND_BF16 ? round_bf16(x) : x);
                }
                break;
              }
            }
          }
          FOR_U acc.v[u] = x;
          continue;  // `fetched` holds the VOP_UNI_END
        }
      }
      // ---- one value per lane (VI_UNIFORM): compute element 0 and copy it ----
      if (w0 & VI_UNIFORM) {
        const uint32_t kind = (w0 >> 16) & 0xfu;
        float x = acc.v[0][0];
        if (op >= VOP_SRC_BASE) {
          const float sv = kind == VK_IMM ? __uint_as_float(imm) : (kind == VK_SREG ? sreg_read(sr, a) : x);
          x = uniform_binary(op, sub, x, sv);
        } else if (op == VOP_UN) {
          x = uniform_unary(sub, x);
        } else {
          x = uniform_cast(sub, x);
        }
        const uint32_t rnd = (w0 >> 20) & 0x3u;
        const bool rounds = op == VOP_BINF || op == VOP_UN || (op == VOP_CAST && (sub == VC_I2F || sub == VC_RND));
        if (rounds) x = rnd == VRND_F16 ? round_f16(x) : (rnd == VRND_BF16 ? round_bf16(x) : x);
        FOR_U acc.v[u] = x;
        continue;
      }
      if (op >= VOP_SRC_BASE) {
        const uint32_t kind = (w0 >> 16) & 0xfu;
        // ---- scalar source (immediate or S register): no need to widen it to U*E values ----
        if ((kind == VK_IMM || kind == VK_SREG || kind == VK_SREG2) && (op == VOP_BINF || op == VOP_BINI || op == VOP_CMP)) {
          float sv = kind == VK_IMM ? __uint_as_float(imm) : sreg_read(sr, a);
          if (op == VOP_BINF) {
            // one operation, or two chained ones (VK_SREG2: the second sits in the immediate)
            uint32_t bsub = sub & 0x3fu, brnd = (w0 >> 20) & 0x3u;
            for (uint32_t left = kind == VK_SREG2 ? 2u : 1u;;) {
              switch (bsub) {
                case VB_ADD: FOR_U acc.v[u] = acc.v[u] + sv; break;
                case VB_SUB: FOR_U acc.v[u] = acc.v[u] - sv; break;
                case VB_RSUB: FOR_U acc.v[u] = sv - acc.v[u]; break;
                case VB_MUL: FOR_U acc.v[u] = acc.v[u] * sv; break;
                case VB_DIV: FOR_U acc.v[u] = acc.v[u] / sv; break;
                case VB_RDIV: FOR_U acc.v[u] = sv / acc.v[u]; break;
                case VB_MIN: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] < sv ? acc.v[u][e] : sv; break;
                case VB_MAX: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] > sv ? acc.v[u][e] : sv; break;
                case VB_AND: FOR_U FOR_E acc.v[u][e] = (acc.v[u][e] != 0.0f && sv != 0.0f) ? 1.0f : 0.0f; break;
                case VB_OR: FOR_U FOR_E acc.v[u][e] = (acc.v[u][e] != 0.0f || sv != 0.0f) ? 1.0f : 0.0f; break;
                case VB_POW: FOR_U acc.v[u] = slab_pow(acc.v[u], vf8(sv)); break;
                default: FOR_U acc.v[u] = slab_pow(vf8(sv), acc.v[u]); break;
              }
              apply_rnd(acc, brnd);
              if (--left == 0u) break;
              bsub = imm & 0x3fu;
              brnd = (imm >> 16) & 0x3u;
              sv = sreg_read(sr, (imm >> 8) & 0xffu);
            }
          } else if (op == VOP_BINI) {
            const uint32_t si = __float_as_uint(sv);
            switch (sub & 0x3fu) {
              case VBI_ADD: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(acc.v[u][e]) + si); break;
              case VBI_SUB: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(acc.v[u][e]) - si); break;
              case VBI_RSUB: FOR_U FOR_E acc.v[u][e] = __uint_as_float(si - __float_as_uint(acc.v[u][e])); break;
              case VBI_MUL: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(acc.v[u][e]) * si); break;
              case VBI_MIN: FOR_U FOR_E acc.v[u][e] = __int_as_float(min(__float_as_int(acc.v[u][e]), static_cast<int32_t>(si))); break;
              case VBI_WRAP: FOR_U FOR_E acc.v[u][e] = __int_as_float(wrap_index(__float_as_int(acc.v[u][e]), static_cast<int32_t>(si))); break;
              default: FOR_U FOR_E acc.v[u][e] = __int_as_float(max(__float_as_int(acc.v[u][e]), static_cast<int32_t>(si))); break;
            }
          } else {
            const int32_t si = __float_as_int(sv);
            switch (sub & 0x3fu) {
              case VCMP_EQ: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] == sv ? 1.0f : 0.0f; break;
              case VCMP_NE: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] != sv ? 1.0f : 0.0f; break;
              case VCMP_GT: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] > sv ? 1.0f : 0.0f; break;
              case VCMP_GE: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] >= sv ? 1.0f : 0.0f; break;
              case VCMP_LT: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] < sv ? 1.0f : 0.0f; break;
              case VCMP_LE: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] <= sv ? 1.0f : 0.0f; break;
              case VCMP_INT + VCMP_EQ: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) == si ? 1 : 0); break;
              case VCMP_INT + VCMP_NE: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) != si ? 1 : 0); break;
              case VCMP_INT + VCMP_GT: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) > si ? 1 : 0); break;
              case VCMP_INT + VCMP_GE: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) >= si ? 1 : 0); break;
              case VCMP_INT + VCMP_LT: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) < si ? 1 : 0); break;
              default: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) <= si ? 1 : 0); break;
            }
          }
          if constexpr (SCHED == VS_REDX) {
            if (park_slot != 0u) {  // this was the instruction behind a load that parks its round (x * c, x + c)
              vreg_store(keep_lds, park_slot - 1u, park_fmt, nthreads, tid, acc);
              park_slot = 0u;
            }
          }
          continue;
        }
        // ---- fetch a full-width source operand ----
        Acc src;
        if (kind == VK_MEM) {
          const VMemDesc m = load_desc(prog32, mem_off, a);
          Offs off = last_off;
          if (!(w0 & VI_SAME_OFFS)) {
            if constexpr (SCHED == VS_POINTWISE) {
              FOR_U {
                const uint32_t ku = kidx + u * nthreads;
                off.v[u] = space_offset(ku < h.n_kidx ? ku : 0u, h.kdims, h.n_kdim, m.kstride, true);
              }
            } else {
              const uint64_t koff = space_offset(kvalid ? kidx : 0u, h.kdims, h.n_kdim, m.kstride, !inner_red);
              FOR_U {
                off.v[u] = koff;
                if (in_sweep) {
                  const uint32_t ru = ridx + u * r_step;
                  off.v[u] += space_offset(ru < r_lim ? ru : 0u, h.rdims, h.n_rdim, m.rstride, inner_red);
                }
              }
            }
            if (!(w0 & VI_OFFS_ASIDE)) last_off = off;
          }
          if (op == VOP_LD) {
            if constexpr (SCHED == VS_REDX) {
              // rounds parked in local memory by the load that opened an earlier sweep over this operand
              const uint32_t lr = sweep_rev ? n_rounds - 1u - round : round;
              const uint32_t n_parked = imm & 0xffffu;
              const uint32_t keep_prefix = (imm >> 16) & 0x3u, keep_fmt = (imm >> 20) & 0x3u;  // VI_LD_KEEP_*: see isa_gfx950.h
              const uint32_t keep_at = keep_fmt == VF_F32 ? 2u * lr : lr;  // fp32 values take two planes per slab
              const bool parked = in_sweep && lr < n_parked;
              if (parked && (w0 & VI_LD_KEEP_RD)) {
                vreg_load(keep_lds, keep_at, keep_fmt, nthreads, tid, acc);
                // what was parked is the value behind the next keep_prefix instructions: they are done already
                pc += keep_prefix;
                fetched = code64[pc];
                continue;
              }
              if (in_sweep && (w0 & VI_LD_RED2)) {
                // The round is this load and the float reduce behind it, which closes the round: fetch this round
                // and the next in one trip to memory, reduce both, and go on two rounds further.
                const uint32_t wr = uni(fetched[0]);
                const uint32_t rsub = (wr >> 8) & 0xffu, rslot = wr >> 24;
                const bool have2 = round + 1u < n_rounds;
                const uint32_t ridx2 = sweep_rev ? ridx - r_step * U : ridx + r_step * U;
                Offs off2 = off;
                Slabs sl2 = sl;
                if (have2) {
                  const uint64_t koff = space_offset(kvalid ? kidx : 0u, h.kdims, h.n_kdim, m.kstride, !inner_red);
                  uint32_t nvp2 = 0;
                  FOR_U {
                    const uint32_t ru = ridx2 + u * r_step;
                    const bool ok = kvalid && ru < r_lim;
                    off2.v[u] = koff + space_offset(ok ? ru : 0u, h.rdims, h.n_rdim, m.rstride, inner_red);
                    uint32_t nv = inner_red ? group_valid(ok ? ru : 0u, h.rdims, h.n_rdim, h.inner_extent) : (nvp_out & 0xfu);
                    nv &= ok ? 0xfu : 0u;
                    nvp2 |= nv << (4 * u);
                  }
                  sl2 = slab_state(nvp2);
                }
                constexpr uint32_t kFast = VMF_VEC | VMF_ALIGNED;
                if (have2 && (m.flags & kFast) == kFast && sl.uniform && sl2.uniform) {
                  mem_load_wide_2rounds(m, off, off2, sl.full, sl2.full, acc, src);
                } else {
                  mem_load(m, off, sl, acc);
                  if (have2) mem_load(m, off2, sl2, src);
                }
                if (w0 & VI_LD_KEEP_WR) {  // (a load with a reduce behind it parks what it loaded: no prefix, fp32)
                  const uint32_t lr2 = sweep_rev ? lr - 1u : lr + 1u;
                  if (lr < n_parked) vreg_store(keep_lds, 2u * lr, VF_F32, nthreads, tid, acc);
                  if (have2 && lr2 < n_parked) vreg_store(keep_lds, 2u * lr2, VF_F32, nthreads, tid, src);
                }
                auto reduce_into_slots = [&](Acc &x, const Slabs &sx) {  // what VOP_RED does, for one round's values
                  if (rsub & VRF_SQUARE) FOR_U x.v[u] = x.v[u] * x.v[u];
                  if (rslot == 0) {
                    red_accumulate<SCHED>(racc0, rsub & 0xfu, x, sx);
                    if (rsub & VRF_PAIR) {
                      FOR_U x.v[u] = x.v[u] * x.v[u];
                      red_accumulate<SCHED>(racc1, rsub & 0xfu, x, sx);
                    }
                  } else {
                    red_accumulate<SCHED>(racc1, rsub & 0xfu, x, sx);
                  }
                };
                reduce_into_slots(acc, sl);
                if (have2) {
                  reduce_into_slots(src, sl2);
                  ++round;
                  ridx = ridx2;
                }
                // the reduce is done: the round ends here, and the next instruction is the load again or what follows the reduce
                pc = round + 1u < n_rounds ? sweep_pc : pc + 1u;
                fetched = code64[pc];
                end_round(true, true);
                continue;
              }
              const bool keep = parked && (w0 & VI_LD_KEEP_WR) != 0;
              const bool pair = take_next_along(m, off, sl, acc, src);
              if (keep) {
                if (keep_prefix == 0) {
                  vreg_store(keep_lds, keep_at, keep_fmt, nthreads, tid, acc);
                } else {  // the value to park is the result of the instruction behind this load
                  park_slot = keep_at + 1u;
                  park_fmt = keep_fmt;
                }
              }
              if (!pair) continue;
            } else if constexpr (SCHED == VS_REDY) {
              if (in_sweep && (w0 & VI_LD_RED2)) {
                // The round is this load and the float reduce behind it, which closes the round. A lane's rounds are
                // rows far apart in memory and nothing else of the wave is in flight meanwhile, so up to four rounds
                // are fetched in one trip and reduced one after the other, in the order of the rounds.
                constexpr int NR = 4;
                const uint32_t wr = uni(fetched[0]);
                const uint32_t rsub = (wr >> 8) & 0xffu, rslot = wr >> 24;
                const uint32_t left = n_rounds - round;
                const uint32_t take = left < static_cast<uint32_t>(NR) ? left : static_cast<uint32_t>(NR);
                constexpr uint32_t kFast = VMF_VEC | VMF_ALIGNED;
                Offs offs[NR];
                Slabs sls[NR];
                Acc xs[NR];
                offs[0] = off;
                sls[0] = sl;
                bool wide_all = take == static_cast<uint32_t>(NR) && (m.flags & kFast) == kFast && sl.uniform;
                const uint64_t koff = space_offset(kvalid ? kidx : 0u, h.kdims, h.n_kdim, m.kstride, true);
#pragma unroll
                for (int j = 1; j < NR; ++j) {
                  uint32_t nvp_j = 0;
                  FOR_U {
                    const uint32_t ru = ridx + (static_cast<uint32_t>(j) * U + u) * r_step;
                    const bool ok = kvalid && ru < r_lim;
                    offs[j].v[u] = koff + space_offset(ok ? ru : 0u, h.rdims, h.n_rdim, m.rstride, false);
                    nvp_j |= (ok ? (nvp_out & 0xfu) : 0u) << (4 * u);
                  }
                  sls[j] = slab_state(nvp_j);
                  wide_all = wide_all && sls[j].uniform;
                }
                if (wide_all) {
#pragma unroll
                  for (int j = 0; j < NR; ++j) mem_load_wide(m, offs[j], sls[j].full, xs[j]);
                } else {
#pragma unroll
                  for (int j = 0; j < NR; ++j)
                    if (static_cast<uint32_t>(j) < take) mem_load(m, offs[j], sls[j], xs[j]);
                }
#pragma unroll
                for (int j = 0; j < NR; ++j) {
                  if (static_cast<uint32_t>(j) >= take) break;
                  Acc &x = xs[j];
                  if (rsub & VRF_SQUARE) FOR_U x.v[u] = x.v[u] * x.v[u];
                  if (rslot == 0) {
                    red_accumulate<SCHED>(racc0, rsub & 0xfu, x, sls[j]);
                    if (rsub & VRF_PAIR) {
                      FOR_U x.v[u] = x.v[u] * x.v[u];
                      red_accumulate<SCHED>(racc1, rsub & 0xfu, x, sls[j]);
                    }
                  } else {
                    red_accumulate<SCHED>(racc1, rsub & 0xfu, x, sls[j]);
                  }
                }
                STAMP();
                round += take - 1u;
                ridx += (take - 1u) * r_step * U;
                pc = round + 1u < n_rounds ? sweep_pc : pc + 1u;
                fetched = code64[pc];
                end_round(true, true);
                continue;
              }
              if (!take_next_along(m, off, sl, acc, src)) continue;
            } else {
              if (!take_next_along(m, off, sl, acc, src)) continue;
            }
            // the binary instruction behind the load: its operand is in src, the switch below finishes it
          } else if (op == VOP_LDX) {
            acc = mem_gather(m.addr, m.dtype, m.flags, off, sl.nvp, acc);
            continue;
          } else {
            mem_load(m, off, sl, src);
            if (op == VOP_BINF && (imm & VI_PRE_SREG)) {  // an S-register binary in front, while the operand is on its way
              const float pv = sreg_read(sr, (imm >> 8) & 0xffu);
              switch (imm & 0x3fu) {
                case VB_ADD: FOR_U acc.v[u] = acc.v[u] + pv; break;
                case VB_SUB: FOR_U acc.v[u] = acc.v[u] - pv; break;
                case VB_RSUB: FOR_U acc.v[u] = pv - acc.v[u]; break;
                default: FOR_U acc.v[u] = acc.v[u] * pv; break;
              }
              apply_rnd(acc, (imm >> 16) & 0x3u);
            }
          }
        } else if (kind == VK_SREG) {
          const float v = sreg_read(sr, a);
          FOR_U src.v[u] = v;
        } else if (kind == VK_IMM) {
          const float v = __uint_as_float(imm);
          FOR_U src.v[u] = v;
        } else if (kind == VK_REG) {
          vreg_load(planes, a, sub >> 6, nthreads, tid, src);
        } else {
          src = acc;
        }
        switch (op) {
          case VOP_BINF: {
            switch (sub & 0x3fu) {
              case VB_ADD: FOR_U acc.v[u] = acc.v[u] + src.v[u]; break;
              case VB_SUB: FOR_U acc.v[u] = acc.v[u] - src.v[u]; break;
              case VB_RSUB: FOR_U acc.v[u] = src.v[u] - acc.v[u]; break;
              case VB_MUL: FOR_U acc.v[u] = acc.v[u] * src.v[u]; break;
              case VB_DIV: FOR_U acc.v[u] = acc.v[u] / src.v[u]; break;
              case VB_RDIV: FOR_U acc.v[u] = src.v[u] / acc.v[u]; break;
              // on NaN the second operand wins, as in the reference functors (src/vm_gpu.cu:222-233)
              case VB_MIN: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] < src.v[u][e] ? acc.v[u][e] : src.v[u][e]; break;
              case VB_MAX: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] > src.v[u][e] ? acc.v[u][e] : src.v[u][e]; break;
              case VB_AND: FOR_U FOR_E acc.v[u][e] = (acc.v[u][e] != 0.0f && src.v[u][e] != 0.0f) ? 1.0f : 0.0f; break;
              case VB_OR: FOR_U FOR_E acc.v[u][e] = (acc.v[u][e] != 0.0f || src.v[u][e] != 0.0f) ? 1.0f : 0.0f; break;
              case VB_POW: FOR_U acc.v[u] = slab_pow(acc.v[u], src.v[u]); break;
              default: FOR_U acc.v[u] = slab_pow(src.v[u], acc.v[u]); break;
            }
            apply_rnd(acc, (w0 >> 20) & 0x3u);
            break;
          }
          case VOP_BINI: {
            switch (sub & 0x3fu) {
              case VBI_ADD: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(acc.v[u][e]) + __float_as_uint(src.v[u][e])); break;
              case VBI_SUB: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(acc.v[u][e]) - __float_as_uint(src.v[u][e])); break;
              case VBI_RSUB: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(src.v[u][e]) - __float_as_uint(acc.v[u][e])); break;
              case VBI_MUL: FOR_U FOR_E acc.v[u][e] = __uint_as_float(__float_as_uint(acc.v[u][e]) * __float_as_uint(src.v[u][e])); break;
              case VBI_MIN: FOR_U FOR_E acc.v[u][e] = __int_as_float(min(__float_as_int(acc.v[u][e]), __float_as_int(src.v[u][e]))); break;
              case VBI_WRAP: FOR_U FOR_E acc.v[u][e] = __int_as_float(wrap_index(__float_as_int(acc.v[u][e]), __float_as_int(src.v[u][e]))); break;
              default: FOR_U FOR_E acc.v[u][e] = __int_as_float(max(__float_as_int(acc.v[u][e]), __float_as_int(src.v[u][e]))); break;
            }
            break;
          }
          case VOP_CMP: {
            switch (sub & 0x3fu) {
              case VCMP_EQ: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] == src.v[u][e] ? 1.0f : 0.0f; break;
              case VCMP_NE: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] != src.v[u][e] ? 1.0f : 0.0f; break;
              case VCMP_GT: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] > src.v[u][e] ? 1.0f : 0.0f; break;
              case VCMP_GE: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] >= src.v[u][e] ? 1.0f : 0.0f; break;
              case VCMP_LT: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] < src.v[u][e] ? 1.0f : 0.0f; break;
              case VCMP_LE: FOR_U FOR_E acc.v[u][e] = acc.v[u][e] <= src.v[u][e] ? 1.0f : 0.0f; break;
              case VCMP_INT + VCMP_EQ: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) == __float_as_int(src.v[u][e]) ? 1 : 0); break;
              case VCMP_INT + VCMP_NE: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) != __float_as_int(src.v[u][e]) ? 1 : 0); break;
              case VCMP_INT + VCMP_GT: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) > __float_as_int(src.v[u][e]) ? 1 : 0); break;
              case VCMP_INT + VCMP_GE: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) >= __float_as_int(src.v[u][e]) ? 1 : 0); break;
              case VCMP_INT + VCMP_LT: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) < __float_as_int(src.v[u][e]) ? 1 : 0); break;
              default: FOR_U FOR_E acc.v[u][e] = __int_as_float(__float_as_int(acc.v[u][e]) <= __float_as_int(src.v[u][e]) ? 1 : 0); break;
            }
            break;
          }
          case VOP_MSK: {
            // 1/0 in either container: a zero has no bits set below the sign
            mask = 0;
            FOR_U FOR_E mask |= ((__float_as_uint(src.v[u][e]) << 1) != 0 ? 1u : 0u) << (u * E + e);
            break;
          }
          default: {  // VOP_MOVM
            FOR_U FOR_E acc.v[u][e] = ((mask >> (u * E + e)) & 1u) ? src.v[u][e] : acc.v[u][e];
            break;
          }
        }
        if constexpr (SCHED == VS_REDX) {
          if (park_slot != 0u) {  // this was the instruction behind a load that parks its round
            vreg_store(keep_lds, park_slot - 1u, park_fmt, nthreads, tid, acc);
            park_slot = 0u;
          }
        }
        continue;
      }

      switch (op) {
        case VOP_LDR:
          vreg_load(planes, a, sub, nthreads, tid, acc);
          break;
        case VOP_LDS: {
          const float v = sreg_read(sr, a);
          FOR_U acc.v[u] = v;
          break;
        }
        case VOP_LDI: {
          const float v = __uint_as_float(imm);
          FOR_U acc.v[u] = v;
          break;
        }
        case VOP_STR:
          vreg_store(planes, a, sub, nthreads, tid, acc);
          break;
        case VOP_STS:
          sreg_write(sr, a, acc.v[0][0]);
          break;
        case VOP_UNI_END: {
          if constexpr (SCHED == VS_REDX) {
            if (fresh(h.team_is_block) != 0u) {
              // what the run produced lives in the first wave's S registers and accumulator: pass it on
              float *box = reinterpret_cast<float *>(lds + kBoxAt) + box_flip * 16u;
              box_flip ^= 1u;
              if (skips_runs == 0u) {  // the first wave; its lanes hold identical values
                *reinterpret_cast<vf4 *>(box) = vf4{sr.s0, sr.s1, sr.s2, sr.s3};
                *reinterpret_cast<vf4 *>(box + 4) = vf4{sr.s4, sr.s5, sr.s6, sr.s7};
                box[8] = acc.v[0][0];
              }
              __syncthreads();
              const vf4 lo = *reinterpret_cast<const vf4 *>(box), hi = *reinterpret_cast<const vf4 *>(box + 4);
              const float av = box[8];
              sr.s0 = lo[0]; sr.s1 = lo[1]; sr.s2 = lo[2]; sr.s3 = lo[3];
              sr.s4 = hi[0]; sr.s5 = hi[1]; sr.s6 = hi[2]; sr.s7 = hi[3];
              FOR_U acc.v[u] = av;
            }
          }
          break;
        }
        case VOP_ST: {
          const VMemDesc m = load_desc(prog32, mem_off, a);
          Offs off;
          Slabs st = sl;
          if (w0 & VI_SAME_OFFS) {
            off = last_off;
          } else {
            if constexpr (SCHED == VS_POINTWISE) {
              FOR_U {
                const uint32_t ku = kidx + u * nthreads;
                off.v[u] = space_offset(ku < h.n_kidx ? ku : 0u, h.kdims, h.n_kdim, m.kstride, true);
              }
            } else {
              const uint64_t koff = space_offset(kvalid ? kidx : 0u, h.kdims, h.n_kdim, m.kstride, !inner_red);
              FOR_U {
                off.v[u] = koff;
                if (in_sweep) {
                  const uint32_t ru = ridx + u * r_step;
                  off.v[u] += space_offset(ru < r_lim ? ru : 0u, h.rdims, h.n_rdim, m.rstride, inner_red);
                }
              }
            }
            last_off = off;
          }
          if constexpr (SCHED != VS_POINTWISE) {
            if (!in_sweep) {  // one lane per output, one slab: never the wide path
              st.nvp = r_local == 0 ? (sl.nvp & 0xfu) : 0u;
              st.uniform = false;
            }
          }
          mem_store(m, off, st, acc);
          break;
        }
        case VOP_UN: {
          switch (sub) {
            case VU_SQRT: FOR_U acc.v[u] = slab_sqrt(acc.v[u]); break;
            case VU_ABS: FOR_U FOR_E acc.v[u][e] = fabsf(acc.v[u][e]); break;
            case VU_LOG: FOR_U acc.v[u] = slab_log(acc.v[u]); break;
            case VU_EXP: FOR_U acc.v[u] = slab_exp(acc.v[u]); break;
            case VU_ISFINITE: FOR_U FOR_E acc.v[u][e] = isfinite(acc.v[u][e]) ? 1.0f : 0.0f; break;
            case VU_ROUND: FOR_U FOR_E acc.v[u][e] = rintf(acc.v[u][e]); break;
            case VU_FLOOR: FOR_U FOR_E acc.v[u][e] = floorf(acc.v[u][e]); break;
            case VU_CEIL: FOR_U FOR_E acc.v[u][e] = ceilf(acc.v[u][e]); break;
            case VU_TRUNC: FOR_U FOR_E acc.v[u][e] = truncf(acc.v[u][e]); break;
            default:  // VU_IABS, wraps for INT32_MIN like the reference (src/vm_gpu.cu:262-266)
              FOR_U FOR_E {
                const uint32_t x = __float_as_uint(acc.v[u][e]);
                acc.v[u][e] = __uint_as_float(static_cast<int32_t>(x) < 0 ? 0u - x : x);
              }
              break;
          }
          apply_rnd(acc, (w0 >> 20) & 0x3u);
          break;
        }
        case VOP_CAST: {
          if (sub == VC_F2I) {
            FOR_U FOR_E acc.v[u][e] = __int_as_float(static_cast<int32_t>(acc.v[u][e]));
          } else if (sub == VC_I2F) {
            FOR_U FOR_E acc.v[u][e] = static_cast<float>(__float_as_int(acc.v[u][e]));
            apply_rnd(acc, (w0 >> 20) & 0x3u);
          } else if (sub == VC_RND) {
            apply_rnd(acc, (w0 >> 20) & 0x3u);
          } else {
            FOR_U FOR_E acc.v[u][e] = acc.v[u][e] != 0.0f ? 1.0f : 0.0f;
          }
          break;
        }
        default:
          break;
      }

      if constexpr (SCHED != VS_POINTWISE) {
        switch (op) {
          case VOP_RED: {
            if (sub & VRF_SQUARE) FOR_U acc.v[u] = acc.v[u] * acc.v[u];  // the emitter fuses only where acc is dead afterwards
            if (sub & VRF_INT) {
              if (a == 0) {
                red_accumulate_int<SCHED>(racc0, sub & 0xfu, acc, sl.nvp);
              } else {
                red_accumulate_int<SCHED>(racc1, sub & 0xfu, acc, sl.nvp);
              }
            } else if (a == 0) {
              red_accumulate<SCHED>(racc0, sub & 0xfu, acc, sl);
              if (sub & VRF_PAIR) {  // the emitter pairs only where acc is dead afterwards
                FOR_U acc.v[u] = acc.v[u] * acc.v[u];
                red_accumulate<SCHED>(racc1, sub & 0xfu, acc, sl);
              }
            } else {
              red_accumulate<SCHED>(racc1, sub & 0xfu, acc, sl);
            }
            break;
          }
          case VOP_SWEEP: {
            in_sweep = true;
            round = 0;
            sweep_pc = pc;
            slot_kinds = imm;
            red_init<SCHED>(racc0, slot_kinds & 0xfu);
            red_init<SCHED>(racc1, (slot_kinds >> 4) & 0xfu);
            sweep_rev = SCHED == VS_REDX && (sub & VSW_REVERSE) != 0;
            ridx = r_base + r_local + (sweep_rev ? (n_rounds - 1u) * r_step * U : 0u);
            break;
          }
          case VOP_FIN: {
            const bool as_int = (sub & VRF_INT) != 0;  // the partial is an int32 value held exactly by the double
            if constexpr (SCHED == VS_REDY) {
              vf8 t;
              FOR_E {
                const double d = a == 0 ? racc0.v[e] : racc1.v[e];
                t[e] = as_int ? __int_as_float(static_cast<int32_t>(d)) : static_cast<float>(d);
              }
              FOR_U acc.v[u] = t;
            } else {
              const double d = a == 0 ? racc0.v[0] : racc1.v[0];
              const float t = as_int ? __int_as_float(static_cast<int32_t>(d)) : static_cast<float>(d);
              FOR_U acc.v[u] = t;
            }
            break;
          }
          default:
            break;
        }

        end_round(ends, op == VOP_SWEEP || ends);
      }
    }
  }
  STAMP();
}

}  // namespace

#if DVM_VEC_U == DVM_VEC_U_WIDE
// the wide build: more registers per lane, so at most 512 lanes per workgroup
extern "C" __global__ void __launch_bounds__(512) dvm_vm_vec_pw_u4(const VmParam p) { vm_vector<VS_POINTWISE>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_vec_rx_u4(const VmParam p) { vm_vector<VS_REDX>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_vec_ry_u4(const VmParam p) { vm_vector<VS_REDY>(p); }
#else
extern "C" __global__ void __launch_bounds__(1024) dvm_vm_vec_pw(const VmParam p) { vm_vector<VS_POINTWISE>(p); }
extern "C" __global__ void __launch_bounds__(1024) dvm_vm_vec_rx(const VmParam p) { vm_vector<VS_REDX>(p); }
// (the schedule that keeps the innermost axis holds one fp64 partial per element and slot and fetches four rounds
// per trip: it takes more registers than 1024 lanes leave, and the host gives it at most 512)
extern "C" __global__ void __launch_bounds__(512) dvm_vm_vec_ry(const VmParam p) { vm_vector<VS_REDY>(p); }
extern "C" __global__ void __launch_bounds__(1024) dvm_vm_vec_rx_parts(const VmParam p) { vm_vector<VS_REDX, true>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_vec_ry_parts(const VmParam p) { vm_vector<VS_REDY, true>(p); }
#endif
