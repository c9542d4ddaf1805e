// gfx950 vector VM, sweep build: programs that reduce the innermost axis (VS_REDX) and whose sweeps are chains
// of float arithmetic behind one load (the normalisations, softmax, plain reduces with consumers) run here.
//
// The generic interpreter (vm_vector.hip) decodes one instruction word per dispatch and per round of a sweep: the
// decode, a tree of scalar compares, costs more issue slots than the sixteen elements a lane then works on. Here
// a sweep is a native loop over its rounds: the opening load, its parked rounds, the valid counts and the walk
// through the reduced index space are handled once per round by straight code, and the instructions of the body run
// in a small loop of their own that knows nothing but the body's vocabulary: no program counter logic, no
// per-output runs, no V registers, no offsets of its own per operand (every operand of a body shares the walk
// through the reduced index space with the load that opens it). Between the sweeps a program only handles one
// value per output; those instructions run on a single float per lane.
//
// The instruction words are the generic interpreter's (isa_gfx950.h): a program flagged VS_SWEEPS gives the same
// bits here as there without the flag (the host sets the flag when every instruction is in this file's
// vocabulary). The program is read from the kernel argument through the scalar cache; nothing is copied to local
// memory first.
//
// Replaces the reference's interpreter loop (src/vm_gpu.cu:1552-1617) and RunOp switch (src/vm_gpu.cu:941-1548)
// for these programs, as vm_vector.hip does for the rest.
#include <type_traits>

#include "vec_common.h"

namespace {

// the program, copied from the kernel argument once per workgroup
__shared__ uint32_t prog_lds[DVM_PARAM_BYTES / 4];

// acc = acc (sub) s with one value s per lane
__device__ __forceinline__ void lane_binary(Acc &acc, uint32_t sub, float s) {
  if (sub == VB_MUL) {
    FOR_U acc.v[u] = acc.v[u] * s;
  } else if (sub == VB_ADD) {
    FOR_U acc.v[u] = acc.v[u] + s;
  } else if (sub == VB_SUB) {
    FOR_U acc.v[u] = acc.v[u] - s;
  } else if (sub == VB_RSUB) {
    FOR_U acc.v[u] = s - acc.v[u];
  } else if (sub == VB_DIV) {
    FOR_U acc.v[u] = acc.v[u] / s;
  } else if (sub == VB_RDIV) {
    FOR_U acc.v[u] = s / acc.v[u];
  } else if (sub == VB_MIN) {
    FOR_U FOR_E acc.v[u][e] = acc.v[u][e] < s ? acc.v[u][e] : s;
  } else {  // VB_MAX
    FOR_U FOR_E acc.v[u][e] = acc.v[u][e] > s ? acc.v[u][e] : s;
  }
}

// acc = acc (sub) src, element by element
__device__ __forceinline__ void slab_binary(Acc &acc, uint32_t sub, const Acc &src) {
  if (sub == VB_MUL) {
    FOR_U acc.v[u] = acc.v[u] * src.v[u];
  } else if (sub == VB_ADD) {
    FOR_U acc.v[u] = acc.v[u] + src.v[u];
  } else if (sub == VB_SUB) {
    FOR_U acc.v[u] = acc.v[u] - src.v[u];
  } else if (sub == VB_RSUB) {
    FOR_U acc.v[u] = src.v[u] - acc.v[u];
  } else if (sub == VB_DIV) {
    FOR_U acc.v[u] = acc.v[u] / src.v[u];
  } else if (sub == VB_RDIV) {
    FOR_U acc.v[u] = src.v[u] / acc.v[u];
  } else if (sub == VB_MIN) {  // on NaN the second operand wins, as in the reference functors (src/vm_gpu.cu:222-233)
    FOR_U FOR_E acc.v[u][e] = acc.v[u][e] < src.v[u][e] ? acc.v[u][e] : src.v[u][e];
  } else {  // VB_MAX
    FOR_U FOR_E acc.v[u][e] = acc.v[u][e] > src.v[u][e] ? acc.v[u][e] : src.v[u][e];
  }
}

// A uniform value as it is now (see fresh() in vec_common.h), also when the compiler holds it in a vector register.
__device__ __forceinline__ uint32_t fresh_s(uint32_t x) {
  uint32_t y = __builtin_amdgcn_readfirstlane(x);
  asm volatile("" : "+s"(y));
  return y;
}

// One reduce step of a round. The guarded form (slabs that are partly valid in some lane) tests every element against
// the lane's valid count; the count passes through an empty assembly statement on that path, or the compiler
// computes those sixteen tests at the top of every round, for the rounds that never take the path as well.
__device__ __forceinline__ void reduce_round(double &r, uint32_t kind, const Acc &x, const Slabs &sl) {
  RedAcc<VS_REDX> t;
  t.v[0] = r;
  if (sl.uniform) {
    red_accumulate<VS_REDX>(t, kind, x, sl);
  } else {
    Slabs guarded = sl;
    asm volatile("" : "+v"(guarded.nvp));
    red_accumulate<VS_REDX>(t, kind, x, guarded);
  }
  r = t.v[0];
}

__device__ __forceinline__ float round_to(float x, uint32_t rnd) {
  return rnd == VRND_F16 ? round_f16(x) : (rnd == VRND_BF16 ? round_bf16(x) : x);
}


template <bool PARTS>
__device__ __forceinline__ void vm_vector_sweeps(const VmParam &p) {
#ifdef DVM_VEC_STAMPS
  const uint64_t stamp_base = p.w[DVM_PARAM_WORDS - 1];  // (a scalar load from the kernel argument)
  uint32_t stamp_n = 0;
#endif
  // The blob arrives as a kernel argument, and that segment may live in host memory, uncached: every scalar load
  // from it is then a trip over the bus (0.8 us measured per instruction word read that way). So the workgroup
  // copies the words the program occupies into local memory once, in one trip, and decodes from there.
  {
    const uint32_t *src = reinterpret_cast<const uint32_t *>(p.w);
    const VVecHeader *hp = reinterpret_cast<const VVecHeader *>(p.w);
    uint32_t used = (hp->code_off + hp->n_code) * 2;
    used = used < DVM_PARAM_BYTES / 4 ? used : DVM_PARAM_BYTES / 4;
    const uint32_t trips = (used + blockDim.x - 1) / blockDim.x;
    for (uint32_t t = 0; t < trips; ++t) {  // uniform trip count, clamped indices: no per-lane branch
      uint32_t i = t * blockDim.x + threadIdx.x;
      i = i < used ? i : used - 1;
      prog_lds[i] = src[i];
    }
    __syncthreads();
  }
  STAMP();
  // (No index is clamped: the launch checks that the tables lie inside the blob, that every operand index names a
  // descriptor and that every sweep's body ends before the program does.)
  const vu2 *prog64 = reinterpret_cast<const vu2 *>(prog_lds);
  auto word32 = [&](uint32_t i) -> uint32_t { return uni(prog_lds[i]); };  // 32-bit word i of the blob
  // Header fields the rounds of a sweep need stay in scalar registers; the others are read where they are used
  // (HDR_NOW: the index passes through an empty assembly statement, so the compiler cannot move the read to the top
  // of the kernel and keep its result alive through every loop: scalar registers are what this kernel runs out of).
#define HDR(field) word32(static_cast<uint32_t>(offsetof(VVecHeader, field) / 4))
#define HDR_NOW(field) word32(fresh_s(static_cast<uint32_t>(offsetof(VVecHeader, field) / 4)))
  const uint32_t n_rdim = HDR(n_rdim);
  const uint32_t n_ridx = HDR(n_ridx), inner_extent = HDR(inner_extent);
  const uint32_t mem_off = HDR(mem_off), code_off = HDR(code_off);
  // the first axis of the reduced index space (the host gives this build programs of at most two kept and two reduced axes)
  const uint32_t rd_extent = HDR(rdims[0].extent), rd_magic = HDR(rdims[0].magic), rd_shift = HDR(rdims[0].shift);
  auto code_at = [&](uint32_t pc) -> vu2 {  // (the caller makes the halves uniform where it branches on them)
    return prog64[code_off + pc];
  };
  // A memory operand's descriptor. Only what the kernel branches on (element type, flags) is made wave-uniform: the
  // address and the strides only ever enter per-lane arithmetic, where a copy in every lane serves as well.
  struct Desc {
    uint64_t addr;
    uint32_t dtype, flags, ks0, ks1, rs0, rs1;
  };
  auto desc_at = [&](uint32_t idx) -> Desc {
    const vu4 *dq = reinterpret_cast<const vu4 *>(prog_lds + 2u * (mem_off + idx * static_cast<uint32_t>(sizeof(VMemDesc) / 8)));
    const vu4 q0 = dq[0], q1 = dq[1], q2 = dq[2];
    Desc d;
    d.addr = static_cast<uint64_t>(q0[0]) | (static_cast<uint64_t>(q0[1]) << 32);
    d.dtype = uni(q0[2]);
    d.flags = uni(q0[3]);
    d.ks0 = q1[0];
    d.ks1 = q1[1];
    d.rs0 = q2[0];
    d.rs1 = q2[1];
    return d;
  };

  const uint32_t tid = threadIdx.x;
  const uint32_t nthreads = blockDim.x;
  // per-team runs (VOP_UNI_BEGIN .. VOP_UNI_END) are computed by the first wave when the team is the workgroup
  uint32_t skips_runs, k_local, r_local, k_per_wg, r_step;
  {
    const uint32_t tlog = HDR_NOW(team_log2);
    const bool team_is_block = HDR_NOW(team_is_block) != 0u;
    skips_runs = (team_is_block && uni(tid >> 6) != 0u) ? 1u : 0u;
    if (team_is_block) {
      k_local = 0; r_local = tid; k_per_wg = 1; r_step = nthreads;
    } else {
      k_local = tid >> tlog; r_local = tid & ((1u << tlog) - 1u); k_per_wg = nthreads >> tlog; r_step = 1u << tlog;
    }
  }
  vf4 *keep_lds = reinterpret_cast<vf4 *>(lds + nthreads) + HDR_NOW(n_vslot) * U * nthreads;  // rounds parked by VI_LD_KEEP_WR
  const uint32_t r_span = PARTS ? HDR(r_chunk) : n_ridx;
  const uint32_t n_rounds = (r_span + r_step * U - 1) / (r_step * U);

  SRegs sr;
  sr.s0 = sr.s1 = sr.s2 = sr.s3 = sr.s4 = sr.s5 = sr.s6 = sr.s7 = 0.0f;
  auto sreg_get = [&](uint32_t i) -> float { return sreg_read(sr, i); };
  double racc0 = 0.0, racc1 = 0.0;
  uint32_t red_flip = 0, box_flip = 0;

  for (uint32_t item = blockIdx.x; item < HDR_NOW(n_items); item += gridDim.x) {
    const uint32_t kidx = item * k_per_wg + k_local;
    const bool kvalid = kidx < HDR_NOW(n_kidx);
    const uint32_t kpos = kvalid ? kidx : 0u;
    uint32_t r_base = 0, r_lim = n_ridx;
    if constexpr (PARTS) {
      r_base = (kidx / HDR_NOW(k_per_chunk)) * HDR_NOW(r_chunk);
      r_lim = (r_base + r_span < n_ridx) ? r_base + r_span : n_ridx;
    }
    // the lane's element offset along the kept axes (one or two of them)
    uint32_t kc0 = kpos, kc1 = 0;
    if (HDR_NOW(n_kdim) > 1u) {
      kc1 = (__umulhi(kpos, HDR_NOW(kdims[0].magic)) + kpos) >> HDR_NOW(kdims[0].shift);
      kc0 = kpos - kc1 * HDR_NOW(kdims[0].extent);
    }
    auto kept_offset = [&](const Desc &m) -> uint64_t {
      return static_cast<uint64_t>(kc0) * m.ks0 + static_cast<uint64_t>(kc1) * m.ks1;
    };

    float x = 0.0f;     // the accumulator between sweeps: one value per lane
    bool xmask = false; // the predicate of VOP_MSK between sweeps
    uint64_t last_koff = 0;
    uint32_t pc = 0;
    vu2 fetched = code_at(0);
    while (true) {
      const uint32_t w0 = uni(fetched[0]), imm = uni(fetched[1]);
      const uint32_t op = w0 & 0x7fu;
      if (op == VOP_END) break;
      const uint32_t sub = (w0 >> 8) & 0xffu, a = w0 >> 24, kind = (w0 >> 16) & 0xfu, rnd = (w0 >> 20) & 0x3u;

      if (op != VOP_SWEEP) {
        // ---- one value per lane ----
#ifdef DVM_VEC_STAMPS_FINE
        STAMP();
#endif
        pc += (op == VOP_UNI_BEGIN && skips_runs != 0u) ? imm : 1u;  // (the waves that skip a run go on at its VOP_UNI_END)
        fetched = code_at(pc);
        if (op >= VOP_SRC_BASE) {
          float sv;
          if (kind == VK_MEM) {
            const Desc m = desc_at(a);
            if (!(w0 & VI_SAME_OFFS)) {
              const uint64_t koff = kept_offset(m);
              if (!(w0 & VI_OFFS_ASIDE) || op == VOP_LD) last_koff = koff;
              const float v = elem_load(m.addr, m.dtype, koff);
              sv = kvalid ? v : 0.0f;
            } else {
              const float v = elem_load(m.addr, m.dtype, last_koff);
              sv = kvalid ? v : 0.0f;
            }
          } else {
            sv = kind == VK_IMM ? __uint_as_float(imm) : (kind == VK_ACC ? x : sreg_get(a));
          }
          if (op == VOP_LD) {
            x = sv;
          } else if (op == VOP_MSK) {
            xmask = (__float_as_uint(sv) << 1) != 0u;
          } else if (op == VOP_MOVM) {
            x = xmask ? sv : x;
          } else {
            x = uniform_binary(op, sub, x, sv);
            if (op == VOP_BINF) {
              x = round_to(x, rnd);
              if (kind == VK_SREG2) {
                x = uniform_binary(VOP_BINF, imm & 0x3fu, x, sreg_get((imm >> 8) & 0xffu));
                x = round_to(x, (imm >> 16) & 0x3u);
              }
            }
          }
          continue;
        }
        switch (op) {
          case VOP_FIN: {
            const double d = a == 0 ? racc0 : racc1;
            x = (sub & VRF_INT) ? __int_as_float(static_cast<int32_t>(d)) : static_cast<float>(d);
            break;
          }
          case VOP_LDS: x = sreg_get(a); break;
          case VOP_LDI: x = __uint_as_float(imm); break;
          case VOP_STS: sreg_write(sr, a, x); break;
          case VOP_UN:  // (square root and logarithm in line: the out-of-line forms save registers to scratch memory around the call)
            x = round_to(sub == VU_SQRT ? sqrtf(x) : (sub == VU_LOG ? logf(x) : uniform_unary(sub, x)), rnd);
            break;
          case VOP_CAST: {
            x = uniform_cast(sub, x);
            if (sub == VC_I2F || sub == VC_RND) x = round_to(x, rnd);
            break;
          }
          case VOP_ST: {  // one lane per output
            const Desc m = desc_at(a);
            if (!(w0 & VI_SAME_OFFS)) last_koff = kept_offset(m);
            Offs off;
            FOR_U off.v[u] = last_koff;
            Acc out;
            FOR_U out.v[u] = x;
            mem_store_slow(m.addr, m.dtype, m.flags & ~static_cast<uint32_t>(VMF_VEC | VMF_GATHER), off, (kvalid && r_local == 0u) ? 1u : 0u, out);
            break;
          }
          case VOP_UNI_END: {
            if (HDR_NOW(team_is_block) != 0u) {
              // what the run produced lives in the first wave's S registers and accumulator: pass it on
              float *box = reinterpret_cast<float *>(lds + kBoxAt) + box_flip * 16u;
              box_flip ^= 1u;
              if (skips_runs == 0u) {
                *reinterpret_cast<vf4 *>(box) = vf4{sr.s0, sr.s1, sr.s2, sr.s3};
                *reinterpret_cast<vf4 *>(box + 4) = vf4{sr.s4, sr.s5, sr.s6, sr.s7};
                box[8] = x;
              }
              __syncthreads();
              const vf4 lo = *reinterpret_cast<const vf4 *>(box), hi = *reinterpret_cast<const vf4 *>(box + 4);
              x = box[8];
              sr.s0 = lo[0]; sr.s1 = lo[1]; sr.s2 = lo[2]; sr.s3 = lo[3];
              sr.s4 = hi[0]; sr.s5 = hi[1]; sr.s6 = hi[2]; sr.s7 = hi[3];
            }
            break;
          }
          default:  // VOP_UNI_BEGIN, VOP_ENDSWEEP (of a sweep the host has emptied)
            break;
        }
        continue;
      }

      // ---- a sweep: a native loop over its rounds ----
      STAMP();
      const uint32_t slot_kinds = imm;
      const uint32_t k0 = slot_kinds & 0xfu, k1 = (slot_kinds >> 4) & 0xfu;
      const bool rev = (sub & VSW_REVERSE) != 0;
      vu2 ldw = code_at(pc + 1u);  // the VOP_LD that opens the body
      ldw[0] = uni(ldw[0]);
      ldw[1] = uni(ldw[1]);
      const uint32_t body_pc = pc + 2u;
      // the opening load's operand; every other operand of the body walks the reduced axes as it does, or not at all
      const Desc ma = desc_at(ldw[0] >> 24);
      const uint64_t a_koff = kept_offset(ma);
      const uint32_t rs0 = ma.rs0, rs1 = ma.rs1;
      // the first instruction's operand rides with the opening load when both can take the wide path
      constexpr uint32_t kFast = VMF_VEC | VMF_ALIGNED;
      vu2 first_w = code_at(body_pc);
      first_w[0] = uni(first_w[0]);
      first_w[1] = uni(first_w[1]);
      uint32_t pair0 = ((first_w[0] & 0x7fu) == VOP_BINF && ((first_w[0] >> 16) & 0xfu) == VK_MEM && (first_w[0] & VI_SAME_OFFS) != 0 &&
                        !(first_w[1] & VI_PRE_SREG) && (ma.flags & kFast) == kFast) ? 1u : 0u;
      Desc mb = ma;
      if (pair0 != 0u) {
        mb = desc_at(first_w[0] >> 24);
        pair0 = (mb.flags & kFast) == kFast ? 1u : 0u;
      }
      auto as_mem = [&](const Desc &d) -> VMemDesc {
        VMemDesc m;
        m.addr = d.addr;
        m.dtype = d.dtype;
        m.flags = d.flags;
        return m;
      };

      racc0 = red_identity(k0 <= VR_MIN ? k0 : VR_SUM);
      racc1 = red_identity(k1 <= VR_MIN ? k1 : VR_SUM);

      uint32_t body_end = body_pc;  // index behind the instruction that closes the round (known after the first round)
      // One round. INTERIOR: every slab of every lane of the wave is full (all rounds of a sweep but the last one or
      // two): the valid counts are constants there, and with them every test of them in the loads, stores and reduces.
      auto do_round = [&](auto interior_tag, uint32_t lr, uint32_t ridx) {
        constexpr bool INTERIOR = decltype(interior_tag)::value;
        Slabs sl;
        Offs roff;
        if constexpr (INTERIOR) {
          sl.nvp = kAllFull;
          sl.full = (1u << U) - 1u;
          sl.uniform = true;
          FOR_U {
            const uint32_t rc = ridx + u * r_step;
            uint32_t c0 = rc, c1 = 0;
            if (n_rdim > 1u) {
              c1 = (__umulhi(rc, rd_magic) + rc) >> rd_shift;
              c0 = rc - c1 * rd_extent;
            }
            roff.v[u] = (static_cast<uint64_t>(c0) * rs0) * static_cast<uint32_t>(E) + static_cast<uint64_t>(c1) * rs1;
          }
        } else {
          // valid counts and the walk through the reduced index space, per slab
          uint32_t nvp = 0;
          FOR_U {
            const uint32_t ru = ridx + u * r_step;
            const bool ok = kvalid && ru < r_lim;
            const uint32_t rc = ok ? ru : 0u;
            uint32_t c0 = rc, c1 = 0;  // coordinates along the one or two reduced axes; the first counts groups of E
            if (n_rdim > 1u) {
              c1 = (__umulhi(rc, rd_magic) + rc) >> rd_shift;
              c0 = rc - c1 * rd_extent;
            }
            const uint32_t left = inner_extent - c0 * E;
            uint32_t nv = left < static_cast<uint32_t>(E) ? left : static_cast<uint32_t>(E);
            nv &= ok ? 0xfu : 0u;
            nvp |= nv << (4 * u);
            roff.v[u] = (static_cast<uint64_t>(c0) * rs0) * static_cast<uint32_t>(E) + static_cast<uint64_t>(c1) * rs1;
          }
          sl = slab_state(nvp);
        }
        auto offsets_of = [&](const Desc &d) -> Offs {
          const uint64_t koff = kept_offset(d);
          const bool walks = (d.rs0 | d.rs1) != 0u;
          Offs o;
          FOR_U o.v[u] = koff + (walks ? roff.v[u] : 0ull);
          return o;
        };

        // What the rounds have in common is tested where it is used, on values the compiler takes for new each
        // round (fresh_s): tests moved in front of the loop would each keep a pair of scalar registers busy.
        const uint32_t l0 = fresh_s(ldw[0]), l1 = fresh_s(ldw[1]);
        const bool keep_wr = (l0 & VI_LD_KEEP_WR) != 0, keep_rd = (l0 & VI_LD_KEEP_RD) != 0;
        const uint32_t n_parked = (l0 & (VI_LD_KEEP_WR | VI_LD_KEEP_RD)) ? (l1 & 0xffffu) : 0u;
        const uint32_t keep_prefix = (l1 >> 16) & 0x3u, keep_fmt = (l1 >> 20) & 0x3u;
        Desc da = ma, db = mb;
        da.dtype = fresh_s(ma.dtype);
        da.flags = fresh_s(ma.flags);
        db.dtype = fresh_s(mb.dtype);

        Acc acc, operand;
        const bool parked = lr < n_parked;
        const uint32_t keep_at = keep_fmt == VF_F32 ? 2u * lr : lr;  // fp32 values take two planes per slab
        uint32_t bpc = body_pc;
        bool have_operand = false;  // the first instruction's operand is in `operand` already
        if (parked && keep_rd) {
          bpc += keep_prefix;  // what was parked is the value behind the first keep_prefix instructions
          // The round starts from local memory; when the first instruction it executes fetches a memory operand (the
          // weight row of a normalisation), that trip starts first and the parked slabs are unpacked under it.
          const vu2 ahead = code_at(bpc);
          const uint32_t aw = uni(ahead[0]);
          if ((aw & 0x7fu) == VOP_BINF && ((aw >> 16) & 0xfu) == VK_MEM) {
            const Desc d = desc_at(aw >> 24);
            mem_load(as_mem(d), offsets_of(d), sl, operand);
            have_operand = true;
          }
          vreg_load(keep_lds, keep_at, keep_fmt, nthreads, tid, acc);
        } else {
          Offs off;
          FOR_U off.v[u] = a_koff + roff.v[u];
          if (fresh_s(pair0) != 0u && sl.uniform) {
            mem_load2_wide(as_mem(da), as_mem(db), off, sl.full, acc, operand);
            have_operand = true;
          } else {
            mem_load(as_mem(da), off, sl, acc);
          }
          if (parked && keep_wr && keep_prefix == 0u) vreg_store(keep_lds, keep_at, keep_fmt, nthreads, tid, acc);
        }
        bool park_next = parked && keep_wr && !keep_rd && keep_prefix != 0u;  // the value behind the first instruction is what this round parks

        vu2 bfetched = code_at(bpc);
        while (true) {
          const uint32_t w = uni(bfetched[0]), bimm = uni(bfetched[1]);
          ++bpc;
          bfetched = code_at(bpc);
          const uint32_t bop = w & 0x7fu, bsub = (w >> 8) & 0xffu, bk = (w >> 16) & 0xfu, brnd = (w >> 20) & 0x3u, ba = w >> 24;
          if (bop == VOP_BINF) {
            if (bk == VK_MEM) {
              if (!have_operand) {
                const Desc d = desc_at(ba);
                mem_load(as_mem(d), offsets_of(d), sl, operand);
              }
              have_operand = false;
              if (bimm & VI_PRE_SREG) {  // an S-register binary in front, while the operand is on its way
                lane_binary(acc, bimm & 0x3fu, sreg_get((bimm >> 8) & 0xffu));
                apply_rnd(acc, (bimm >> 16) & 0x3u);
              }
              slab_binary(acc, bsub & 0x3fu, operand);
              apply_rnd(acc, brnd);
            } else if (bk == VK_ACC) {
              operand = acc;
              slab_binary(acc, bsub & 0x3fu, operand);
              apply_rnd(acc, brnd);
            } else {
              lane_binary(acc, bsub & 0x3fu, bk == VK_IMM ? __uint_as_float(bimm) : sreg_get(ba));
              apply_rnd(acc, brnd);
              if (bk == VK_SREG2) {
                lane_binary(acc, bimm & 0x3fu, sreg_get((bimm >> 8) & 0xffu));
                apply_rnd(acc, (bimm >> 16) & 0x3u);
              }
            }
          } else if (bop == VOP_RED) {
            if (bsub & VRF_SQUARE) FOR_U acc.v[u] = acc.v[u] * acc.v[u];
            if (ba == 0u) {
              reduce_round(racc0, bsub & 0xfu, acc, sl);
              if (bsub & VRF_PAIR) {
                FOR_U acc.v[u] = acc.v[u] * acc.v[u];
                reduce_round(racc1, bsub & 0xfu, acc, sl);
              }
            } else {
              reduce_round(racc1, bsub & 0xfu, acc, sl);
            }
          } else if (bop == VOP_ST) {
            const Desc d = desc_at(ba);
            mem_store(as_mem(d), offsets_of(d), sl, acc);
          } else if (bop == VOP_LD) {  // another operand's round (two reduces of two inputs in one sweep)
            const Desc d = desc_at(ba);
            mem_load(as_mem(d), offsets_of(d), sl, acc);
          } else if (bop == VOP_UN) {
            switch (bsub) {
              case VU_EXP: FOR_U acc.v[u] = slab_exp(acc.v[u]); break;
              case VU_ABS: FOR_U FOR_E acc.v[u][e] = fabsf(acc.v[u][e]); break;
              case VU_SQRT: FOR_U acc.v[u] = slab_sqrt(acc.v[u]); break;
              case VU_LOG: FOR_U acc.v[u] = slab_log(acc.v[u]); break;
              case VU_ISFINITE: FOR_U FOR_E acc.v[u][e] = isfinite(acc.v[u][e]) ? 1.0f : 0.0f; break;
              case VU_ROUND: FOR_U FOR_E acc.v[u][e] = rintf(acc.v[u][e]); break;
              case VU_FLOOR: FOR_U FOR_E acc.v[u][e] = floorf(acc.v[u][e]); break;
              case VU_CEIL: FOR_U FOR_E acc.v[u][e] = ceilf(acc.v[u][e]); break;
              default: FOR_U FOR_E acc.v[u][e] = truncf(acc.v[u][e]); break;
            }
            apply_rnd(acc, brnd);
          } else if (bop == VOP_CAST) {  // VC_RND
            apply_rnd(acc, brnd);
          }
          if (park_next) {
            vreg_store(keep_lds, keep_at, keep_fmt, nthreads, tid, acc);
            park_next = false;
          }
          if (w & VI_ENDS) break;
        }
        body_end = bpc;
      };

      // A statistics sweep (the body is one float reduce) takes two interior rounds per trip to memory: the second
      // round's slabs land in the registers an operand would use, and both rounds are reduced in their order.
      const bool two_per_trip = (first_w[0] & 0x7fu) == VOP_RED && (first_w[0] & VI_ENDS) != 0u && (ldw[0] & VI_LD_KEEP_RD) == 0u &&
                                (ma.flags & kFast) == kFast;
      auto do_two_rounds = [&](uint32_t lr, uint32_t ridx, uint32_t lr2, uint32_t ridx2) {
        auto walk = [&](uint32_t at) -> Offs {
          Offs o;
          FOR_U {
            const uint32_t rc = at + u * r_step;
            uint32_t c0 = rc, c1 = 0;
            if (n_rdim > 1u) {
              c1 = (__umulhi(rc, rd_magic) + rc) >> rd_shift;
              c0 = rc - c1 * rd_extent;
            }
            o.v[u] = a_koff + (static_cast<uint64_t>(c0) * rs0) * static_cast<uint32_t>(E) + static_cast<uint64_t>(c1) * rs1;
          }
          return o;
        };
        Slabs sl;
        sl.nvp = kAllFull;
        sl.full = (1u << U) - 1u;
        sl.uniform = true;
        Desc da = ma;
        da.dtype = fresh_s(ma.dtype);
        Acc x0, x1;
        mem_load_wide_2rounds(as_mem(da), walk(ridx), walk(ridx2), sl.full, sl.full, x0, x1);
        const uint32_t l0 = fresh_s(ldw[0]), l1 = fresh_s(ldw[1]);
        if (l0 & VI_LD_KEEP_WR) {  // (a load with a reduce behind it parks what it loaded: no prefix)
          const uint32_t n_parked = l1 & 0xffffu, fmt = (l1 >> 20) & 0x3u;
          if (lr < n_parked) vreg_store(keep_lds, fmt == VF_F32 ? 2u * lr : lr, fmt, nthreads, tid, x0);
          if (lr2 < n_parked) vreg_store(keep_lds, fmt == VF_F32 ? 2u * lr2 : lr2, fmt, nthreads, tid, x1);
        }
        const uint32_t w = fresh_s(first_w[0]);
        const uint32_t bsub = (w >> 8) & 0xffu;
        auto reduce_into_slots = [&](Acc &x) {
          if (bsub & VRF_SQUARE) FOR_U x.v[u] = x.v[u] * x.v[u];
          if ((w >> 24) == 0u) {
            reduce_round(racc0, bsub & 0xfu, x, sl);
            if (bsub & VRF_PAIR) {
              FOR_U x.v[u] = x.v[u] * x.v[u];
              reduce_round(racc1, bsub & 0xfu, x, sl);
            }
          } else {
            reduce_round(racc1, bsub & 0xfu, x, sl);
          }
        };
        reduce_into_slots(x0);
        reduce_into_slots(x1);
        body_end = body_pc + 1u;
      };

      const bool whole_groups = (inner_extent & (E - 1u)) == 0u;
      for (uint32_t round = 0; round < n_rounds; ++round) {
        const uint32_t lr = rev ? n_rounds - 1u - round : round;
        const uint32_t ridx = r_base + r_local + lr * r_step * U;
        // (the last slab of the lane decides: the indices of a lane's slabs ascend)
        const bool lane_full = kvalid && ridx + (U - 1u) * r_step < r_lim;
        if (whole_groups && wave_all(lane_full)) {
          if (two_per_trip && round + 1u < n_rounds) {
            const uint32_t lr2 = rev ? lr - 1u : lr + 1u;
            const uint32_t ridx2 = r_base + r_local + lr2 * r_step * U;
            if (wave_all(kvalid && ridx2 + (U - 1u) * r_step < r_lim)) {
              do_two_rounds(lr, ridx, lr2, ridx2);
              ++round;
              continue;
            }
          }
          do_round(std::true_type{}, lr, ridx);
        } else {
          do_round(std::false_type{}, lr, ridx);
        }
      }
      pc = body_end;
      fetched = code_at(pc);
      STAMP();
      if (k0 <= VR_MIN || k1 <= VR_MIN) {
        red_finish_x(racc0, racc1, k0, k1, HDR_NOW(team_log2), HDR_NOW(team_is_block) != 0u, tid, nthreads, red_flip, lds);
      }
      STAMP();
    }
  }
  STAMP();
}
#undef STAMP

#undef HDR
#undef HDR_NOW

}  // namespace

extern "C" __global__ void __launch_bounds__(1024) dvm_vm_vec_rx_sw(const VmParam p) { vm_vector_sweeps<false>(p); }
extern "C" __global__ void __launch_bounds__(1024) dvm_vm_vec_rx_sw_parts(const VmParam p) { vm_vector_sweeps<true>(p); }
