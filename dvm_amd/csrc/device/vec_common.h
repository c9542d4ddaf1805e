// Helpers shared by the vector VM kernels (vm_vector.hip, vm_vector_sweep.hip): element and slab accesses to memory
// operands, reduce partials and their combination across lanes, S and V registers, index arithmetic, and the
// arithmetic of instructions that work on one value per lane.
#ifndef DVM_DEVICE_VEC_COMMON_H_
#define DVM_DEVICE_VEC_COMMON_H_
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../isa_gfx950.h"

namespace {

constexpr int E = DVM_VEC_E;
constexpr int U = DVM_VEC_U;

typedef float vf8 __attribute__((ext_vector_type(8)));
typedef float vf4 __attribute__((ext_vector_type(4)));
typedef uint32_t vu4 __attribute__((ext_vector_type(4)));
typedef uint32_t vu2 __attribute__((ext_vector_type(2)));
typedef _Float16 vh8 __attribute__((ext_vector_type(8)));

#define DVM_GLOBAL __attribute__((address_space(1)))

// dynamic local memory of a workgroup (reduce partials and hand-over boxes, V registers, parked rounds; laid out by the host)
extern __shared__ double lds[];
#define FOR_U _Pragma("unroll") for (int u = 0; u < U; ++u)
#define FOR_E _Pragma("unroll") for (int e = 0; e < E; ++e)

struct Acc {
  vf8 v[U];
};

// packed per-slab valid counts: 4 bits per slab
constexpr uint32_t kAllOnes = U == 4 ? 0x1111u : (U == 2 ? 0x11u : 0x1u);
constexpr uint32_t kAllFull = kAllOnes * 8u;

__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
// Arguments of an out-of-line function arrive in vector registers even when every lane holds the same value;
// reading them back through the first lane lets the function branch on them with scalar branches.
__device__ __forceinline__ uint64_t uni64(uint64_t v) {
  return (static_cast<uint64_t>(uni(static_cast<uint32_t>(v >> 32))) << 32) | uni(static_cast<uint32_t>(v));
}

__device__ __forceinline__ uint32_t fast_div(uint32_t n, const VDim &d) { return (__umulhi(n, d.magic) + n) >> d.shift; }

__device__ __forceinline__ float round_f16(float x) { return static_cast<float>(static_cast<_Float16>(x)); }

// gfx950 converts fp32 to bf16 in hardware (round to nearest even, NaN stays NaN): v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float x) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x)); }
__device__ __forceinline__ float round_bf16(float x) { return static_cast<float>(static_cast<__bf16>(x)); }
typedef float vf2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const vf2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ void apply_rnd(Acc &a, uint32_t rnd) {
  if (rnd == VRND_NONE) return;
  if (rnd == VRND_F16) {
    FOR_U FOR_E a.v[u][e] = round_f16(a.v[u][e]);
  } else {
    FOR_U FOR_E a.v[u][e] = round_bf16(a.v[u][e]);
  }
}

// Library functions with internal (per-lane) branches stay out of the interpreter loop.
// exp(x) = exp2(x * log2(e)) with the product carried in two floats (the rounding of a single product would cost
// |x| * 2^-24 of relative accuracy: 80 units in the last place at x = 88) and v_exp_f32 for the power: about one and a
// half units in the last place, no branches, a dozen instructions an element where the library call took twenty plus
// the call. Results below the smallest normal number come out as 0 (v_exp_f32 has no denormal results), +-inf and NaN
// as they should.
__device__ __forceinline__ float exp_f32(float x) {
  const float kLog2eHi = 1.44269502162933349609375f, kLog2eLo = 1.925963033500011e-08f, kLn2 = 0.693147182464599609375f;
  const float hi = x * kLog2eHi;
  float lo = __builtin_fmaf(x, kLog2eLo, __builtin_fmaf(x, kLog2eHi, -hi));
  // (inf - inf above when the product overflows, which a finite x beyond 2.4e38 does as well as an infinite one:
  // the lowest float a masked softmax fills in)
  lo = __builtin_fabsf(hi) < __builtin_huge_valf() ? lo : 0.0f;
  const float p = __builtin_amdgcn_exp2f(hi);
  return p < __builtin_huge_valf() ? __builtin_fmaf(p * kLn2, lo, p) : p;  // (inf * lo; a NaN passes through)
}
__device__ __forceinline__ vf8 slab_exp(vf8 x) {
  FOR_E x[e] = exp_f32(x[e]);
  return x;
}
__device__ __attribute__((noinline)) vf8 slab_log(vf8 x) {
  FOR_E x[e] = logf(x[e]);
  return x;
}
__device__ __attribute__((noinline)) vf8 slab_pow(vf8 x, vf8 y) {
  FOR_E x[e] = powf(x[e], y[e]);
  return x;
}
__device__ __attribute__((noinline)) vf8 slab_sqrt(vf8 x) {
  FOR_E x[e] = sqrtf(x[e]);
  return x;
}

// ---- memory operands -------------------------------------------------------

__device__ __forceinline__ float elem_load(uint64_t base, uint32_t dtype, uint64_t off) {
  switch (dtype) {
    case VDT_F32:
      return reinterpret_cast<const DVM_GLOBAL float *>(base)[off];
    case VDT_I32:
      return __int_as_float(reinterpret_cast<const DVM_GLOBAL int32_t *>(base)[off]);
    case VDT_F16:
      return static_cast<float>(reinterpret_cast<const DVM_GLOBAL _Float16 *>(base)[off]);
    case VDT_BF16:
      return __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const DVM_GLOBAL uint16_t *>(base)[off]) << 16);
    case VDT_IOTA:  // no memory: the element is its own offset
      return __int_as_float(static_cast<int32_t>(base + off));
    default:  // VDT_BOOL
      return reinterpret_cast<const DVM_GLOBAL uint8_t *>(base)[off] != 0 ? 1.0f : 0.0f;
  }
}

__device__ __forceinline__ void elem_store(uint64_t base, uint32_t dtype, uint64_t off, float v) {
  switch (dtype) {
    case VDT_F32:
      reinterpret_cast<DVM_GLOBAL float *>(base)[off] = v;
      break;
    case VDT_I32:
      reinterpret_cast<DVM_GLOBAL int32_t *>(base)[off] = __float_as_int(v);
      break;
    case VDT_F16:
      reinterpret_cast<DVM_GLOBAL _Float16 *>(base)[off] = static_cast<_Float16>(v);
      break;
    case VDT_BF16:
      reinterpret_cast<DVM_GLOBAL uint16_t *>(base)[off] = static_cast<uint16_t>(f32_to_bf16_bits(v));
      break;
    case VDT_IOTA:  // (nothing to write to; the launch refuses such programs)
      break;
    default:
      reinterpret_cast<DVM_GLOBAL uint8_t *>(base)[off] = v != 0.0f ? 1 : 0;
      break;
  }
}

// Slow path of a slab: scalar per-element accesses (ragged tail, unaligned rows, stride-0 operand).
__device__ __forceinline__ vf8 slab_load_slow(const VMemDesc &m, uint64_t off, int nv) {
  vf8 out = 0.0f;
  if (m.flags & VMF_GATHER) {
    const uint64_t step = m.flags >> 8;
    FOR_E {
      if (e < nv) out[e] = elem_load(m.addr, m.dtype, off + e * step);
    }
    return out;
  }
  if (!(m.flags & VMF_VEC)) {
    out = elem_load(m.addr, m.dtype, off);
    return out;
  }
  FOR_E {
    if (e < nv) out[e] = elem_load(m.addr, m.dtype, off + e);
  }
  return out;
}

__device__ __forceinline__ void slab_store_slow(const VMemDesc &m, uint64_t off, int nv, vf8 in) {
  if (m.flags & VMF_GATHER) {
    const uint64_t step = m.flags >> 8;
    FOR_E {
      if (e < nv) elem_store(m.addr, m.dtype, off + e * step, in[e]);
    }
    return;
  }
  if (!(m.flags & VMF_VEC)) {
    elem_store(m.addr, m.dtype, off, in[0]);
    return;
  }
  FOR_E {
    if (e < nv) elem_store(m.addr, m.dtype, off + e, in[e]);
  }
}

// The interpreter loop must contain uniform branches only: one divergent branch anywhere in it makes
// the compiler linearise the whole dispatch (every handler guarded by predicate checks, register
// copies on every path). Per-lane conditions therefore live in these out-of-line slow paths, which
// take and return the accumulator by value (VGPRs), and the loop picks between the wide path and
// them with a wave-wide vote.
__device__ __forceinline__ bool wave_all(bool c) { return __builtin_amdgcn_ballot_w64(!c) == 0; }

struct Offs {
  uint64_t v[U];
};

__device__ __attribute__((noinline)) Acc mem_load_slow(uint64_t addr, uint32_t dtype, uint32_t flags, Offs off, uint32_t nvp) {
  addr = uni64(addr);
  dtype = uni(dtype);
  flags = uni(flags);
  VMemDesc m;
  m.addr = addr;
  m.dtype = dtype;
  m.flags = flags;
  const bool fast = (flags & (VMF_VEC | VMF_ALIGNED)) == (VMF_VEC | VMF_ALIGNED);
  Acc out;
  FOR_U {
    const int nv = static_cast<int>((nvp >> (4 * u)) & 0xfu);
    out.v[u] = 0.0f;
    if (nv == 0) continue;
    if (fast && nv == E) {
      if (dtype == VDT_F32 || dtype == VDT_I32) {
        const DVM_GLOBAL vf4 *p = reinterpret_cast<const DVM_GLOBAL vf4 *>(addr + off.v[u] * 4);
        out.v[u] = __builtin_shufflevector(p[0], p[1], 0, 1, 2, 3, 4, 5, 6, 7);
        continue;
      }
      if (dtype == VDT_F16) {
        out.v[u] = __builtin_convertvector(*reinterpret_cast<const DVM_GLOBAL vh8 *>(addr + off.v[u] * 2), vf8);
        continue;
      }
    }
    out.v[u] = slab_load_slow(m, off.v[u], nv);
  }
  return out;
}

__device__ __attribute__((noinline)) void mem_store_slow(uint64_t addr, uint32_t dtype, uint32_t flags, Offs off, uint32_t nvp, Acc in) {
  addr = uni64(addr);
  dtype = uni(dtype);
  flags = uni(flags);
  VMemDesc m;
  m.addr = addr;
  m.dtype = dtype;
  m.flags = flags;
  FOR_U {
    const int nv = static_cast<int>((nvp >> (4 * u)) & 0xfu);
    if (nv == 0) continue;
    slab_store_slow(m, off.v[u], nv, in.v[u]);
  }
}

// VOP_LDX: element e of a slab comes from the operand's offset for that element plus the lane's own int32 value
// (an offset in elements the program has computed from an index tensor).
__device__ __attribute__((noinline)) Acc mem_gather(uint64_t addr, uint32_t dtype, uint32_t flags, Offs off, uint32_t nvp, Acc idx) {
  addr = uni64(addr);
  dtype = uni(dtype);
  flags = uni(flags);
  const uint64_t step = (flags & VMF_GATHER) ? (flags >> 8) : ((flags & VMF_VEC) ? 1u : 0u);
  Acc out;
  FOR_U {
    const int nv = static_cast<int>((nvp >> (4 * u)) & 0xfu);
    out.v[u] = 0.0f;
    FOR_E {
      if (e < nv) {
        const int64_t at = static_cast<int64_t>(off.v[u] + e * step) + static_cast<int64_t>(__float_as_int(idx.v[u][e]));
        out.v[u][e] = elem_load(addr, dtype, static_cast<uint64_t>(at));
      }
    }
  }
  return out;
}

// Which slabs of a round the whole wave can treat alike. `full`: bit u is set when slab u is full in every lane;
// `uniform`: every slab is either full in every lane or empty in every lane, so the wave takes the wide paths on
// the slabs in `full` and skips the others (the last round of a sweep usually has some slabs past the end).
struct Slabs {
  uint32_t nvp;      // valid counts, 4 bits per slab
  uint32_t full;
  bool uniform;
};

__device__ __forceinline__ Slabs slab_state(uint32_t nvp) {
  Slabs s;
  s.nvp = nvp;
  s.full = 0;
  uint32_t mixed = 0;
  FOR_U {
    const uint32_t nv = (nvp >> (4 * u)) & 0xfu;
    const bool all_full = wave_all(nv == static_cast<uint32_t>(E));
    const bool all_empty = wave_all(nv == 0u);
    s.full |= (all_full ? 1u : 0u) << u;
    mixed |= (all_full || all_empty) ? 0u : 1u;
  }
  s.uniform = mixed == 0u;
  return s;
}

// Wide path of a load: the slabs in `full` are full and aligned in every lane of the wave (the others are empty
// in every lane and read as zero). All loads are issued before any use.
__device__ __forceinline__ void mem_load_wide(const VMemDesc &m, const Offs &off, uint32_t full, Acc &out) {
  const uint32_t dtype = m.dtype;
  if (dtype == VDT_F32 || dtype == VDT_I32) {
    vf4 a[U], b[U];
    FOR_U {
      a[u] = 0.0f;
      b[u] = 0.0f;
      if ((full >> u) & 1u) {
        const DVM_GLOBAL vf4 *p = reinterpret_cast<const DVM_GLOBAL vf4 *>(m.addr + off.v[u] * 4);
        a[u] = p[0];
        b[u] = p[1];
      }
    }
    FOR_U out.v[u] = __builtin_shufflevector(a[u], b[u], 0, 1, 2, 3, 4, 5, 6, 7);
  } else if (dtype == VDT_BF16) {
    vu4 a[U];
    FOR_U {
      a[u] = 0u;
      if ((full >> u) & 1u) a[u] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(m.addr + off.v[u] * 2);
    }
    FOR_U {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        out.v[u][2 * i] = __uint_as_float(a[u][i] << 16);
        out.v[u][2 * i + 1] = __uint_as_float(a[u][i] & 0xffff0000u);
      }
    }
  } else if (dtype == VDT_F16) {
    vh8 a[U];
    FOR_U {
      a[u] = static_cast<_Float16>(0.0f);
      if ((full >> u) & 1u) a[u] = *reinterpret_cast<const DVM_GLOBAL vh8 *>(m.addr + off.v[u] * 2);
    }
    FOR_U out.v[u] = __builtin_convertvector(a[u], vf8);
  } else {
    vu2 a[U];
    FOR_U {
      a[u] = 0u;
      if ((full >> u) & 1u) a[u] = *reinterpret_cast<const DVM_GLOBAL vu2 *>(m.addr + off.v[u]);
    }
    FOR_U {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        out.v[u][e] = ((a[u][0] >> (8 * e)) & 0xffu) ? 1.0f : 0.0f;
        out.v[u][e + 4] = ((a[u][1] >> (8 * e)) & 0xffu) ? 1.0f : 0.0f;
      }
    }
  }
}

// Two operands that walk memory identically (same element offsets), both on the wide path: every load of both is
// issued before anything is used, so the pair costs one trip to memory instead of two.
__device__ __forceinline__ void mem_load2_wide(const VMemDesc &m, const VMemDesc &mb, const Offs &off, uint32_t full, Acc &x, Acc &y) {
  if (m.dtype == VDT_BF16 && mb.dtype == VDT_BF16) {
    vu4 a[U], b[U];
    FOR_U {
      a[u] = 0u;
      b[u] = 0u;
      if ((full >> u) & 1u) {
        a[u] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(m.addr + off.v[u] * 2);
        b[u] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(mb.addr + off.v[u] * 2);
      }
    }
    FOR_U {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x.v[u][2 * i] = __uint_as_float(a[u][i] << 16);
        x.v[u][2 * i + 1] = __uint_as_float(a[u][i] & 0xffff0000u);
        y.v[u][2 * i] = __uint_as_float(b[u][i] << 16);
        y.v[u][2 * i + 1] = __uint_as_float(b[u][i] & 0xffff0000u);
      }
    }
  } else if (m.dtype == VDT_F16 && mb.dtype == VDT_F16) {
    vh8 a[U], b[U];
    FOR_U {
      a[u] = static_cast<_Float16>(0.0f);
      b[u] = static_cast<_Float16>(0.0f);
      if ((full >> u) & 1u) {
        a[u] = *reinterpret_cast<const DVM_GLOBAL vh8 *>(m.addr + off.v[u] * 2);
        b[u] = *reinterpret_cast<const DVM_GLOBAL vh8 *>(mb.addr + off.v[u] * 2);
      }
    }
    FOR_U {
      x.v[u] = __builtin_convertvector(a[u], vf8);
      y.v[u] = __builtin_convertvector(b[u], vf8);
    }
  } else if ((m.dtype == VDT_F32 || m.dtype == VDT_I32) && (mb.dtype == VDT_F32 || mb.dtype == VDT_I32)) {
    vf4 a0[U], a1[U], b0[U], b1[U];
    FOR_U {
      a0[u] = a1[u] = b0[u] = b1[u] = 0.0f;
      if ((full >> u) & 1u) {
        const DVM_GLOBAL vf4 *pa = reinterpret_cast<const DVM_GLOBAL vf4 *>(m.addr + off.v[u] * 4);
        const DVM_GLOBAL vf4 *pb = reinterpret_cast<const DVM_GLOBAL vf4 *>(mb.addr + off.v[u] * 4);
        a0[u] = pa[0];
        a1[u] = pa[1];
        b0[u] = pb[0];
        b1[u] = pb[1];
      }
    }
    FOR_U {
      x.v[u] = __builtin_shufflevector(a0[u], a1[u], 0, 1, 2, 3, 4, 5, 6, 7);
      y.v[u] = __builtin_shufflevector(b0[u], b1[u], 0, 1, 2, 3, 4, 5, 6, 7);
    }
  } else {  // operands of different widths: one after the other
    mem_load_wide(m, off, full, x);
    mem_load_wide(mb, off, full, y);
  }
}

// One operand at the element offsets of two rounds, both on the wide path: again every load is issued before
// anything is used.
__device__ __forceinline__ void mem_load_wide_2rounds(const VMemDesc &m, const Offs &off, const Offs &off2, uint32_t full, uint32_t full2,
                                                      Acc &x, Acc &y) {
  if (m.dtype == VDT_F32 || m.dtype == VDT_I32) {
    vf4 a0[U], a1[U], b0[U], b1[U];
    FOR_U {
      a0[u] = a1[u] = b0[u] = b1[u] = 0.0f;
      if ((full >> u) & 1u) {
        const DVM_GLOBAL vf4 *pa = reinterpret_cast<const DVM_GLOBAL vf4 *>(m.addr + off.v[u] * 4);
        a0[u] = pa[0];
        a1[u] = pa[1];
      }
      if ((full2 >> u) & 1u) {
        const DVM_GLOBAL vf4 *pb = reinterpret_cast<const DVM_GLOBAL vf4 *>(m.addr + off2.v[u] * 4);
        b0[u] = pb[0];
        b1[u] = pb[1];
      }
    }
    FOR_U {
      x.v[u] = __builtin_shufflevector(a0[u], a1[u], 0, 1, 2, 3, 4, 5, 6, 7);
      y.v[u] = __builtin_shufflevector(b0[u], b1[u], 0, 1, 2, 3, 4, 5, 6, 7);
    }
  } else if (m.dtype == VDT_BF16) {
    vu4 a[U], b[U];
    FOR_U {
      a[u] = 0u;
      b[u] = 0u;
      if ((full >> u) & 1u) a[u] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(m.addr + off.v[u] * 2);
      if ((full2 >> u) & 1u) b[u] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(m.addr + off2.v[u] * 2);
    }
    FOR_U {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x.v[u][2 * i] = __uint_as_float(a[u][i] << 16);
        x.v[u][2 * i + 1] = __uint_as_float(a[u][i] & 0xffff0000u);
        y.v[u][2 * i] = __uint_as_float(b[u][i] << 16);
        y.v[u][2 * i + 1] = __uint_as_float(b[u][i] & 0xffff0000u);
      }
    }
  } else if (m.dtype == VDT_F16) {
    vh8 a[U], b[U];
    FOR_U {
      a[u] = static_cast<_Float16>(0.0f);
      b[u] = static_cast<_Float16>(0.0f);
      if ((full >> u) & 1u) a[u] = *reinterpret_cast<const DVM_GLOBAL vh8 *>(m.addr + off.v[u] * 2);
      if ((full2 >> u) & 1u) b[u] = *reinterpret_cast<const DVM_GLOBAL vh8 *>(m.addr + off2.v[u] * 2);
    }
    FOR_U {
      x.v[u] = __builtin_convertvector(a[u], vf8);
      y.v[u] = __builtin_convertvector(b[u], vf8);
    }
  } else {
    mem_load_wide(m, off, full, x);
    mem_load_wide(m, off2, full2, y);
  }
}

__device__ __forceinline__ void mem_store_wide(const VMemDesc &m, const Offs &off, uint32_t full, const Acc &in) {
  const uint32_t dtype = m.dtype;
  FOR_U {
    if (!((full >> u) & 1u)) continue;
    if (dtype == VDT_F32 || dtype == VDT_I32) {
      DVM_GLOBAL vf4 *p = reinterpret_cast<DVM_GLOBAL vf4 *>(m.addr + off.v[u] * 4);
      p[0] = __builtin_shufflevector(in.v[u], in.v[u], 0, 1, 2, 3);
      p[1] = __builtin_shufflevector(in.v[u], in.v[u], 4, 5, 6, 7);
    } else if (dtype == VDT_BF16) {
      vu4 a;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = pack_bf16(in.v[u][2 * i], in.v[u][2 * i + 1]);
      *reinterpret_cast<DVM_GLOBAL vu4 *>(m.addr + off.v[u] * 2) = a;
    } else if (dtype == VDT_F16) {
      *reinterpret_cast<DVM_GLOBAL vh8 *>(m.addr + off.v[u] * 2) = __builtin_convertvector(in.v[u], vh8);
    } else {
      vu2 a = 0u;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        a[0] |= (in.v[u][e] != 0.0f ? 1u : 0u) << (8 * e);
        a[1] |= (in.v[u][e + 4] != 0.0f ? 1u : 0u) << (8 * e);
      }
      *reinterpret_cast<DVM_GLOBAL vu2 *>(m.addr + off.v[u]) = a;
    }
  }
}

__device__ __forceinline__ void mem_load(const VMemDesc &m, const Offs &off, const Slabs &sl, Acc &out) {
  const uint32_t nvp = sl.nvp;
  const bool fast = (m.flags & (VMF_VEC | VMF_ALIGNED)) == (VMF_VEC | VMF_ALIGNED);
  if (fast && sl.uniform) {
    mem_load_wide(m, off, sl.full, out);
  } else if (!(m.flags & (VMF_VEC | VMF_GATHER)) && (m.dtype == VDT_F32 || m.dtype == VDT_I32)) {
    // one 32-bit element per slab, replicated (an operand broadcast along the innermost axis: a per-channel
    // scale, a per-row statistic); lanes without a valid slab read the base element and get zero, like the
    // guarded path. Inline: the out-of-line path saves registers to scratch memory around the call.
    FOR_U {
      const bool ok = ((nvp >> (4 * u)) & 0xfu) != 0u;
      const float v = reinterpret_cast<const DVM_GLOBAL float *>(m.addr)[ok ? off.v[u] : 0u];
      out.v[u] = ok ? v : 0.0f;
    }
  } else {
    out = mem_load_slow(m.addr, m.dtype, m.flags, off, nvp);
  }
}

__device__ __forceinline__ void mem_store(const VMemDesc &m, const Offs &off, const Slabs &sl, const Acc &in) {
  const bool fast = (m.flags & (VMF_VEC | VMF_ALIGNED)) == (VMF_VEC | VMF_ALIGNED);
  if (fast && sl.uniform) {
    mem_store_wide(m, off, sl.full, in);
  } else {
    mem_store_slow(m.addr, m.dtype, m.flags, off, sl.nvp, in);
  }
}

// ---- reduce helpers ----------------------------------------------------------

__device__ __forceinline__ double red_combine(uint32_t kind, double r, double v) {
  if (kind == VR_SUM) return r + v;
  if (kind == VR_MAX) return (v > r || v != v) ? v : r;  // NaN propagates, as NumPy's max/min
  return (v < r || v != v) ? v : r;
}

__device__ __forceinline__ double red_identity(uint32_t kind) {
  if (kind == VR_SUM) return 0.0;
  if (kind == VR_MAX) return -__builtin_huge_val();
  return __builtin_huge_val();
}

template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xf, 0xf, false);
  hi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xf, 0xf, false);
  return __hiloint2double(hi, lo);
}

__device__ __forceinline__ double shfl_xor_f64(double v, int mask) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __shfl_xor(lo, mask, 64);
  hi = __shfl_xor(hi, mask, 64);
  return __hiloint2double(hi, lo);
}

// REDX keeps one fp64 partial per slot (the elements of an instruction are
// combined pairwise first); REDY keeps one per element of the lane's group.
template <int SCHED>
struct RedAcc {
  double v[SCHED == VS_REDY ? E : 1];
};

template <int SCHED>
__device__ __forceinline__ void red_init(RedAcc<SCHED> &r, uint32_t kind) {
  const double idv = red_identity(kind);
#pragma unroll
  for (int e = 0; e < (SCHED == VS_REDY ? E : 1); ++e) r.v[e] = idv;
}

// One reduce step for a fixed kind; the kind is resolved once per instruction, outside the element loops.
template <int KIND, typename T>
__device__ __forceinline__ T red_op(T r, T v) {
  if constexpr (KIND == VR_SUM) return r + v;
  if constexpr (KIND == VR_MAX) return (v > r || v != v) ? v : r;  // NaN propagates, as NumPy's max/min
  return (v < r || v != v) ? v : r;
}

template <int SCHED, int KIND>
__device__ __forceinline__ void red_accumulate_k(RedAcc<SCHED> &r, const Acc &x, uint32_t nvp) {
  constexpr float idv = KIND == VR_SUM ? 0.0f : (KIND == VR_MAX ? -__builtin_huge_valf() : __builtin_huge_valf());
  FOR_U {
    const int nv = static_cast<int>((nvp >> (4 * u)) & 0xfu);
    if constexpr (SCHED == VS_REDY) {
      FOR_E {
        const double t = red_op<KIND>(r.v[e], static_cast<double>(x.v[u][e]));
        r.v[e] = e < nv ? t : r.v[e];
      }
    } else {
      // The 8 elements of a slab are combined pairwise in fp32 (the blocking NumPy's float32 sum
      // uses as well); every further step accumulates in fp64.
      float d[E];
      FOR_E d[e] = e < nv ? x.v[u][e] : idv;  // selects, not branches
#pragma unroll
      for (int w = 1; w < E; w <<= 1)
#pragma unroll
        for (int e = 0; e + w < E; e += 2 * w) d[e] = red_op<KIND>(d[e], d[e + w]);
      const double t = red_op<KIND>(r.v[0], static_cast<double>(d[0]));
      r.v[0] = nv > 0 ? t : r.v[0];
    }
  }
}

// The slabs in `full` are full in every lane of the wave, the others empty (the common rounds): no per-element guards.
template <int SCHED, int KIND>
__device__ __forceinline__ void red_accumulate_full(RedAcc<SCHED> &r, const Acc &x, uint32_t full) {
  FOR_U {
    if (!((full >> u) & 1u)) continue;
    if constexpr (SCHED == VS_REDY) {
      FOR_E r.v[e] = red_op<KIND>(r.v[e], static_cast<double>(x.v[u][e]));
    } else {
      float d[E];
      FOR_E d[e] = x.v[u][e];
#pragma unroll
      for (int w = 1; w < E; w <<= 1)
#pragma unroll
        for (int e = 0; e + w < E; e += 2 * w) d[e] = red_op<KIND>(d[e], d[e + w]);
      r.v[0] = red_op<KIND>(r.v[0], static_cast<double>(d[0]));
    }
  }
}

template <int SCHED>
__device__ __forceinline__ void red_accumulate(RedAcc<SCHED> &r, uint32_t kind, const Acc &x, const Slabs &sl) {
  const uint32_t nvp = sl.nvp;
  if (sl.uniform) {
    if (kind == VR_SUM) {
      red_accumulate_full<SCHED, VR_SUM>(r, x, sl.full);
    } else if (kind == VR_MAX) {
      red_accumulate_full<SCHED, VR_MAX>(r, x, sl.full);
    } else {
      red_accumulate_full<SCHED, VR_MIN>(r, x, sl.full);
    }
    return;
  }
  if (kind == VR_SUM) {
    red_accumulate_k<SCHED, VR_SUM>(r, x, nvp);
  } else if (kind == VR_MAX) {
    red_accumulate_k<SCHED, VR_MAX>(r, x, nvp);
  } else {
    red_accumulate_k<SCHED, VR_MIN>(r, x, nvp);
  }
}

// max / min over int32 values (the accumulator holds their bit patterns): integer compares inside a slab, the
// running partial as a double, which holds every int32 exactly, so the combine across lanes is the float one.
template <int SCHED>
__device__ __forceinline__ void red_accumulate_int(RedAcc<SCHED> &r, uint32_t kind, const Acc &x, uint32_t nvp) {
  const bool is_max = kind == VR_MAX;
  FOR_U {
    const int nv = static_cast<int>((nvp >> (4 * u)) & 0xfu);
    if constexpr (SCHED == VS_REDY) {
      FOR_E {
        const double v = static_cast<double>(__float_as_int(x.v[u][e]));
        const double t = is_max ? (v > r.v[e] ? v : r.v[e]) : (v < r.v[e] ? v : r.v[e]);
        r.v[e] = e < nv ? t : r.v[e];
      }
    } else {
      int32_t best = is_max ? INT32_MIN : INT32_MAX;
      FOR_E {
        const int32_t v = __float_as_int(x.v[u][e]);
        const int32_t t = is_max ? max(best, v) : min(best, v);
        best = e < nv ? t : best;
      }
      const double v = static_cast<double>(best);
      const double t = is_max ? (v > r.v[0] ? v : r.v[0]) : (v < r.v[0] ? v : r.v[0]);
      r.v[0] = nv > 0 ? t : r.v[0];
    }
  }
}

// Local memory shared by the lanes of a workgroup, in doubles from the start of the dynamic segment:
//   [0, 64)   partials of the waves at the end of a sweep: two buffers (used in turn) of two slots of 16 waves;
//   [64, 80)  what the first wave hands to the others after a per-team run: two buffers (in turn) of 16 floats.
// With the buffers used in turn a wave cannot overwrite what a slower wave still has to read: between two uses of
// one buffer lies the barrier of the other one, which the slower wave only reaches once its reads are done.
// VS_REDY uses [0, E * lanes) as one buffer with barriers on both sides.
constexpr uint32_t kPartialsPerBuffer = 32;
constexpr uint32_t kBoxAt = 64;

// End of a sweep, innermost axis reduced: combines the partials of both slots across the lanes that share an
// output (a team inside a wave by shuffles; a team that is the workgroup through local memory, one barrier for
// both slots). Every one of those lanes ends up with the results. `flip` selects the buffer and is toggled.
__device__ __forceinline__ void red_finish_x(double &r0, double &r1, uint32_t k0, uint32_t k1, uint32_t tlog, bool team_is_block,
                                             uint32_t tid, uint32_t nthreads, uint32_t &flip, double *shared) {
  k0 = uni(k0);
  k1 = uni(k1);
  tlog = uni(tlog);
  team_is_block = uni(team_is_block ? 1u : 0u) != 0u;
  nthreads = uni(nthreads);
  const bool on0 = k0 <= VR_MIN, on1 = k1 <= VR_MIN;
  double t0 = r0, t1 = r1;
  const uint32_t span = team_is_block ? 64u : (1u << tlog);
  // Inside a row of 16 lanes the partner's value comes through the data-parallel-primitive path of the vector unit
  // (neighbour, next pair, the mirror image within 8 and within 16: each step doubles the lanes whose partials a lane
  // holds, and both partners compute the same sum), which costs an instruction instead of a trip through local
  // memory; the rows of a wave are combined by shuffles.
  if (span > 1u) {
    if (on0) t0 = red_combine(k0, t0, dpp_f64<0xB1>(t0));  // quad_perm [1,0,3,2]
    if (on1) t1 = red_combine(k1, t1, dpp_f64<0xB1>(t1));
  }
  if (span > 2u) {
    if (on0) t0 = red_combine(k0, t0, dpp_f64<0x4E>(t0));  // quad_perm [2,3,0,1]
    if (on1) t1 = red_combine(k1, t1, dpp_f64<0x4E>(t1));
  }
  if (span > 4u) {
    if (on0) t0 = red_combine(k0, t0, dpp_f64<0x141>(t0));  // row_half_mirror
    if (on1) t1 = red_combine(k1, t1, dpp_f64<0x141>(t1));
  }
  if (span > 8u) {
    if (on0) t0 = red_combine(k0, t0, dpp_f64<0x140>(t0));  // row_mirror
    if (on1) t1 = red_combine(k1, t1, dpp_f64<0x140>(t1));
  }
  for (uint32_t msk = 16; msk < span; msk <<= 1) {
    if (on0) t0 = red_combine(k0, t0, shfl_xor_f64(t0, msk));
    if (on1) t1 = red_combine(k1, t1, shfl_xor_f64(t1, msk));
  }
  if (team_is_block) {
    double *buf = shared + flip * kPartialsPerBuffer;
    flip ^= 1u;
    const uint32_t wave = tid >> 6, nw = (nthreads + 63u) >> 6;
    buf[wave] = t0;  // every lane of a wave holds the wave's value: identical writes, no per-lane branch
    buf[16 + wave] = t1;
    __syncthreads();
    // lane j takes wave (j mod 16)'s partial; four shuffle steps leave the total in every lane
    const uint32_t j = tid & 15u;
    const double a0 = buf[j], a1 = buf[16 + j];
    t0 = j < nw ? a0 : red_identity(k0);
    t1 = j < nw ? a1 : red_identity(k1);
    if (on0) {  // the 16 partials of a row of lanes: the same four steps
      t0 = red_combine(k0, t0, dpp_f64<0xB1>(t0));
      t0 = red_combine(k0, t0, dpp_f64<0x4E>(t0));
      t0 = red_combine(k0, t0, dpp_f64<0x141>(t0));
      t0 = red_combine(k0, t0, dpp_f64<0x140>(t0));
    }
    if (on1) {
      t1 = red_combine(k1, t1, dpp_f64<0xB1>(t1));
      t1 = red_combine(k1, t1, dpp_f64<0x4E>(t1));
      t1 = red_combine(k1, t1, dpp_f64<0x141>(t1));
      t1 = red_combine(k1, t1, dpp_f64<0x140>(t1));
    }
  }
  r0 = t0;
  r1 = t1;
}

// End of a sweep, innermost axis kept: the rows of the workgroup that share an output group combine their
// partials through local memory (DVM_VEC_RED_SCRATCH_DOUBLES doubles: one per lane and element). Every lane writes
// its E partials; the lane of row r then combines, for element r (and r + rows, ...) of its group, the partials of
// all rows in row order and leaves the result where row 0's was; after a second barrier every lane reads the E
// results of its group. Three barriers per slot, and each partial is read once.
template <int SCHED>
__device__ __forceinline__ RedAcc<SCHED> red_finish_y(RedAcc<SCHED> r, uint32_t rk, uint32_t tlog, uint32_t nthreads, uint32_t k_local,
                                                      uint32_t r_local, double *scratch) {
  rk = uni(rk);
  tlog = uni(tlog);
  nthreads = uni(nthreads);
  if constexpr (SCHED == VS_REDY) {
    const uint32_t tx = 1u << tlog, ty = nthreads >> tlog;
    if (ty > 1) {
      __syncthreads();  // (what an earlier sweep left here has been read)
      FOR_E scratch[(e * ty + r_local) * tx + k_local] = r.v[e];
      __syncthreads();
      for (uint32_t v = r_local; v < static_cast<uint32_t>(E); v += ty) {
        const double *col = scratch + v * ty * tx + k_local;
        double t = col[0];
        uint32_t j = 1;
        for (; j + 4 <= ty; j += 4) {  // four reads in flight, combined in row order
          const double a0 = col[j * tx], a1 = col[(j + 1) * tx], a2 = col[(j + 2) * tx], a3 = col[(j + 3) * tx];
          t = red_combine(rk, t, a0);
          t = red_combine(rk, t, a1);
          t = red_combine(rk, t, a2);
          t = red_combine(rk, t, a3);
        }
        for (; j < ty; ++j) t = red_combine(rk, t, col[j * tx]);
        scratch[v * ty * tx + k_local] = t;
      }
      __syncthreads();
      FOR_E r.v[e] = scratch[e * ty * tx + k_local];
    }
  }
  return r;
}

// ---- S registers (one float per lane, VGPRs) -----------------------------------

struct SRegs {
  float s0, s1, s2, s3, s4, s5, s6, s7;
};

__device__ __forceinline__ float sreg_read(const SRegs &sr, uint32_t idx) {
  switch (idx) {
    case 0: return sr.s0;
    case 1: return sr.s1;
    case 2: return sr.s2;
    case 3: return sr.s3;
    case 4: return sr.s4;
    case 5: return sr.s5;
    case 6: return sr.s6;
    default: return sr.s7;
  }
}

__device__ __forceinline__ void sreg_write(SRegs &sr, uint32_t idx, float v) {
  switch (idx) {
    case 0: sr.s0 = v; break;
    case 1: sr.s1 = v; break;
    case 2: sr.s2 = v; break;
    case 3: sr.s3 = v; break;
    case 4: sr.s4 = v; break;
    case 5: sr.s5 = v; break;
    case 6: sr.s6 = v; break;
    default: sr.s7 = v; break;
  }
}

// ---- V registers (U*E values per lane, local memory) -----------------------------
// A slot is U planes of 16 bytes per lane; slab u of slot s lives at
// plane[(s*U + u) * nthreads + tid]. A lane only touches its own column, so no
// barrier is needed. fp32 values take two slots, fp16/bf16-representable
// values are packed into one.
__device__ __forceinline__ void vreg_store(vf4 *planes, uint32_t slot, uint32_t fmt, uint32_t nthreads, uint32_t tid,
                                           const Acc &a) {
  if (fmt == VF_F32) {
    FOR_U {
      planes[(slot * U + u) * nthreads + tid] = __builtin_shufflevector(a.v[u], a.v[u], 0, 1, 2, 3);
      planes[((slot + 1) * U + u) * nthreads + tid] = __builtin_shufflevector(a.v[u], a.v[u], 4, 5, 6, 7);
    }
  } else if (fmt == VF_F16) {
    FOR_U {
      vh8 hv = __builtin_convertvector(a.v[u], vh8);
      planes[(slot * U + u) * nthreads + tid] = *reinterpret_cast<vf4 *>(&hv);
    }
  } else {
    FOR_U {
      vu4 b;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        b[i] = (__float_as_uint(a.v[u][2 * i]) >> 16) | (__float_as_uint(a.v[u][2 * i + 1]) & 0xffff0000u);
      planes[(slot * U + u) * nthreads + tid] = *reinterpret_cast<vf4 *>(&b);
    }
  }
}

__device__ __forceinline__ void vreg_load(const vf4 *planes, uint32_t slot, uint32_t fmt, uint32_t nthreads, uint32_t tid,
                                          Acc &a) {
  if (fmt == VF_F32) {
    FOR_U {
      const vf4 lo = planes[(slot * U + u) * nthreads + tid];
      const vf4 hi = planes[((slot + 1) * U + u) * nthreads + tid];
      a.v[u] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  } else if (fmt == VF_F16) {
    FOR_U {
      vf4 raw = planes[(slot * U + u) * nthreads + tid];
      a.v[u] = __builtin_convertvector(*reinterpret_cast<vh8 *>(&raw), vf8);
    }
  } else {
    FOR_U {
      vf4 raw = planes[(slot * U + u) * nthreads + tid];
      vu4 b = *reinterpret_cast<vu4 *>(&raw);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a.v[u][2 * i] = __uint_as_float(b[i] << 16);
        a.v[u][2 * i + 1] = __uint_as_float(b[i] & 0xffff0000u);
      }
    }
  }
}

// A memory operand's descriptor from the program in local memory. Only what the interpreter branches on (element
// type, flags) is made wave-uniform; the address and the strides only ever enter per-lane arithmetic, where a copy
// in every lane serves as well as a scalar register and costs no v_readfirstlane and no scalar registers.
__device__ __forceinline__ VMemDesc load_desc(const uint32_t *prog32, uint32_t mem_off_words, uint32_t idx) {
  const vu4 *d = reinterpret_cast<const vu4 *>(prog32 + 2 * mem_off_words + idx * (sizeof(VMemDesc) / 4));
  const vu4 d0 = d[0], d1 = d[1], d2 = d[2];
  VMemDesc m;
  m.addr = static_cast<uint64_t>(d0[0]) | (static_cast<uint64_t>(d0[1]) << 32);
  m.dtype = uni(d0[2]);
  m.flags = uni(d0[3]);
#pragma unroll
  for (int i = 0; i < DVM_VEC_MAXR; ++i) {
    m.kstride[i] = d1[i];
    m.rstride[i] = d2[i];
  }
  return m;
}

// Splits a flat index of an index space into its coordinates and returns the
// element offset sum(coord * stride). The innermost-axis coordinate counts
// E-groups when `inner` is set and is converted to elements.
// `dims` points at the axis table in local memory: its entries feed per-lane arithmetic only, so they are read
// where they are needed (one 128-bit read per division) instead of living in scalar registers for the whole launch.
// A uniform value as it is now, for a test that should be made where it stands: a test of a loop-invariant value is
// otherwise hoisted out of the interpreter loop, and its result then occupies a pair of scalar registers for the
// whole launch (enough of those and the kernel spills scalar registers into lanes of a vector register, which every
// use reads back).
__device__ __forceinline__ uint32_t fresh(uint32_t x) {
  asm volatile("" : "+s"(x));
  return x;
}

// (three and four axes, out of line: rare, and inlined at every memory instruction their tests of the axis count sat
// in scalar registers that the hot paths then had to spill)
__device__ __attribute__((noinline)) uint64_t space_offset_rest(uint32_t n, const VDim *dims, uint32_t ndim, uint32_t s1, uint32_t s2,
                                                                uint32_t s3) {
  const uint32_t stride[DVM_VEC_MAXR] = {0u, s1, s2, s3};
  uint64_t off = 0;
#pragma unroll
  for (int i = 1; i < DVM_VEC_MAXR; ++i) {
    if (i < static_cast<int>(ndim)) {
      uint32_t c = n;
      if (i + 1 < static_cast<int>(ndim)) {
        const vu4 dv = *reinterpret_cast<const vu4 *>(dims + i);
        const uint32_t q = (__umulhi(n, dv[1]) + n) >> dv[2];
        c = n - q * dv[0];
        n = q;
      }
      off += static_cast<uint64_t>(c) * stride[i];
    }
  }
  return off;
}

__device__ __forceinline__ uint64_t space_offset(uint32_t n, const VDim *dims, uint32_t ndim,
                                                 const uint32_t (&stride)[DVM_VEC_MAXR], bool inner) {
  // a space of one axis (rows of a matrix, elements of a row): no division, and one uniform branch here instead of
  // two per axis (a dozen scalar branches per memory instruction otherwise: they, not the arithmetic, were most of
  // what the offsets of an instruction cost)
  ndim = fresh(ndim);
  if (ndim <= 1u) return (static_cast<uint64_t>(n) * stride[0]) * (inner ? static_cast<uint32_t>(E) : 1u);
  // the first axis, then the second alone when there are two (one more uniform branch), else the rest
  uint64_t off;
  {
    const vu4 dv = *reinterpret_cast<const vu4 *>(dims);  // extent, magic, shift, pad
    const uint32_t q = (__umulhi(n, dv[1]) + n) >> dv[2];
    off = (static_cast<uint64_t>(n - q * dv[0]) * stride[0]) * (inner ? static_cast<uint32_t>(E) : 1u);
    n = q;
  }
  if (ndim == 2u) return off + static_cast<uint64_t>(n) * stride[1];
  return off + space_offset_rest(n, dims, uni(ndim), stride[1], stride[2], stride[3]);
}

// Valid element count (0..E) of the E-group with flat index n in a space whose first axis counts groups.
__device__ __forceinline__ uint32_t group_valid(uint32_t n, const VDim *dims, uint32_t ndim,
                                                uint32_t inner_extent) {
  uint32_t c = n;
  if (fresh(ndim) > 1u) {
    const vu4 dv = *reinterpret_cast<const vu4 *>(dims);
    c = n - ((__umulhi(n, dv[1]) + n) >> dv[2]) * dv[0];
  }
  const uint32_t left = inner_extent - c * E;
  return left < static_cast<uint32_t>(E) ? left : static_cast<uint32_t>(E);
}

// VBI_WRAP: an index into an axis of extent n, negative values counting from the end, clipped into the axis
__device__ __forceinline__ int32_t wrap_index(int32_t i, int32_t n) {
  i = i < 0 ? i + n : i;
  i = i < n - 1 ? i : n - 1;
  return i > 0 ? i : 0;
}

// Arithmetic on one value per lane, for instructions flagged VI_UNIFORM. Inlined, so that the opcode stays
// in scalar registers and the selection below is a scalar branch (as arguments of an out-of-line function
// the opcodes travel in vector registers and every case is walked under an execution mask); the library
// functions with internal per-lane branches go through the out-of-line slab helpers.
__device__ __forceinline__ float uniform_binary(uint32_t op, uint32_t sub, float x, float y) {
  if (op == VOP_BINF) {
    switch (sub & 0x3fu) {
      case VB_ADD: return x + y;
      case VB_SUB: return x - y;
      case VB_RSUB: return y - x;
      case VB_MUL: return x * y;
      case VB_DIV: return x / y;
      case VB_RDIV: return y / x;
      case VB_MIN: return x < y ? x : y;
      case VB_MAX: return x > y ? x : y;
      case VB_AND: return (x != 0.0f && y != 0.0f) ? 1.0f : 0.0f;
      case VB_OR: return (x != 0.0f || y != 0.0f) ? 1.0f : 0.0f;
      case VB_POW: return slab_pow(vf8(x), vf8(y))[0];
      default: return slab_pow(vf8(y), vf8(x))[0];
    }
  }
  const uint32_t xi = __float_as_uint(x), yi = __float_as_uint(y);
  const int32_t xs = __float_as_int(x), ys = __float_as_int(y);
  if (op == VOP_BINI) {
    switch (sub & 0x3fu) {
      case VBI_ADD: return __uint_as_float(xi + yi);
      case VBI_SUB: return __uint_as_float(xi - yi);
      case VBI_RSUB: return __uint_as_float(yi - xi);
      case VBI_MUL: return __uint_as_float(xi * yi);
      case VBI_MIN: return __int_as_float(min(xs, ys));
      case VBI_WRAP: return __int_as_float(wrap_index(xs, ys));
      default: return __int_as_float(max(xs, ys));
    }
  }
  const uint32_t t = sub & 0x7u;
  if (sub & VCMP_INT) {
    const bool c = t == VCMP_EQ ? xs == ys : t == VCMP_NE ? xs != ys : t == VCMP_GT ? xs > ys : t == VCMP_GE ? xs >= ys : t == VCMP_LT ? xs < ys : xs <= ys;
    return __int_as_float(c ? 1 : 0);
  }
  const bool c = t == VCMP_EQ ? x == y : t == VCMP_NE ? x != y : t == VCMP_GT ? x > y : t == VCMP_GE ? x >= y : t == VCMP_LT ? x < y : x <= y;
  return c ? 1.0f : 0.0f;
}

__device__ __forceinline__ float uniform_unary(uint32_t sub, float x) {
  switch (sub) {
    case VU_SQRT: return slab_sqrt(vf8(x))[0];
    case VU_ABS: return fabsf(x);
    case VU_LOG: return slab_log(vf8(x))[0];
    case VU_EXP: return slab_exp(vf8(x))[0];
    case VU_ISFINITE: return isfinite(x) ? 1.0f : 0.0f;
    case VU_ROUND: return rintf(x);
    case VU_FLOOR: return floorf(x);
    case VU_CEIL: return ceilf(x);
    case VU_TRUNC: return truncf(x);
    default: {
      const uint32_t v = __float_as_uint(x);
      return __uint_as_float(static_cast<int32_t>(v) < 0 ? 0u - v : v);
    }
  }
}

__device__ __forceinline__ float uniform_cast(uint32_t sub, float x) {
  if (sub == VC_F2I) return __int_as_float(static_cast<int32_t>(x));
  if (sub == VC_I2F) return static_cast<float>(__float_as_int(x));
  if (sub == VC_RND) return x;
  return x != 0.0f ? 1.0f : 0.0f;
}

// Builds with -DDVM_VEC_STAMPS write the memory clock (100 MHz) at the STAMP() marks of the interpreter kernels, one row of 32 stamps per
// wave, to the address in the last word of the blob when that word is not zero: where a launch spends its time,
// wave by wave. Nothing of it exists in a regular build.
#ifdef DVM_VEC_STAMPS
#define STAMP()                                                                                               \
  do {                                                                                                        \
    if (stamp_base != 0 && stamp_n < 32u) {                                                                   \
      const uint64_t now = __builtin_amdgcn_s_memrealtime();                                                  \
      if ((threadIdx.x & 63u) == 0u)                                                                          \
        reinterpret_cast<DVM_GLOBAL uint64_t *>(stamp_base)[(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 32u + stamp_n] = now; \
      ++stamp_n;                                                                                              \
    }                                                                                                         \
  } while (0)
#else
#define STAMP() do {} while (0)
#endif

}  // namespace

#endif  // DVM_DEVICE_VEC_COMMON_H_
