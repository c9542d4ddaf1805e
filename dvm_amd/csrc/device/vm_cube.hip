// gfx950 matmul VM: MFMA tile loop with an interpreted epilogue applied from registers.
//
// Role in the reference: the cube kernels (device semantics src/vm_aic.cce:34-470: fp32
// accumulation, one rounding to the operand type on write-out) plus the mix kernel's post-fusion
// vector program (src/xkernel.cc:304-360). The reference's CUDA backend has no matmul at all
// (src/system.cc:290-294); this kernel is specific to CDNA4:
//  * v_mfma_f32_32x32x16 (bf16 / f16), 64-wide waves, each wave owns a (TM*32) x (TN*32) block of
//    accumulators that never leaves registers until the epilogue has run;
//  * operand tiles are staged through local memory with k contiguous and rows padded by 16 bytes,
//    so every fragment read is one conflict-free 128-bit access; operands whose k axis is strided
//    in memory (B of an NN product, A of a TN product) are transposed in registers on the way in;
//  * local memory is double buffered, the next tile's global loads are in flight while the MFMAs
//    of the current one run;
//  * the epilogue decodes the vector VM's instruction words (wave-uniform) and works on the 16
//    accumulator values a lane holds of one 32x32 tile, so bias add, activation and casts cost no
//    extra pass over memory.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../isa_gfx950.h"

namespace {

#define DVM_GLOBAL __attribute__((address_space(1)))

typedef float vf16 __attribute__((ext_vector_type(16)));
typedef uint32_t vu4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

constexpr int BK = 64;          // k extent of a staged tile
constexpr int LDS_ROW = BK + 8; // elements per padded row (144 bytes)

__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

__device__ __forceinline__ float round_f16(float x) { return static_cast<float>(static_cast<_Float16>(x)); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
  r = (x != x) ? 0x7fc00000u : r;
  return r >> 16;
}
__device__ __forceinline__ float round_bf16(float x) { return __uint_as_float(f32_to_bf16_bits(x) << 16); }

template <bool IS_BF16>
__device__ __forceinline__ vf16 mfma(vu4 a, vu4 b, vf16 c) {
  if constexpr (IS_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8 *>(&a), *reinterpret_cast<bf16x8 *>(&b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<half8 *>(&a), *reinterpret_cast<half8 *>(&b), c, 0, 0, 0);
  }
}

// ---- staging one operand tile: ROWS rows (m or n) x BK (k), k contiguous in local memory -------------
// Source with k contiguous (A when !trans_a, B when trans_b): 16-byte chunks copied as they are.
// Source with k strided (row index contiguous): 8x8 element blocks, transposed in registers.
template <int ROWS>
struct Stage {
  static constexpr int CHUNKS = ROWS * BK / 8 / 256;  // 16-byte chunks per thread
  // a k-strided source moves whole 8x8 blocks (8 chunks): ROWS blocks per tile, one per thread for
  // the first ROWS threads
  vu4 r[CHUNKS < 8 ? 8 : CHUNKS];
};

// k-contiguous source, every chunk in range and 16-byte aligned
template <int ROWS>
__device__ __forceinline__ void stage_load_kc(Stage<ROWS> &s, uint64_t base, uint32_t ld, uint32_t row0, uint32_t k0, uint32_t tid) {
#pragma unroll
  for (int i = 0; i < Stage<ROWS>::CHUNKS; ++i) {
    const uint32_t c = tid + 256u * i;
    const uint32_t row = c / (BK / 8), kc = (c % (BK / 8)) * 8;
    s.r[i] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(base + (static_cast<uint64_t>(row0 + row) * ld + k0 + kc) * 2);
  }
}

template <int ROWS>
__device__ __forceinline__ void stage_store_kc(const Stage<ROWS> &s, uint16_t *tile, uint32_t tid) {
#pragma unroll
  for (int i = 0; i < Stage<ROWS>::CHUNKS; ++i) {
    const uint32_t c = tid + 256u * i;
    const uint32_t row = c / (BK / 8), kc = (c % (BK / 8)) * 8;
    *reinterpret_cast<vu4 *>(tile + row * LDS_ROW + kc) = s.r[i];
  }
}

// k-strided source (memory is [k][row]): thread t < ROWS handles the 8x8 block (kb, rb) = (t / (ROWS/8), t % (ROWS/8))
template <int ROWS>
__device__ __forceinline__ void stage_load_ks(Stage<ROWS> &s, uint64_t base, uint32_t ld, uint32_t row0, uint32_t k0, uint32_t tid) {
  static_assert(ROWS <= 256, "one block per thread");
  if (tid < ROWS) {
    const uint32_t kb = tid / (ROWS / 8), rb = tid % (ROWS / 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s.r[j] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(base + (static_cast<uint64_t>(k0 + kb * 8 + j) * ld + row0 + rb * 8) * 2);
    }
  }
}

template <int ROWS>
__device__ __forceinline__ void stage_store_ks(const Stage<ROWS> &s, uint16_t *tile, uint32_t tid) {
  if (tid < ROWS) {
    const uint32_t kb = tid / (ROWS / 8), rb = tid % (ROWS / 8);
    // in[j][i]: k = kb*8 + j, row = rb*8 + i  ->  out row i holds k = kb*8 .. +7
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      vu4 o = 0u;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t w = s.r[j][i / 2];
        const uint32_t e = (i & 1) ? (w >> 16) : (w & 0xffffu);
        o[j / 2] |= e << (16 * (j & 1));
      }
      *reinterpret_cast<vu4 *>(tile + (rb * 8 + i) * LDS_ROW + kb * 8) = o;
    }
  }
}

// Generic staging of one tile straight into local memory, element by element (edges, unaligned or
// odd leading dimensions). Slow, correct for every shape.
template <int ROWS>
__device__ __attribute__((noinline)) void stage_generic(uint16_t *tile, uint64_t base, uint32_t ld, uint32_t row0, uint32_t k0,
                                                        uint32_t rows, uint32_t kext, uint32_t k_contig, uint32_t tid) {
  for (uint32_t e = tid; e < ROWS * BK; e += 256u) {
    const uint32_t row = e / BK, kk = e % BK;
    const uint32_t gr = row0 + row, gk = k0 + kk;
    uint16_t v = 0;
    if (gr < rows && gk < kext) {
      const uint64_t idx = k_contig ? static_cast<uint64_t>(gr) * ld + gk : static_cast<uint64_t>(gk) * ld + gr;
      v = reinterpret_cast<const DVM_GLOBAL uint16_t *>(base)[idx];
    }
    tile[row * LDS_ROW + kk] = v;
  }
}

// ---- epilogue -------------------------------------------------------------------------------------

struct Frag {
  vf16 v;
};

__device__ __forceinline__ float elem_load(uint64_t base, uint32_t dtype, uint64_t off) {
  switch (dtype) {
    case VDT_F32: return reinterpret_cast<const DVM_GLOBAL float *>(base)[off];
    case VDT_I32: return __int_as_float(reinterpret_cast<const DVM_GLOBAL int32_t *>(base)[off]);
    case VDT_F16: return static_cast<float>(reinterpret_cast<const DVM_GLOBAL _Float16 *>(base)[off]);
    case VDT_BF16: return __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const DVM_GLOBAL uint16_t *>(base)[off]) << 16);
    default: return reinterpret_cast<const DVM_GLOBAL uint8_t *>(base)[off] != 0 ? 1.0f : 0.0f;
  }
}

__device__ __forceinline__ void elem_store(uint64_t base, uint32_t dtype, uint64_t off, float v) {
  switch (dtype) {
    case VDT_F32: reinterpret_cast<DVM_GLOBAL float *>(base)[off] = v; break;
    case VDT_I32: reinterpret_cast<DVM_GLOBAL int32_t *>(base)[off] = __float_as_int(v); break;
    case VDT_F16: reinterpret_cast<DVM_GLOBAL _Float16 *>(base)[off] = static_cast<_Float16>(v); break;
    case VDT_BF16: reinterpret_cast<DVM_GLOBAL uint16_t *>(base)[off] = static_cast<uint16_t>(f32_to_bf16_bits(v)); break;
    default: reinterpret_cast<DVM_GLOBAL uint8_t *>(base)[off] = v != 0.0f ? 1 : 0; break;
  }
}

// Memory operand of the epilogue for the fragment whose lane column is `col` and whose 16 rows are
// row_base + 8*(r/4) + (r%4). Out-of-range positions read 0 / are not written.
__device__ __attribute__((noinline)) Frag frag_load(uint64_t addr, uint32_t dtype, uint32_t sn, uint32_t sm, uint64_t boff,
                                                   uint32_t row_base, uint32_t col, uint32_t m, uint32_t n) {
  Frag f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const uint32_t row = row_base + 8 * (r / 4) + (r % 4);
    float v = 0.0f;
    if (row < m && col < n) v = elem_load(addr, dtype, boff + static_cast<uint64_t>(row) * sm + static_cast<uint64_t>(col) * sn);
    f.v[r] = v;
  }
  return f;
}

__device__ __attribute__((noinline)) void frag_store(uint64_t addr, uint32_t dtype, uint32_t sn, uint32_t sm, uint64_t boff,
                                                    uint32_t row_base, uint32_t col, uint32_t m, uint32_t n, Frag f) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const uint32_t row = row_base + 8 * (r / 4) + (r % 4);
    if (row < m && col < n) elem_store(addr, dtype, boff + static_cast<uint64_t>(row) * sm + static_cast<uint64_t>(col) * sn, f.v[r]);
  }
}

__device__ __attribute__((noinline)) vf16 frag_exp(vf16 x) {
#pragma unroll
  for (int r = 0; r < 16; ++r) x[r] = expf(x[r]);
  return x;
}
__device__ __attribute__((noinline)) vf16 frag_log(vf16 x) {
#pragma unroll
  for (int r = 0; r < 16; ++r) x[r] = logf(x[r]);
  return x;
}
__device__ __attribute__((noinline)) vf16 frag_pow(vf16 x, vf16 y) {
#pragma unroll
  for (int r = 0; r < 16; ++r) x[r] = powf(x[r], y[r]);
  return x;
}
__device__ __attribute__((noinline)) vf16 frag_sqrt(vf16 x) {
#pragma unroll
  for (int r = 0; r < 16; ++r) x[r] = sqrtf(x[r]);
  return x;
}

#define FOR_R _Pragma("unroll") for (int r = 0; r < 16; ++r)

__device__ __forceinline__ void apply_rnd(vf16 &a, uint32_t rnd) {
  if (rnd == VRND_F16) {
    FOR_R a[r] = round_f16(a[r]);
  } else if (rnd == VRND_BF16) {
    FOR_R a[r] = round_bf16(a[r]);
  }
}

// Runs the epilogue program on one accumulator fragment.
struct EpiArgs {
  uint32_t m, n, mem_off, code_off;
};

__device__ __attribute__((noinline)) void run_epilogue(vf16 acc, const uint32_t *prog32, EpiArgs h, uint32_t batch0, uint32_t batch1,
                                                      uint32_t row_base, uint32_t col) {
  const uint32_t *code32 = prog32 + 2 * h.code_off;
  vf16 t0 = 0.0f, t1 = 0.0f;
  uint32_t mask = 0;
  uint32_t pc = 0;
  while (true) {
    const uint32_t w0 = uni(code32[2 * pc]);
    const uint32_t imm = uni(code32[2 * pc + 1]);
    ++pc;
    const uint32_t op = w0 & 0xffu;
    if (op == VOP_END) break;
    const uint32_t sub = (w0 >> 8) & 0xffu, a = w0 >> 24, rnd = (w0 >> 20) & 0x3u;
    if (op >= VOP_SRC_BASE || op == VOP_ST) {
      const uint32_t kind = op == VOP_ST ? static_cast<uint32_t>(VK_MEM) : ((w0 >> 16) & 0xfu);
      vf16 src;
      if (kind == VK_MEM) {
        const uint32_t *d = prog32 + 2 * h.mem_off + a * (sizeof(VCubeMem) / 4);
        const uint64_t addr = static_cast<uint64_t>(uni(d[0])) | (static_cast<uint64_t>(uni(d[1])) << 32);
        const uint32_t dtype = uni(d[2]), sn = uni(d[4]), sm = uni(d[5]), sb0 = uni(d[6]), sb1 = uni(d[7]);
        const uint64_t boff = static_cast<uint64_t>(batch0) * sb0 + static_cast<uint64_t>(batch1) * sb1;
        if (op == VOP_ST) {
          Frag f;
          f.v = acc;
          frag_store(addr, dtype, sn, sm, boff, row_base, col, h.m, h.n, f);
          continue;
        }
        src = frag_load(addr, dtype, sn, sm, boff, row_base, col, h.m, h.n).v;
      } else if (kind == VK_IMM) {
        src = __uint_as_float(imm);
      } else if (kind == VK_REG) {
        src = a == 0 ? t0 : t1;
      } else {
        src = acc;
      }
      switch (op) {
        case VOP_LD:
          acc = src;
          break;
        case VOP_BINF:
          switch (sub & 0x3fu) {
            case VB_ADD: acc = acc + src; break;
            case VB_SUB: acc = acc - src; break;
            case VB_RSUB: acc = src - acc; break;
            case VB_MUL: acc = acc * src; break;
            case VB_DIV: acc = acc / src; break;
            case VB_RDIV: acc = src / acc; break;
            case VB_MIN: FOR_R acc[r] = acc[r] < src[r] ? acc[r] : src[r]; break;
            case VB_MAX: FOR_R acc[r] = acc[r] > src[r] ? acc[r] : src[r]; break;
            case VB_AND: FOR_R acc[r] = (acc[r] != 0.0f && src[r] != 0.0f) ? 1.0f : 0.0f; break;
            case VB_OR: FOR_R acc[r] = (acc[r] != 0.0f || src[r] != 0.0f) ? 1.0f : 0.0f; break;
            case VB_POW: acc = frag_pow(acc, src); break;
            default: acc = frag_pow(src, acc); break;
          }
          apply_rnd(acc, rnd);
          break;
        case VOP_BINI:
          switch (sub & 0x3fu) {
            case VBI_ADD: FOR_R acc[r] = __uint_as_float(__float_as_uint(acc[r]) + __float_as_uint(src[r])); break;
            case VBI_SUB: FOR_R acc[r] = __uint_as_float(__float_as_uint(acc[r]) - __float_as_uint(src[r])); break;
            case VBI_RSUB: FOR_R acc[r] = __uint_as_float(__float_as_uint(src[r]) - __float_as_uint(acc[r])); break;
            case VBI_MUL: FOR_R acc[r] = __uint_as_float(__float_as_uint(acc[r]) * __float_as_uint(src[r])); break;
            case VBI_MIN: FOR_R acc[r] = __int_as_float(min(__float_as_int(acc[r]), __float_as_int(src[r]))); break;
            default: FOR_R acc[r] = __int_as_float(max(__float_as_int(acc[r]), __float_as_int(src[r]))); break;
          }
          break;
        case VOP_CMP: {
          const uint32_t t = sub & 0x7u;
          if (sub & VCMP_INT) {
            FOR_R {
              const int32_t x = __float_as_int(acc[r]), y = __float_as_int(src[r]);
              const bool c = t == VCMP_EQ ? x == y : t == VCMP_NE ? x != y : t == VCMP_GT ? x > y : t == VCMP_GE ? x >= y : t == VCMP_LT ? x < y : x <= y;
              acc[r] = __int_as_float(c ? 1 : 0);
            }
          } else {
            FOR_R {
              const float x = acc[r], y = src[r];
              const bool c = t == VCMP_EQ ? x == y : t == VCMP_NE ? x != y : t == VCMP_GT ? x > y : t == VCMP_GE ? x >= y : t == VCMP_LT ? x < y : x <= y;
              acc[r] = c ? 1.0f : 0.0f;
            }
          }
          break;
        }
        case VOP_MSK:
          mask = 0;
          FOR_R mask |= ((__float_as_uint(src[r]) << 1) != 0 ? 1u : 0u) << r;
          break;
        default:  // VOP_MOVM
          FOR_R acc[r] = ((mask >> r) & 1u) ? src[r] : acc[r];
          break;
      }
      continue;
    }
    switch (op) {
      case VOP_LDR:
        acc = a == 0 ? t0 : t1;
        break;
      case VOP_LDI:
        acc = __uint_as_float(imm);
        break;
      case VOP_STR:
        if (a == 0) {
          t0 = acc;
        } else {
          t1 = acc;
        }
        break;
      case VOP_UN:
        switch (sub) {
          case VU_SQRT: acc = frag_sqrt(acc); break;
          case VU_ABS: FOR_R acc[r] = fabsf(acc[r]); break;
          case VU_LOG: acc = frag_log(acc); break;
          case VU_EXP: acc = frag_exp(acc); break;
          case VU_ISFINITE: FOR_R acc[r] = isfinite(acc[r]) ? 1.0f : 0.0f; break;
          case VU_ROUND: FOR_R acc[r] = rintf(acc[r]); break;
          case VU_FLOOR: FOR_R acc[r] = floorf(acc[r]); break;
          case VU_CEIL: FOR_R acc[r] = ceilf(acc[r]); break;
          case VU_TRUNC: FOR_R acc[r] = truncf(acc[r]); break;
          default:
            FOR_R {
              const uint32_t x = __float_as_uint(acc[r]);
              acc[r] = __uint_as_float(static_cast<int32_t>(x) < 0 ? 0u - x : x);
            }
            break;
        }
        apply_rnd(acc, rnd);
        break;
      case VOP_CAST:
        if (sub == VC_F2I) {
          FOR_R acc[r] = __int_as_float(static_cast<int32_t>(acc[r]));
        } else if (sub == VC_I2F) {
          FOR_R acc[r] = static_cast<float>(__float_as_int(acc[r]));
          apply_rnd(acc, rnd);
        } else if (sub == VC_RND) {
          apply_rnd(acc, rnd);
        } else {
          FOR_R acc[r] = acc[r] != 0.0f ? 1.0f : 0.0f;
        }
        break;
      default:
        break;
    }
  }
}

// TM x TN 32x32 MFMA tiles per wave, 2 x 2 waves per workgroup.
template <bool IS_BF16, int TM, int TN>
__device__ __forceinline__ void vm_cube(const VmParam &p) {
  constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
  extern __shared__ double lds_raw[];
  __shared__ uint32_t prog32[DVM_PARAM_BYTES / 4];
  {
    const uint32_t *src = reinterpret_cast<const uint32_t *>(p.w);
    const uint32_t trips = (DVM_PARAM_BYTES / 4 + 255) / 256;
    for (uint32_t t = 0; t < trips; ++t) {
      uint32_t i = t * 256 + threadIdx.x;
      i = i < DVM_PARAM_BYTES / 4 ? i : DVM_PARAM_BYTES / 4 - 1;
      prog32[i] = src[i];
    }
    __syncthreads();
  }
  VCubeHeader h;
  {
    uint32_t *hw = reinterpret_cast<uint32_t *>(&h);
#pragma unroll
    for (int i = 0; i < static_cast<int>(sizeof(VCubeHeader) / 4); ++i) hw[i] = uni(prog32[i]);
  }
  uint16_t *lds = reinterpret_cast<uint16_t *>(lds_raw);
  // two buffers of [A tile | B tile]; offsets in elements from `lds`, so every access stays a local-memory access
  constexpr uint32_t kBufElems = (BM + BN) * LDS_ROW;
  constexpr uint32_t kBOff = BM * LDS_ROW;

  const uint32_t tid = threadIdx.x;
  const uint32_t wave = tid >> 6, lane = tid & 63u;
  const uint32_t wm = wave >> 1, wn = wave & 1u;
  const uint32_t tiles_per_batch = h.tiles_m * h.tiles_n;
  const uint32_t n_tiles = tiles_per_batch * h.nb0 * h.nb1;
  const uint32_t nk = (h.k + BK - 1) / BK;
  const bool a_kc = h.trans_a == 0, b_kc = h.trans_b != 0;

  for (uint32_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    const uint32_t batch = t / tiles_per_batch, tt = t % tiles_per_batch;
    const uint32_t bi0 = batch / h.nb1, bi1 = batch % h.nb1;
    // neighbouring workgroups share a row of A tiles: walk n fastest
    const uint32_t tm = tt / h.tiles_n, tn = tt % h.tiles_n;
    const uint32_t m0 = tm * BM, n0 = tn * BN;
    const uint64_t a_base = h.a_addr + (static_cast<uint64_t>(bi0) * h.a_sb0 + static_cast<uint64_t>(bi1) * h.a_sb1) * 2;
    const uint64_t b_base = h.b_addr + (static_cast<uint64_t>(bi0) * h.b_sb0 + static_cast<uint64_t>(bi1) * h.b_sb1) * 2;

    vf16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = 0.0f;

    if (h.fast && m0 + BM <= h.m && n0 + BN <= h.n) {
      Stage<BM> sa;
      Stage<BN> sb;
      if (a_kc) stage_load_kc<BM>(sa, a_base, h.lda, m0, 0, tid); else stage_load_ks<BM>(sa, a_base, h.lda, m0, 0, tid);
      if (b_kc) stage_load_kc<BN>(sb, b_base, h.ldb, n0, 0, tid); else stage_load_ks<BN>(sb, b_base, h.ldb, n0, 0, tid);
      if (a_kc) stage_store_kc<BM>(sa, lds, tid); else stage_store_ks<BM>(sa, lds, tid);
      if (b_kc) stage_store_kc<BN>(sb, lds + kBOff, tid); else stage_store_ks<BN>(sb, lds + kBOff, tid);
      __syncthreads();
      for (uint32_t kt = 0; kt < nk; ++kt) {
        const uint32_t cur = kt & 1u;
        const bool more = kt + 1 < nk;
        if (more) {
          const uint32_t k0 = (kt + 1) * BK;
          if (a_kc) stage_load_kc<BM>(sa, a_base, h.lda, m0, k0, tid); else stage_load_ks<BM>(sa, a_base, h.lda, m0, k0, tid);
          if (b_kc) stage_load_kc<BN>(sb, b_base, h.ldb, n0, k0, tid); else stage_load_ks<BN>(sb, b_base, h.ldb, n0, k0, tid);
        }
        const uint16_t *at = lds + cur * kBufElems + (wm * TM * 32 + (lane & 31u)) * LDS_ROW + (lane >> 5) * 8;
        const uint16_t *bt = lds + cur * kBufElems + kBOff + (wn * TN * 32 + (lane & 31u)) * LDS_ROW + (lane >> 5) * 8;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
          vu4 af[TM], bf[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const vu4 *>(at + i * 32 * LDS_ROW + kk * 16);
#pragma unroll
          for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const vu4 *>(bt + j * 32 * LDS_ROW + kk * 16);
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma<IS_BF16>(af[i], bf[j], acc[i][j]);
        }
        if (more) {
          if (a_kc) stage_store_kc<BM>(sa, lds + (cur ^ 1u) * kBufElems, tid); else stage_store_ks<BM>(sa, lds + (cur ^ 1u) * kBufElems, tid);
          if (b_kc) stage_store_kc<BN>(sb, lds + (cur ^ 1u) * kBufElems + kBOff, tid); else stage_store_ks<BN>(sb, lds + (cur ^ 1u) * kBufElems + kBOff, tid);
        }
        __syncthreads();
      }
    } else {
      for (uint32_t kt = 0; kt < nk; ++kt) {
        stage_generic<BM>(lds, a_base, h.lda, m0, kt * BK, h.m, h.k, a_kc ? 1u : 0u, tid);
        stage_generic<BN>(lds + kBOff, b_base, h.ldb, n0, kt * BK, h.n, h.k, b_kc ? 1u : 0u, tid);
        __syncthreads();
        const uint16_t *at = lds + (wm * TM * 32 + (lane & 31u)) * LDS_ROW + (lane >> 5) * 8;
        const uint16_t *bt = lds + kBOff + (wn * TN * 32 + (lane & 31u)) * LDS_ROW + (lane >> 5) * 8;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
          vu4 af[TM], bf[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const vu4 *>(at + i * 32 * LDS_ROW + kk * 16);
#pragma unroll
          for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const vu4 *>(bt + j * 32 * LDS_ROW + kk * 16);
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma<IS_BF16>(af[i], bf[j], acc[i][j]);
        }
        __syncthreads();
      }
    }

    // epilogue, fragment by fragment, straight from the accumulators
    const EpiArgs ea = {h.m, h.n, h.mem_off, h.code_off};
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t row_base = m0 + (wm * TM + i) * 32 + (lane >> 5) * 4;
        const uint32_t col = n0 + (wn * TN + j) * 32 + (lane & 31u);
        run_epilogue(acc[i][j], prog32, ea, bi0, bi1, row_base, col);
      }
    }
  }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(256) dvm_vm_cube_bf16_big(const VmParam p) { vm_cube<true, 4, 4>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_cube_f16_big(const VmParam p) { vm_cube<false, 4, 4>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_cube_bf16_mid(const VmParam p) { vm_cube<true, 2, 2>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_cube_f16_mid(const VmParam p) { vm_cube<false, 2, 2>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_cube_bf16_small(const VmParam p) { vm_cube<true, 1, 1>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_cube_f16_small(const VmParam p) { vm_cube<false, 1, 1>(p); }
