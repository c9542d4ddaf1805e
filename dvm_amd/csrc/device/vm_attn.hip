// gfx950 fused attention: two MFMA stages with the softmax between them, one launch.
//
// Role in the reference: none on any backend. The reference runs examples/03_attention.py:39-50 as
// three sub-kernels (Q K^T on the cube unit, the softmax as a vector kernel over the full score
// matrix, P V on the cube unit; the cut rule is src/xkernel.cc:2097-2107), so the [sq][skv] scores
// travel through memory twice. This kernel keeps them in registers:
//  * a workgroup (4 waves) owns 256 query rows of one (batch, head), a wave 64 of them; the keys are
//    walked in blocks of 64 with a running row max and row sum (online softmax);
//  * stage 1 computes the TRANSPOSED scores S^T = K Q^T with v_mfma_f32_32x32x16: in the MFMA result
//    layout a lane then holds one query (column) and 16 keys (rows) per tile, so the row max, the row
//    sum and the rescale factor of a query are per-lane values: no cross-lane reduction except one
//    exchange between the two half-waves;
//  * the probabilities go to the second MFMA straight from those registers: O^T += V^T P^T sums
//    over keys, and the order of that sum is free, so the keys a lane happens to hold are fed as they
//    are and the V^T fragment is read in the matching (permuted) key order;
//  * K and V blocks go from memory to local memory directly (global_load_lds_dwordx4), as they lie in
//    memory (head dimension contiguous), in the XOR-swizzled tile layout of the matmul kernel, double
//    buffered, block j+1 in flight during the whole of block j: no staging registers, no ds_write;
//  * the V^T fragments stage 2 needs (keys contiguous per lane) come out of that layout with
//    ds_read_b64_tr_b16, the transposing local-memory read of gfx950;
//  * Q fragments are read from memory once and stay in registers.
// Scores stay in fp32 between the stages (the three-kernel graph rounds them to the operand type);
// the result agrees with the NumPy golden of examples/03_attention.py:20-28 within its 1e-2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../isa_gfx950.h"

namespace {

#define DVM_GLOBAL __attribute__((address_space(1)))

typedef float vf16 __attribute__((ext_vector_type(16)));
typedef float vf2 __attribute__((ext_vector_type(2)));
typedef uint32_t vu4 __attribute__((ext_vector_type(4)));
typedef uint32_t vu2 __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

constexpr int BKV = DVM_ATTN_BKV;  // keys per block
constexpr int ROW = 64;            // elements per local-memory tile row (128 bytes)

__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

template <bool IS_BF16>
__device__ __forceinline__ vf16 mfma(vu4 a, vu4 b, vf16 c) {
  if constexpr (IS_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8 *>(&a), *reinterpret_cast<bf16x8 *>(&b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<half8 *>(&a), *reinterpret_cast<half8 *>(&b), c, 0, 0, 0);
  }
}

// 2^x for x <= 0 (scores minus their running maximum): the bare hardware instruction; results below the
// normal range flush to zero, which is what a softmax weight of that size amounts to anyway.
__device__ __forceinline__ float exp2_neg(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ bool wave_all(bool c) { return __builtin_amdgcn_ballot_w64(!c) == 0; }

template <bool IS_BF16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const vf2 v = {lo, hi};
  if constexpr (IS_BF16) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  } else {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, half2v));
  }
}

// Element offset of 16-byte chunk `chunk` (0..7) of row `row` in a tile of 64-element rows.
__device__ __forceinline__ uint32_t tile_off(uint32_t row, uint32_t chunk) {
  return row * ROW + ((chunk ^ ((row ^ (row >> 3)) & 7u)) << 3);
}

// Local memory per buffer: K block and V block, each as D / 64 tiles [64 keys][64 d] (two d halves at D = 128).
constexpr uint32_t kKTile = BKV * ROW;  // elements of one half tile

// NQT: 32-query tiles per wave. 2: four waves of 64 queries, one per SIMD with all 512 registers; 1: eight waves of
// 32 queries, two per SIMD, so that one wave's softmax (vector ALU) runs under the other's MFMAs.
// D: head dimension, 64 or 128.
template <bool IS_BF16, int NQT, int D>
__device__ __forceinline__ void vm_attn(const VmParam &p) {
  static_assert(D == 64 || D == 128, "head dimension");
  constexpr int HT = D / 64;                  // half tiles per K or V block
  constexpr uint32_t kVOff = HT * kKTile;     // V block after the K block
  constexpr uint32_t kBuf = 2 * HT * kKTile;  // elements per buffer
  constexpr int WQ = 32 * NQT;             // query rows per wave
#ifndef DVM_ATTN_PIN8
#define DVM_ATTN_PIN8 1
#endif
  constexpr bool PIN = NQT == 2 || DVM_ATTN_PIN8;
  constexpr uint32_t NTHR = 64u * (DVM_ATTN_BQ / WQ);
  extern __shared__ double lds_raw[];
  uint16_t *lds = reinterpret_cast<uint16_t *>(lds_raw);
  const VAttnHeader *hp = reinterpret_cast<const VAttnHeader *>(p.w);
  const uint32_t sq = hp->sq, skv = hp->skv, q_blocks = hp->q_blocks;
  const float scale = hp->scale;
  const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63u;
  const uint32_t lj = lane & 31u, lh = lane >> 5;
  // Workgroups are dealt to the 8 XCDs round robin and each XCD has its own L2: workgroup w takes position
  // (w % 8) * (grid / 8) + w / 8 of the (head, query block) order, so the query blocks of one head, which
  // all read the same K and V, run on one XCD at the same time and share them in its L2.
  uint32_t pos = blockIdx.x;
  if ((gridDim.x & 7u) == 0) pos = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const uint32_t b = pos / q_blocks, qb = pos % q_blocks;
  // the (batch, head) pair's matrices: strides in elements from the header (views are read in place)
  const uint32_t b_out = b / hp->nb_inner, b_in = b % hp->nb_inner;
  auto base_of = [&](uint64_t addr, int which) -> uint64_t {
    return addr + (static_cast<uint64_t>(b_out) * hp->outer_stride[which] + static_cast<uint64_t>(b_in) * hp->inner_stride[which]) * 2;
  };
  const uint64_t q_base = base_of(hp->q_addr, 0), k_base = base_of(hp->k_addr, 1), v_base = base_of(hp->v_addr, 2), o_base = base_of(hp->o_addr, 3);
  const uint32_t ldq = hp->row_stride[0], ldk = hp->row_stride[1], ldv = hp->row_stride[2], ldo = hp->row_stride[3];
  const uint32_t q0 = qb * DVM_ATTN_BQ + wave * WQ;

  // Q fragments (B operand of stage 1): lane (j, h) holds Q[q0 + 32*qt + j][16*kk + 8*h .. +7]; rows
  // past the end repeat the last row (their results are never stored)
  vu4 qf[NQT][D / 16];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    uint32_t row = q0 + 32 * qt + lj;
    row = row < sq ? row : sq - 1;
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk)
      qf[qt][kk] = *reinterpret_cast<const DVM_GLOBAL vu4 *>(q_base + (static_cast<uint64_t>(row) * ldq + 16 * kk + 8 * lh) * 2);
  }

  // Staging. A block of K or V is 64 keys x 128 d = two half tiles (d < 64, d >= 64) of 64 rows x 8 chunks of
  // 16 bytes. Chunk position p = NTHR*i + tid of a block is half tile p/512, key (p%512)/8, physical chunk tid%8
  // (with 256 lanes: half tile i/2, key 32*(i&1) + tid/8; with 512: half tile i, key tid/8); the lane fetches
  // the logical chunk that belongs there (physical ^ swizzle(key)), and a wave's 64 chunks land in 1 KB of
  // consecutive local memory.
  constexpr uint32_t KPS = NTHR / 8;       // keys one step of all lanes covers
  constexpr int STEPS = 64 / KPS;          // steps per half tile
  uint32_t col_off[2];  // byte offset of the lane's chunk inside its row, for even / odd steps
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    const uint32_t key = KPS * par + (tid >> 3);
    const uint32_t logical = (tid & 7u) ^ ((key ^ (key >> 3)) & 7u);
    col_off[par] = (logical << 3) * 2u;
  }
  const uint32_t wave_first = uni(wave) * 64u;
  // (a last block with fewer than BKV keys: the rows past the end fetch the last key again, their scores are masked)
  auto fetch_kv = [&](uint32_t key0, uint32_t buf) {
    uint16_t *kdst = lds + buf * kBuf, *vdst = lds + buf * kBuf + kVOff;
    const DVM_GLOBAL char *ksrc = reinterpret_cast<const DVM_GLOBAL char *>(k_base + static_cast<uint64_t>(key0) * ldk * 2);
    const DVM_GLOBAL char *vsrc = reinterpret_cast<const DVM_GLOBAL char *>(v_base + static_cast<uint64_t>(key0) * ldv * 2);
    const uint32_t last_row = skv - 1u - key0;  // uniform; BKV - 1 or more in a full block
#pragma unroll
    for (int i = 0; i < HT * STEPS; ++i) {
      // step i % STEPS of half tile i / STEPS: later keys, then d 64..
      uint32_t row = (i % STEPS) * KPS + (tid >> 3);
      if (last_row < static_cast<uint32_t>(BKV) - 1u) row = row > last_row ? last_row : row;
      const uint32_t col = (i / STEPS) * 64u * 2u + col_off[(i % STEPS) & 1];
      const uint32_t dst_off = (static_cast<uint32_t>(i) * NTHR + wave_first) * 8u;
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const DVM_GLOBAL void *>(ksrc + (row * ldk * 2u + col)), (__attribute__((address_space(3))) void *)(kdst + dst_off), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const DVM_GLOBAL void *>(vsrc + (row * ldv * 2u + col)), (__attribute__((address_space(3))) void *)(vdst + dst_off), 16, 0, 0);
    }
  };

  vf16 o_acc[D / 32][NQT];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) o_acc[dt][qt] = 0.0f;
  float m_run[NQT], l_run[NQT];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    m_run[qt] = -1.0e30f;
    l_run[qt] = 0.0f;
  }
  const float c_log2 = scale * 1.44269504088896340736f;  // scores are handled in the log2 domain

  // Fragment reads. For row = 32*t + j of a tile the swizzle is swz0 ^ 4*(t & 1) with swz0 = (j ^ j>>3) & 7,
  // so every read address is a per-lane base plus (x ^ constant) plus a constant: no register per address.
  const uint32_t swz0 = (lj ^ (lj >> 3)) & 7u;
  const uint32_t lane_row = lj * ROW;
  const uint32_t k_x = (lh ^ swz0) << 3;  // K fragment: chunk 2*(kk&3) + h
  // V^T fragments through ds_read_b64_tr_b16. Within a group of 16 lanes, lane r = 4*j + q supplies the
  // address of 4 consecutive d of key K_j, and lane i of the group receives d0 + i of K_0..K_3. Groups
  // 0/1 take d0 = 0/16 of a 32-wide d tile for the keys of half-wave 0, groups 2/3 the same for half-wave
  // 1 (the half-waves' keys differ by 4, as in the score registers).
  const uint32_t tr_j = (lane & 15u) >> 2, tr_q = lane & 3u, tr_g = lane >> 4;
  const uint32_t tr_key = 4u * (tr_g >> 1) + tr_j;                 // key inside its group of 8 (low 3 bits)
  const uint32_t tr_chunk = 2u * (tr_g & 1u) + (tr_q >> 1);          // 16-byte chunk inside the half d tile
  const uint32_t tr_base = tr_key * ROW + 4u * (tr_q & 1u);          // row part + the half of the chunk
  const uint32_t tr_x = (tr_chunk ^ tr_key) << 3;
  const uint32_t n_blocks = (skv + BKV - 1) / BKV;
  fetch_kv(0, 0);
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0): the barrier does not wait for direct loads by itself
  __syncthreads();
  vf16 s[2][NQT];
  vu4 pf[2][2][NQT];  // [key tile][16-key step][query tile]: B operand of stage 2
  // stage 1: S^T[key][query] for 2 key tiles x NQT query tiles. The fragments of step kk+1 are read while the
  // MFMAs of step kk run (pinned: with one wave per SIMD nothing else would hide the local-memory latency).
  auto stage1 = [&](const uint16_t *kbuf) {
    vu4 kf[2][2];
    auto read_k = [&](int fb, int kk) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
        kf[fb][kt] = *reinterpret_cast<const vu4 *>(kbuf + (kk >> 2) * kKTile + kt * 32 * ROW + lane_row + (k_x ^ static_cast<uint32_t>((((kk & 3) * 2) ^ (4 * kt)) << 3)));
    };
    read_k(0, 0);
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
      __builtin_amdgcn_sched_barrier(0);
      if (kk + 1 < D / 16) read_k((kk + 1) & 1, kk + 1);
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
          if (kk == 0) {
            const vf16 zero = 0.0f;
            s[kt][qt] = mfma<IS_BF16>(kf[0][kt], qf[qt][0], zero);
          } else {
            s[kt][qt] = mfma<IS_BF16>(kf[kk & 1][kt], qf[qt][kk], s[kt][qt]);
          }
        }
      if (kk + 1 < D / 16 && PIN) {  // the two fragment reads of the next step between the 2 * NQT MFMAs of this one
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (NQT == 2) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // softmax of a block, per query (= per lane, both half-waves share a query)
  auto softmax = [&]() {
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      float mx = s[0][qt][0];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kt][qt][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run[qt], mx * c_log2);
      const float alpha = exp2_neg(m_run[qt] - m_new);
      m_run[qt] = m_new;
      float sum = 0.0f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float pv = exp2_neg(s[kt][qt][r] * c_log2 - m_new);
          s[kt][qt][r] = pv;
          sum += pv;
        }
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int e = 0; e < 4; ++e) pf[kt][st][qt][e] = pack2<IS_BF16>(s[kt][qt][8 * st + 2 * e], s[kt][qt][8 * st + 2 * e + 1]);
      }
      l_run[qt] = l_run[qt] * alpha + sum;
      // after the first blocks the running maximum rarely moves: skip the rescale when no lane needs it
      if (!wave_all(alpha == 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) o_acc[dt][qt] = o_acc[dt][qt] * alpha;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // stage 2: O^T[d][query] += V^T[d][key] P^T[key][query]. Step (kt, st) contracts the 16 keys the
  // lane's registers 8*st .. 8*st+7 of tile kt hold: keys 32*kt + 16*st + {0..3, 8..11} + 4*h. Fragments
  // of the next step are read under the MFMAs of the current one.
  auto stage2 = [&](const uint16_t *vbuf) {
    vu4 vf[2][D / 32];
    auto read_v = [&](int fb, int step) {
      const int kt = step >> 1, st = step & 1;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt) {
        // keys C + tr_key and C + 8 + tr_key, C = 32*kt + 16*st; swizzle(key) = (key & 7) ^ ((key >> 3) & 7), chunk =
        // 4*(dt & 1) | tr_chunk: every address is a lane base plus (tr_x ^ constant) plus a constant
        vu2 part[2];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const int c = kt * 32 + st * 16 + w * 8;
          const uint16_t *ptr = vbuf + (dt >> 1) * kKTile + c * ROW + tr_base + (tr_x ^ static_cast<uint32_t>(((4 * (dt & 1)) ^ ((c >> 3) & 7)) << 3));
          part[w] = __builtin_bit_cast(vu2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(ptr)));
        }
        vf[fb][dt] = vu4{part[0][0], part[0][1], part[1][0], part[1][1]};
      }
    };
    read_v(0, 0);
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      __builtin_amdgcn_sched_barrier(0);
      if (step + 1 < 4) read_v((step + 1) & 1, step + 1);
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) o_acc[dt][qt] = mfma<IS_BF16>(vf[step & 1][dt], pf[step >> 1][step & 1][qt], o_acc[dt][qt]);
      if (step + 1 < 4 && PIN) {  // the eight transposing reads of the next step between the 4 * NQT MFMAs of this one
#pragma unroll
        for (int q = 0; q < (D / 32) * NQT; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2 / NQT, 0);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // Running the waves that share a SIMD one phase apart (softmax and stage 2 of block kb-1, then stage 1 of block
  // kb, with a third K/V buffer) was measured with eight waves and is slower (819-835 us against 767-788 us): the
  // hardware interleaves the two waves well enough, and the rotation costs 50 registers.
  for (uint32_t kb = 0; kb < n_blocks; ++kb) {
    const uint32_t cur = kb & 1u;
    // the other buffer was read for the last time before the barrier that ended the previous block
    if (kb + 1 < n_blocks) fetch_kv((kb + 1) * BKV, cur ^ 1u);
    stage1(lds + cur * kBuf);
    if (kb * BKV + BKV > skv) {
      // keys past the end: register r of key tile kt holds key 32*kt + 8*(r/4) + 4*h + r%4 of the block (scale > 0)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const uint32_t key = kb * BKV + 32u * kt + 8u * (r >> 2) + 4u * lh + (r & 3);
#pragma unroll
          for (int qt = 0; qt < NQT; ++qt) s[kt][qt][r] = key < skv ? s[kt][qt][r] : -1.0e30f;
        }
    }
    softmax();
    stage2(lds + cur * kBuf + kVOff);
    __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0): the next block has landed
    __syncthreads();
  }

  // O[query][d] = O^T / l, rounded once to the operand type. Lane (j, h) holds, per d tile and register
  // group g, d = 32*dt + 8*g + 4*h + 0..3: four consecutive values = one 8-byte store.
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const float l = l_run[qt] + __shfl_xor(l_run[qt], 32);
    const float inv = 1.0f / l;
    const uint32_t row = q0 + 32 * qt + lj;
    if (row < sq) {
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          vu2 w;
          w[0] = pack2<IS_BF16>(o_acc[dt][qt][4 * g] * inv, o_acc[dt][qt][4 * g + 1] * inv);
          w[1] = pack2<IS_BF16>(o_acc[dt][qt][4 * g + 2] * inv, o_acc[dt][qt][4 * g + 3] * inv);
          *reinterpret_cast<DVM_GLOBAL vu2 *>(o_base + (static_cast<uint64_t>(row) * ldo + dt * 32 + 8 * g + 4 * lh) * 2) = w;
        }
      }
    }
  }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(256) dvm_vm_attn_f16(const VmParam p) { vm_attn<false, 2, 128>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_attn_bf16(const VmParam p) { vm_attn<true, 2, 128>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_attn_f16_w8(const VmParam p) { vm_attn<false, 1, 128>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_attn_bf16_w8(const VmParam p) { vm_attn<true, 1, 128>(p); }
// head dimension 64
extern "C" __global__ void __launch_bounds__(256) dvm_vm_attn_f16_d64(const VmParam p) { vm_attn<false, 2, 64>(p); }
extern "C" __global__ void __launch_bounds__(256) dvm_vm_attn_bf16_d64(const VmParam p) { vm_attn<true, 2, 64>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_attn_f16_w8_d64(const VmParam p) { vm_attn<false, 1, 64>(p); }
extern "C" __global__ void __launch_bounds__(512) dvm_vm_attn_bf16_w8_d64(const VmParam p) { vm_attn<true, 1, 64>(p); }
