// gfx950 matmul VM: MFMA tile loop followed by an interpreted epilogue on the tile, before anything
// reaches memory.
//
// Role in the reference: the cube kernels (device semantics src/vm_aic.cce:34-470: fp32
// accumulation, one rounding to the operand type on write-out) plus the mix kernel's post-fusion
// vector program (src/xkernel.cc:304-360). The reference's CUDA backend has no matmul at all
// (src/system.cc:290-294); this kernel is specific to CDNA4:
//  * v_mfma_f32_32x32x16 (bf16 / f16), 64-wide waves, WM x 2 waves per workgroup, each wave owning a
//    (TM*32) x (TN*32) block of fp32 accumulators that stays in registers for the whole k loop;
//  * the 256x256 tile (four or eight waves) walks k in stages of 32 through a ring of four stage buffers in
//    local memory, every operand layout a straight direct-to-LDS copy (global_load_lds_dwordx4), the k-strided
//    ones read back through ds_read_b64_tr_b16 (tile_loop_ring below);
//  * the 128x128 and 64x64 tiles stage 64 k at a time, double buffered, k contiguous in local memory: rows of
//    128 bytes whose eight 16-byte chunks are XOR-swizzled by the row number; operands whose k axis is strided in
//    memory (B of an NN product, A of a TN product) are transposed in registers there, 8x8 elements per lane;
//  * fragments are double buffered in registers: the reads of step s+1 are in flight while the MFMAs of step s run;
//  * the epilogue runs in two passes over half tiles: accumulators go to local memory once, row
//    major, and come back as slabs of 8 consecutive columns per lane, so every memory operand of the
//    epilogue and every store is a coalesced 128-bit access; the epilogue program is the vector
//    VM's instruction words, decoded wave-uniformly.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../isa_gfx950.h"

namespace {

#define DVM_GLOBAL __attribute__((address_space(1)))

typedef float vf16 __attribute__((ext_vector_type(16)));
typedef float vf4 __attribute__((ext_vector_type(4)));
typedef uint32_t vu4 __attribute__((ext_vector_type(4)));
typedef uint32_t vu2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

constexpr int BK = 64;   // k extent of a staged tile = one 128-byte row of 16-bit elements
constexpr int NTEMP = DVM_CUBE_NTEMP;

__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

__device__ __forceinline__ float round_f16(float x) { return static_cast<float>(static_cast<_Float16>(x)); }
// gfx950 converts fp32 to bf16 in hardware (round to nearest even, NaN stays NaN): v_cvt_pk_bf16_f32
typedef float vf2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float x) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x)); }
__device__ __forceinline__ float round_bf16(float x) { return static_cast<float>(static_cast<__bf16>(x)); }
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const vf2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  const vf2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, half2v));
}

template <bool IS_BF16>
__device__ __forceinline__ vf16 mfma(vu4 a, vu4 b, vf16 c) {
  if constexpr (IS_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8 *>(&a), *reinterpret_cast<bf16x8 *>(&b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<half8 *>(&a), *reinterpret_cast<half8 *>(&b), c, 0, 0, 0);
  }
}

// Element offset of 16-byte chunk `chunk` (0..7) of row `row` inside a staged tile.
__device__ __forceinline__ uint32_t tile_off(uint32_t row, uint32_t chunk) {
  return row * BK + ((chunk ^ ((row ^ (row >> 3)) & 7u)) << 3);
}

// ---- staging one operand tile: ROWS rows (m or n) x BK (k) ---------------------------------------------
// KC source (k contiguous in memory: A when !trans_a, B when trans_b): the tile is a straight copy, so it
// goes from memory to local memory directly (global_load_lds_dwordx4: a wave's 64 x 16 bytes land in 1 KB
// of consecutive local memory, the swizzle is applied by choosing which chunk each lane fetches); no
// registers, no ds_write, and the data may be in flight for a whole k tile.
// KS source (k strided, the row index contiguous): 8x8 element blocks through registers, transposed on
// the way (v_perm_b32), then written with ds_write_b128.
struct LaneOffsets {
  int32_t v[2];  // (signed: a row that is clamped back inside the operand lies before the row the loop would fetch)
};

template <int ROWS, bool KC, int NTHR>
struct Stage;

template <int ROWS, int NTHR>
struct Stage<ROWS, true, NTHR> {
  static constexpr int N = ROWS * BK / 8 / NTHR;  // 16-byte chunks per thread
  static constexpr uint32_t RPS = NTHR / 8;        // rows one step of all threads covers
  static constexpr int N_LOADS = N, N_WRITES = 0;

  // Chunk position p = NTHR*i + tid of the tile holds row p/8, logical chunk (p%8) ^ swizzle(row): with
  // row = RPS*i + tid/8 the swizzle depends at most on the parity of i (RPS = 32; not at all for 64), hence
  // two byte offsets per lane.
  // rows_valid < ROWS (a tile of which only the first rows lie inside the operand; tiles of at most two chunks per
  // lane only): the rows past the end fetch the last valid row instead, so that no load leaves the operand; what
  // they feed are accumulator rows the epilogue never stores.
  static constexpr bool kCanClamp = N <= 2;
  static __device__ __forceinline__ LaneOffsets lane_offset(uint32_t ld, uint32_t tid, uint32_t rows_valid = ROWS) {
    LaneOffsets o;
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      const uint32_t row = RPS * par + (tid >> 3);
      const uint32_t logical = (tid & 7u) ^ ((row ^ (row >> 3)) & 7u);
      uint32_t from = tid >> 3;  // row fetched, relative to the first row of chunk `par`
      int32_t back = 0;
      if (kCanClamp && row >= rows_valid) back = static_cast<int32_t>(rows_valid - 1u) - static_cast<int32_t>(row);
      o.v[par] = (static_cast<int32_t>(from) + back) * static_cast<int32_t>(ld * 2u) + static_cast<int32_t>((logical << 3) * 2u);
    }
    return o;
  }

  // origin: address of element (row0, k0) of the operand
  __device__ __forceinline__ void fetch(uint64_t origin, uint32_t ld, const LaneOffsets &lane, uint32_t tid, uint16_t *tile) {
    const DVM_GLOBAL char *base = reinterpret_cast<const DVM_GLOBAL char *>(origin);
    const uint32_t wave_first = uni(tid >> 6) * 64u;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const DVM_GLOBAL char *src = base + (static_cast<int64_t>(static_cast<uint64_t>(i) * RPS * ld * 2u) + lane.v[i & 1]);
      uint16_t *dst = tile + (static_cast<uint32_t>(i) * NTHR + wave_first) * 8u;
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const DVM_GLOBAL void *>(src), (__attribute__((address_space(3))) void *)(dst), 16, 0, 0);
    }
  }
  __device__ __forceinline__ void commit(uint16_t *, uint32_t) const {}
};

template <int ROWS, int NTHR>
struct Stage<ROWS, false, NTHR> {
  static_assert(ROWS <= 256, "one 8x8 block per thread, the first ROWS threads");
  // 8 (k) x 8 (rows) element blocks, ROWS of them per tile. With 256 lanes one lane takes a whole block; with 512
  // lanes and 256 rows two lanes share one, each taking 4 of its rows (8-byte loads, half the registers).
  static constexpr int TPB = (NTHR == 512 && ROWS == 256) ? 2 : 1;  // lanes per block
  static constexpr int RPT = 8 / TPB;                               // rows of the block a lane owns
  static constexpr int N = 8;
  static constexpr int N_LOADS = 8, N_WRITES = RPT;
  typedef uint32_t Row __attribute__((ext_vector_type(RPT / 2)));   // RPT 16-bit elements of one k
  Row r[N];

  static __device__ __forceinline__ bool active(uint32_t tid) { return (ROWS * TPB == NTHR) || tid < ROWS * TPB; }

  static __device__ __forceinline__ LaneOffsets lane_offset(uint32_t ld, uint32_t tid) {
    const uint32_t blk = tid / TPB, part = tid % TPB;
    const uint32_t kb = blk / (ROWS / 8), rb = blk % (ROWS / 8);
    LaneOffsets o;
    o.v[0] = o.v[1] = static_cast<int32_t>((kb * 8u * ld + rb * 8u + part * RPT) * 2u);
    return o;
  }

  __device__ __forceinline__ void fetch(uint64_t origin, uint32_t ld, const LaneOffsets &lane, uint32_t tid, uint16_t *) {
    const DVM_GLOBAL char *base = reinterpret_cast<const DVM_GLOBAL char *>(origin);
    if (active(tid)) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        r[j] = *reinterpret_cast<const DVM_GLOBAL Row *>(base + static_cast<uint64_t>(j) * ld * 2u + lane.v[0]);
      }
    }
  }

  __device__ __forceinline__ void commit(uint16_t *tile, uint32_t tid) const {
    if (active(tid)) {
      const uint32_t blk = tid / TPB, part = tid % TPB;
      const uint32_t kb = blk / (ROWS / 8), rb = blk % (ROWS / 8);
      // r[j] holds k = kb*8 + j, rows rb*8 + part*RPT .. +RPT-1; the tile wants, per row, k = kb*8 .. +7
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        vu4 o;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const uint32_t lo = r[2 * jj][i >> 1], hi = r[2 * jj + 1][i >> 1];
          // bytes of the result, least significant first: (i odd ? upper : lower) half of lo, then of hi
          o[jj] = __builtin_amdgcn_perm(hi, lo, (i & 1) ? 0x07060302u : 0x05040100u);
        }
        *reinterpret_cast<vu4 *>(tile + tile_off(rb * 8 + part * RPT + i, kb)) = o;
      }
    }
  }
};

// Generic staging of one tile straight into local memory (edge tiles, odd leading dimensions, unaligned
// operands, a k axis that is no multiple of 64). The unit is a run of 8 elements that are consecutive in memory:
// 8 k of one row (k contiguous) or 8 rows at one k (rows contiguous); a run that lies inside the operand and is
// 16-byte aligned (vec_ok: leading dimension a multiple of 8 and an aligned base) is one 128-bit load, any other
// run goes element by element and reads as zero outside the operand. Slow next to the tile loops, correct for
// every shape.
template <int ROWS, int NTHR>
__device__ __attribute__((noinline)) void stage_generic(uint16_t *tile, uint64_t base, uint32_t ld, uint32_t row0, uint32_t k0,
                                                        uint32_t rows, uint32_t kext, uint32_t k_contig, uint32_t vec_ok, uint32_t tid) {
  const DVM_GLOBAL uint16_t *src = reinterpret_cast<const DVM_GLOBAL uint16_t *>(base);
  if (k_contig) {
    for (uint32_t c = tid; c < ROWS * (BK / 8); c += NTHR) {
      const uint32_t row = c >> 3, kc = c & 7u;
      const uint32_t gr = row0 + row, gk = k0 + kc * 8u;
      vu4 v = {0u, 0u, 0u, 0u};
      if (gr < rows && gk < kext) {
        const uint64_t idx = static_cast<uint64_t>(gr) * ld + gk;
        if (vec_ok != 0u && (gk & 7u) == 0u && gk + 8u <= kext) {  // (a group's k range may start anywhere)
          v = *reinterpret_cast<const DVM_GLOBAL vu4 *>(src + idx);
        } else {
#pragma unroll
          for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t e = gk + j < kext ? src[idx + j] : 0u;
            v[j >> 1] |= e << (16u * (j & 1u));
          }
        }
      }
      *reinterpret_cast<vu4 *>(tile + tile_off(row, kc)) = v;
    }
  } else {
    // consecutive lanes take consecutive runs of rows at one k: neighbouring 16 bytes of memory
    const uint32_t row_vec = vec_ok != 0u && (row0 & 7u) == 0u ? 1u : 0u;
    for (uint32_t c = tid; c < (ROWS / 8) * BK; c += NTHR) {
      const uint32_t rb = c % (ROWS / 8), kk = c / (ROWS / 8);
      const uint32_t gr = row0 + rb * 8u, gk = k0 + kk;
      vu4 v = {0u, 0u, 0u, 0u};
      if (gr < rows && gk < kext) {
        const uint64_t idx = static_cast<uint64_t>(gk) * ld + gr;
        if (row_vec != 0u && gr + 8u <= rows) {
          v = *reinterpret_cast<const DVM_GLOBAL vu4 *>(src + idx);
        } else {
#pragma unroll
          for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t e = gr + j < rows ? src[idx + j] : 0u;
            v[j >> 1] |= e << (16u * (j & 1u));
          }
        }
      }
#pragma unroll
      for (uint32_t j = 0; j < 8; ++j) tile[tile_off(rb * 8u + j, kk >> 3) + (kk & 7u)] = static_cast<uint16_t>(v[j >> 1] >> (16u * (j & 1u)));
    }
  }
}

// ---- the 256x256 tile on four waves: stages of 32 k, four of them in local memory ---------------------
// A stage holds 256 rows x 32 k of each operand (16 KB + 16 KB); four stage buffers make a ring. While
// stage s is multiplied, the direct loads of stages s+1 and s+2 are in flight and those of stage s+3 are
// issued, a few at a time between the MFMAs, into the buffer stage s-1 has just left: every load has two
// full stages (64 MFMAs per wave) to arrive before anyone waits for it, and the four waves never send
// their loads in one burst. Both operand layouts are straight copies:
//  * k contiguous in memory (A, or B of a product with trans_b): rows of 32 k = 64 bytes = four 16-byte
//    chunks, chunk c of row r stored at chunk c ^ ((r >> 2) & 3): the 16 rows that one quarter of a fragment read
//    touches (16 lanes x 16 bytes = all 64 banks once) then sit in 16 different bank groups; one ds_read_b128 per lane;
//  * k strided (B, or A of a product with trans_a): the tile is stored as it lies in memory, 32 k rows of
//    256 elements (512 bytes, 32 chunks), chunk c of k row kr stored at chunk c ^ kswz(kr & 3); a fragment is
//    two ds_read_b64_tr_b16 per lane, which transpose 4 k x 16 rows inside each group of 16 lanes.
// kswz = {0, 10, 4, 14}: the four k rows one transposing read touches land in four different 32-byte
// columns of a 128-byte window, and the two 16-lane groups of a half-wave in different halves of 256 bytes.
constexpr int SK = 32;                           // k extent of a stage
constexpr uint32_t kStageOperand = 256 * SK;     // elements of one operand in a stage buffer
constexpr uint32_t kStageBuf = 2 * kStageOperand;

__device__ __forceinline__ uint32_t kc_swz(uint32_t row) { return (row >> 2) & 3u; }
__device__ __forceinline__ uint32_t ks_swz(uint32_t krow) { return (((krow & 3u) + 4u * (krow & 1u)) << 1); }

template <bool KC, int NTHR>
struct StageLoad {
  static constexpr int N = 1024 / NTHR;  // 16-byte chunks per lane: 256 rows x 64 bytes over the workgroup
  uint32_t lane_off;  // byte offset of the lane's first chunk from the tile's origin
  uint32_t step;      // byte distance between the lane's chunks

  __device__ __forceinline__ void init(uint32_t ld, uint32_t tid) {
    if constexpr (KC) {
      // chunk position p = NTHR*i + tid: row p/4, physical chunk p%4 (NTHR/4 = 64 or 128 rows further do not change the swizzle)
      const uint32_t row = tid >> 2;
      lane_off = row * ld * 2u + (((tid & 3u) ^ kc_swz(row)) << 4);
      step = (NTHR / 4u) * ld * 2u;
    } else {
      // chunk position p = NTHR*i + tid: k row p/32, physical chunk p%32
      const uint32_t kr = tid >> 5;
      lane_off = kr * ld * 2u + (((tid & 31u) ^ ks_swz(kr)) << 4);
      step = (NTHR / 32u) * ld * 2u;
    }
  }
  // origin: address of element (row0, k0) of the operand; dst: the operand's part of a stage buffer
  template <int I>
  __device__ __forceinline__ void issue(uint64_t origin, uint32_t wave_first, uint16_t *dst) const {
    const DVM_GLOBAL char *src = reinterpret_cast<const DVM_GLOBAL char *>(origin) + (lane_off + static_cast<uint32_t>(I) * step);
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const DVM_GLOBAL void *>(src),
                                     (__attribute__((address_space(3))) void *)(dst + (static_cast<uint32_t>(I) * NTHR + wave_first) * 8u), 16, 0, 0);
  }
};

// Fragment reads of one operand for one wave (r0: first of its rows). The reads are written as assembly:
// behind a read the compiler knows about, it waits for every direct load in flight (it cannot tell that the
// load writes another stage buffer), which would drain the ring; the price is that the loop waits for its
// reads by hand (once per step, lgkmcnt(0), with the fragment registers as operands of the wait so that no
// MFMA can move above it).
__device__ __forceinline__ uint32_t lds_byte_address(const void *ptr) {
  return static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) const char *)(ptr)));
}

template <bool KC>
struct FragAddr {
  uint32_t x[4];  // byte offsets inside the operand's part of a stage buffer

  __device__ __forceinline__ void init(uint32_t r0, uint32_t lane) {
    if constexpr (KC) {
      // fragment f, step kk: row r0 + 32f + lane%32, chunk (2kk + lane/32) ^ swz(row); x[kk] for f = 0
      const uint32_t j = lane & 31u, hh = lane >> 5;
      const uint32_t sw = kc_swz(j);  // r0 (a multiple of 64) and 32f do not change it
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) x[kk] = ((r0 + j) * SK + (((2u * kk + hh) ^ sw) << 3)) * 2u;
      x[2] = x[3] = 0;
    } else {
      // fragment f, step kk, half w: the lane supplies k row 16kk + 8*(g>>1) + 4w + jj and the four elements
      // r0 + 32f + 16*(g&1) + 4q .. +3, with g = lane/16, jj = (lane%16)/4, q = lane%4; x[f] for kk = w = 0
      const uint32_t g = lane >> 4, jj = (lane & 15u) >> 2, q = lane & 3u;
      const uint32_t kr = 8u * (g >> 1) + jj;
      const uint32_t sw = ks_swz(jj);
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        const uint32_t chunk = (r0 >> 3) + 4u * f + 2u * (g & 1u) + (q >> 1);
        x[f] = (kr * 256u + ((chunk ^ sw) << 3) + 4u * (q & 1u)) * 2u;
      }
    }
  }
  // base: byte address in local memory of the operand's part of the stage buffer
  template <int F, int KK>
  __device__ __forceinline__ vu4 read(uint32_t base) const {
    if constexpr (KC) {
      vu4 r;
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(base + x[KK]), "n"(F * 32 * SK * 2));
      return r;
    } else {
      vu2 lo, hi;
      const uint32_t addr = base + x[F];
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "n"(KK * 16 * 512));
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(KK * 16 * 512 + 4 * 512));
      return vu4{lo[0], lo[1], hi[0], hi[1]};
    }
  }
};

// The tile loop for WM x 2 waves (WM = 2: 128x128 accumulators per wave, one wave per SIMD; WM = 4: 64x128,
// two per SIMD). a_org / b_org: address of element (m0, 0) of A and (n0, 0) of B; nks: stages (k / 32 >= 2).
template <bool IS_BF16, bool A_KC, bool B_KC, int WM>
__device__ __forceinline__ void tile_loop_ring(vf16 (&acc)[8 / WM][4], uint16_t *lds, uint64_t a_org, uint64_t b_org, uint32_t lda,
                                               uint32_t ldb, uint32_t nks, uint32_t tid) {
  constexpr int NTHR = WM * 128, TM = 8 / WM, TN = 4;
  constexpr int NL = StageLoad<true, NTHR>::N;  // loads per lane, operand and stage
  constexpr int BPG = TN / TM;                  // B fragments a group reads
  static_assert(NL == TM && (NL == 2 || NL == 4), "one A or B load pair per group");
  const uint32_t wave = tid >> 6, lane = tid & 63u;
  const uint32_t wm = wave >> 1, wn = wave & 1u;
  const uint32_t wave_first = uni(wave) * 64u;
  StageLoad<A_KC, NTHR> la;
  StageLoad<B_KC, NTHR> lb;
  la.init(lda, tid);
  lb.init(ldb, tid);
  FragAddr<A_KC> fa;
  FragAddr<B_KC> fb;
  fa.init(wm * (TM * 32u), lane);
  fb.init(wn * 128u, lane);
  const uint64_t a_adv = (A_KC ? static_cast<uint64_t>(SK) : static_cast<uint64_t>(SK) * lda) * 2;
  const uint64_t b_adv = (B_KC ? static_cast<uint64_t>(SK) : static_cast<uint64_t>(SK) * ldb) * 2;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;

  // group g of a stage (TM groups) sends 2 * NL / TM = two of the lane's loads: the first half of the groups
  // A's, the second half B's
  auto issue_pair = [&](uint32_t st, auto group) {
    constexpr int G = decltype(group)::value;
    uint16_t *buf = lds + (st & 3u) * kStageBuf;
    if constexpr (2 * G < TM) {
      const uint64_t ao = a_org + st * a_adv;
      la.template issue<2 * G>(ao, wave_first, buf);
      la.template issue<2 * G + 1>(ao, wave_first, buf);
    } else {
      const uint64_t bo = b_org + st * b_adv;
      lb.template issue<2 * G - TM>(bo, wave_first, buf + kStageOperand);
      lb.template issue<2 * G - TM + 1>(bo, wave_first, buf + kStageOperand);
    }
  };
  vu4 af[2][TM], bf[2][TN];
  const uint32_t lds_base = lds_byte_address(lds);
  auto read_group = [&](auto fbuf, uint32_t st, auto kk, auto group) {  // the fragments group g is in charge of
    constexpr int FB = decltype(fbuf)::value, KK = decltype(kk)::value, G = decltype(group)::value;
    const uint32_t buf = lds_base + (st & 3u) * (kStageBuf * 2u);
    af[FB][G] = fa.template read<G, KK>(buf);
    bf[FB][BPG * G] = fb.template read<BPG * G, KK>(buf + kStageOperand * 2u);
    if constexpr (BPG == 2) bf[FB][2 * G + 1] = fb.template read<2 * G + 1, KK>(buf + kStageOperand * 2u);
  };
  // every read issued so far has returned; the fragments of buffer fbuf may be used from here on
  auto reads_done = [&](int fbuf) {
    if constexpr (TM == 4) {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(af[fbuf][0]), "+v"(af[fbuf][1]), "+v"(af[fbuf][2]), "+v"(af[fbuf][3]), "+v"(bf[fbuf][0]), "+v"(bf[fbuf][1]),
                     "+v"(bf[fbuf][2]), "+v"(bf[fbuf][3]));
    } else {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(af[fbuf][0]), "+v"(af[fbuf][1]), "+v"(bf[fbuf][0]), "+v"(bf[fbuf][1]), "+v"(bf[fbuf][2]), "+v"(bf[fbuf][3]));
    }
  };
  auto mfma_row = [&](int fbuf, int i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = mfma<IS_BF16>(af[fbuf][i], bf[fbuf][j], acc[i][j]);
  };
  // Waits until at most `stages` stages of this wave's loads are outstanding and all its local-memory reads have
  // returned, then meets the other waves. One piece of assembly on purpose: behind __syncthreads() the compiler
  // waits for every outstanding load (the direct loads write local memory), which would drain the ring.
  auto meet = [](auto stages) {
    constexpr int N = decltype(stages)::value * 2 * NL;
    static_assert(N == 0 || N == 4 || N == 8 || N == 16, "vmcnt values spelled out below");
    if constexpr (N == 16) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else if constexpr (N == 8) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else if constexpr (N == 4) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };
  auto for_groups = [&](auto f) {
    f(I0{});
    f(I1{});
    if constexpr (TM == 4) {
      f(std::integral_constant<int, 2>{});
      f(std::integral_constant<int, 3>{});
    }
  };

  for_groups([&](auto g) { issue_pair(0, g); });
  for_groups([&](auto g) { issue_pair(1, g); });
  if (nks > 2) {
    for_groups([&](auto g) { issue_pair(2, g); });
    meet(std::integral_constant<int, 2>{});
  } else {
    meet(I1{});
  }
  for_groups([&](auto g) { read_group(I0{}, 0, I0{}, g); });

  // One stage = two steps of 16 k, each TM groups of four MFMAs (one row of accumulator tiles). Group g of
  // step 0 also reads its fragments of step 1 and sends two of the loads of stage st+3; step 1 first meets the
  // other waves (stage st+1 has landed for everybody, and nobody reads stage st any more, whose buffer the
  // loads issued after the next meeting overwrite), then its group g reads its fragments of stage st+1. The
  // scheduler may not move anything across a group.
  auto stage = [&](uint32_t st, auto loads, auto next) {
    constexpr bool LOADS = decltype(loads)::value, NEXT = decltype(next)::value;
    __builtin_amdgcn_sched_barrier(0);
    reads_done(0);
    __builtin_amdgcn_sched_barrier(0);
    for_groups([&](auto g) {
      read_group(I1{}, st, I1{}, g);
      if constexpr (LOADS) issue_pair(st + 3, g);
      mfma_row(0, decltype(g)::value);
      __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (NEXT) {
      if constexpr (LOADS) meet(std::integral_constant<int, 2>{});  // younger: the loads of stages st+2 and st+3
      else meet(I0{});
    }
    reads_done(1);
    __builtin_amdgcn_sched_barrier(0);
    for_groups([&](auto g) {
      if constexpr (NEXT) read_group(I0{}, st + 1, I0{}, g);
      mfma_row(1, decltype(g)::value);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  uint32_t st = 0;
  for (; st + 3 < nks; ++st) stage(st, std::true_type{}, std::true_type{});
  for (; st + 1 < nks; ++st) stage(st, std::false_type{}, std::true_type{});
  stage(st, std::false_type{}, std::false_type{});
  __syncthreads();
}

// ---- epilogue ---------------------------------------------------------------------------------------
// A slab is 8 consecutive columns of one row of the output; the interpreter works on SL slabs at a
// time (4 when a lane has that many per pass, else 2), held as one vector of fp32 containers
// (element s*8 + e = column e of slab s): with one wave per SIMD the independent elements are what
// hides the VALU latency.
typedef float vf32 __attribute__((ext_vector_type(32)));
template <int SL> struct SlabVec;
template <> struct SlabVec<2> { typedef vf16 type; };
template <> struct SlabVec<4> { typedef vf32 type; };

#define FOR_SE _Pragma("unroll") for (int q = 0; q < SL * 8; ++q)

struct SlabRows {
  uint32_t row[4];  // output row of each slab
  uint32_t ok;      // bit s: slab s is inside the output
};

typedef float vf8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ bool wave_all(bool c) { return __builtin_amdgcn_ballot_w64(!c) == 0; }

__device__ __forceinline__ float cvt_in(uint32_t dtype, uint32_t bits16) {
  return dtype == VDT_F16 ? static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16))) : __uint_as_float(bits16 << 16);
}

__device__ __forceinline__ uint32_t elem_size(uint32_t dtype) {
  return (dtype == VDT_F32 || dtype == VDT_I32) ? 4u : (dtype == VDT_BOOL ? 1u : 2u);
}

// One slab, element by element, with every guard: edges, strided or unaligned operands.
__device__ __attribute__((noinline)) vf8 slab_load_slow(uint64_t addr, uint32_t dtype, uint32_t sn, uint64_t off, uint32_t ncol, uint32_t ok) {
  vf8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float v = 0.0f;
    if (ok != 0 && static_cast<uint32_t>(e) < ncol) {
      const uint64_t o = off + static_cast<uint64_t>(e) * sn;
      switch (dtype) {
        case VDT_F32: v = reinterpret_cast<const DVM_GLOBAL float *>(addr)[o]; break;
        case VDT_I32: v = __int_as_float(reinterpret_cast<const DVM_GLOBAL int32_t *>(addr)[o]); break;
        case VDT_F16:
        case VDT_BF16: v = cvt_in(dtype, reinterpret_cast<const DVM_GLOBAL uint16_t *>(addr)[o]); break;
        default: v = reinterpret_cast<const DVM_GLOBAL uint8_t *>(addr)[o] != 0 ? 1.0f : 0.0f; break;
      }
    }
    out[e] = v;
  }
  return out;
}

__device__ __attribute__((noinline)) void slab_store_slow(uint64_t addr, uint32_t dtype, uint32_t sn, uint64_t off, uint32_t ncol, uint32_t ok, vf8 x) {
  if (ok == 0) return;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if (static_cast<uint32_t>(e) >= ncol) continue;
    const uint64_t o = off + static_cast<uint64_t>(e) * sn;
    const float v = x[e];
    switch (dtype) {
      case VDT_F32: reinterpret_cast<DVM_GLOBAL float *>(addr)[o] = v; break;
      case VDT_I32: reinterpret_cast<DVM_GLOBAL int32_t *>(addr)[o] = __float_as_int(v); break;
      case VDT_F16: reinterpret_cast<DVM_GLOBAL _Float16 *>(addr)[o] = static_cast<_Float16>(v); break;
      case VDT_BF16: reinterpret_cast<DVM_GLOBAL uint16_t *>(addr)[o] = static_cast<uint16_t>(f32_to_bf16_bits(v)); break;
      default: reinterpret_cast<DVM_GLOBAL uint8_t *>(addr)[o] = v != 0.0f ? 1 : 0; break;
    }
  }
}

// Memory operand of the epilogue for SL slabs. col: first column of the slabs, ncol: columns inside
// the output (0..8). The whole wave takes one of three routes (the decision is a wave vote, so the
// common routes carry no per-lane control flow): 128-bit accesses when every lane's slabs are full,
// contiguous and 16-byte aligned; one element per slab when the operand does not vary along a row
// (a column of biases, a scalar); the guarded element loop otherwise.
template <int SL>
__device__ __forceinline__ typename SlabVec<SL>::type epi_load(uint64_t addr, uint32_t dtype, uint32_t sn, uint32_t sm, uint64_t boff,
                                                                const SlabRows &rows, uint32_t col, uint32_t ncol) {
  typename SlabVec<SL>::type out;
  const uint32_t esz = elem_size(dtype);
  const uint32_t full = (1u << SL) - 1u;
  const uint64_t col_off = boff + static_cast<uint64_t>(col) * sn;
  const bool wide = sn == 1 && esz != 1 && ((static_cast<uint64_t>(sm) * esz) & 15u) == 0 &&
                    wave_all(rows.ok == full && ncol == 8 && ((addr + col_off * esz) & 15u) == 0);
  if (wide) {
    // an operand that does not vary with the row (a bias row) is fetched once
    const int distinct = sm == 0 ? 1 : SL;
    if (esz == 4) {
#pragma unroll
      for (int s = 0; s < SL; ++s) {
        if (s < distinct) {
          const uint64_t o = (col_off + static_cast<uint64_t>(rows.row[s]) * sm) * 4;
          const vu4 a = *reinterpret_cast<const DVM_GLOBAL vu4 *>(addr + o), b = *reinterpret_cast<const DVM_GLOBAL vu4 *>(addr + o + 16);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            out[s * 8 + e] = __uint_as_float(a[e]);
            out[s * 8 + 4 + e] = __uint_as_float(b[e]);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) out[s * 8 + e] = out[e];
        }
      }
    } else {
      const bool f16 = dtype == VDT_F16;
#pragma unroll
      for (int s = 0; s < SL; ++s) {
        if (s < distinct) {
          const vu4 a = *reinterpret_cast<const DVM_GLOBAL vu4 *>(addr + (col_off + static_cast<uint64_t>(rows.row[s]) * sm) * 2);
          if (f16) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              out[s * 8 + e] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>((a[e >> 1] >> (16 * (e & 1))) & 0xffffu)));
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) out[s * 8 + e] = __uint_as_float((e & 1) ? (a[e >> 1] & 0xffff0000u) : (a[e >> 1] << 16));
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) out[s * 8 + e] = out[e];
        }
      }
    }
    return out;
  }
  if (sn == 0 && wave_all(rows.ok == full)) {
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const uint64_t o = col_off + static_cast<uint64_t>(rows.row[s]) * sm;
      float v;
      switch (dtype) {
        case VDT_F32: v = reinterpret_cast<const DVM_GLOBAL float *>(addr)[o]; break;
        case VDT_I32: v = __int_as_float(reinterpret_cast<const DVM_GLOBAL int32_t *>(addr)[o]); break;
        case VDT_F16:
        case VDT_BF16: v = cvt_in(dtype, reinterpret_cast<const DVM_GLOBAL uint16_t *>(addr)[o]); break;
        default: v = reinterpret_cast<const DVM_GLOBAL uint8_t *>(addr)[o] != 0 ? 1.0f : 0.0f; break;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) out[s * 8 + e] = v;
    }
    return out;
  }
#pragma unroll
  for (int s = 0; s < SL; ++s) {
    const vf8 v = slab_load_slow(addr, dtype, sn, col_off + static_cast<uint64_t>(rows.row[s]) * sm, ncol, (rows.ok >> s) & 1u);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[s * 8 + e] = v[e];
  }
  return out;
}

template <int SL>
__device__ __forceinline__ void epi_store(uint64_t addr, uint32_t dtype, uint32_t sn, uint32_t sm, uint64_t boff, const SlabRows &rows,
                                          uint32_t col, uint32_t ncol, const typename SlabVec<SL>::type &x) {
  const uint32_t esz = elem_size(dtype);
  const uint32_t full = (1u << SL) - 1u;
  const uint64_t col_off = boff + static_cast<uint64_t>(col) * sn;
  const bool wide = sn == 1 && esz != 1 && ((static_cast<uint64_t>(sm) * esz) & 15u) == 0 &&
                    wave_all(rows.ok == full && ncol == 8 && ((addr + col_off * esz) & 15u) == 0);
  if (wide) {
    if (esz == 4) {
#pragma unroll
      for (int s = 0; s < SL; ++s) {
        const uint64_t o = (col_off + static_cast<uint64_t>(rows.row[s]) * sm) * 4;
        vu4 a, b;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = __float_as_uint(x[s * 8 + e]);
          b[e] = __float_as_uint(x[s * 8 + 4 + e]);
        }
        *reinterpret_cast<DVM_GLOBAL vu4 *>(addr + o) = a;
        *reinterpret_cast<DVM_GLOBAL vu4 *>(addr + o + 16) = b;
      }
    } else if (dtype == VDT_F16) {
#pragma unroll
      for (int s = 0; s < SL; ++s) {
        vu4 a;
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = pack_f16(x[s * 8 + 2 * e], x[s * 8 + 2 * e + 1]);
        *reinterpret_cast<DVM_GLOBAL vu4 *>(addr + (col_off + static_cast<uint64_t>(rows.row[s]) * sm) * 2) = a;
      }
    } else {
#pragma unroll
      for (int s = 0; s < SL; ++s) {
        vu4 a;
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = pack_bf16(x[s * 8 + 2 * e], x[s * 8 + 2 * e + 1]);
        *reinterpret_cast<DVM_GLOBAL vu4 *>(addr + (col_off + static_cast<uint64_t>(rows.row[s]) * sm) * 2) = a;
      }
    }
    return;
  }
#pragma unroll
  for (int s = 0; s < SL; ++s) {
    vf8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = x[s * 8 + e];
    slab_store_slow(addr, dtype, sn, col_off + static_cast<uint64_t>(rows.row[s]) * sm, ncol, (rows.ok >> s) & 1u, v);
  }
}

// out-of-line math on 16 values at a time (arguments and results travel in registers)
__device__ __attribute__((noinline)) vf16 math_exp(vf16 x) {
#pragma unroll
  for (int q = 0; q < 16; ++q) x[q] = expf(x[q]);
  return x;
}
__device__ __attribute__((noinline)) vf16 math_log(vf16 x) {
#pragma unroll
  for (int q = 0; q < 16; ++q) x[q] = logf(x[q]);
  return x;
}
__device__ __attribute__((noinline)) vf16 math_pow(vf16 x, vf16 y) {
#pragma unroll
  for (int q = 0; q < 16; ++q) x[q] = powf(x[q], y[q]);
  return x;
}
__device__ __attribute__((noinline)) vf16 math_sqrt(vf16 x) {
#pragma unroll
  for (int q = 0; q < 16; ++q) x[q] = sqrtf(x[q]);
  return x;
}
template <int SL, typename V, typename F>
__device__ __forceinline__ V by_halves(V x, F f) {
  if constexpr (SL == 2) {
    return f(x);
  } else {
    vf16 lo, hi;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      lo[q] = x[q];
      hi[q] = x[16 + q];
    }
    lo = f(lo);
    hi = f(hi);
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      x[q] = lo[q];
      x[16 + q] = hi[q];
    }
    return x;
  }
}
template <int SL, typename V>
__device__ __forceinline__ V slab_pow(V x, V y) {
  if constexpr (SL == 2) {
    return math_pow(x, y);
  } else {
    vf16 xl, xh, yl, yh;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      xl[q] = x[q];
      xh[q] = x[16 + q];
      yl[q] = y[q];
      yh[q] = y[16 + q];
    }
    xl = math_pow(xl, yl);
    xh = math_pow(xh, yh);
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      x[q] = xl[q];
      x[16 + q] = xh[q];
    }
    return x;
  }
}

template <int SL, typename Slabs>
__device__ __forceinline__ void apply_rnd(Slabs &a, uint32_t rnd) {
  if (rnd == VRND_F16) {
    FOR_SE a[q] = round_f16(a[q]);
  } else if (rnd == VRND_BF16) {
    FOR_SE a[q] = round_bf16(a[q]);
  }
}

struct EpiArgs {
  uint32_t mem_off, code_off, batch0, batch1;
  uint32_t flags;   // VCubeHeader::epi_flags
  uint32_t w0v, immv;  // per lane: the two words of instruction `lane` of the epilogue program (the first 64)
  uint32_t first;      // the instruction the epilogue starts at (VCF_DUMP16: the kernel has done the ones before it)
};

// What the epilogue reads the tile back from: fp32 accumulators (D16 = 0), or values already rounded to the operand
// type and kept as their 16 bits (1: bf16, 2: fp16). One slab = 8 columns of local row `lr`.
template <int D16, int BN>
__device__ __forceinline__ void dump_read_slab(const void *dump, uint32_t lr, uint32_t g, vf4 &lo, vf4 &hi) {
  if constexpr (D16 == 0) {
    const float *src = reinterpret_cast<const float *>(dump) + lr * (BN + 4) + g * 8;
    lo = *reinterpret_cast<const vf4 *>(src);
    hi = *reinterpret_cast<const vf4 *>(src + 4);
  } else {
    const vu4 a = *reinterpret_cast<const vu4 *>(reinterpret_cast<const uint16_t *>(dump) + lr * (BN + 8) + g * 8);
    if constexpr (D16 == 1) {
      lo = vf4{__uint_as_float(a[0] << 16), __uint_as_float(a[0] & 0xffff0000u), __uint_as_float(a[1] << 16), __uint_as_float(a[1] & 0xffff0000u)};
      hi = vf4{__uint_as_float(a[2] << 16), __uint_as_float(a[2] & 0xffff0000u), __uint_as_float(a[3] << 16), __uint_as_float(a[3] & 0xffff0000u)};
    } else {
      auto h2f = [](uint32_t bits) { return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits & 0xffffu))); };
      lo = vf4{h2f(a[0]), h2f(a[0] >> 16), h2f(a[1]), h2f(a[1] >> 16)};
      hi = vf4{h2f(a[2]), h2f(a[2] >> 16), h2f(a[3]), h2f(a[3] >> 16)};
    }
  }
}

// Runs the epilogue program on SL slabs whose accumulator values are in `acc`.
// SLIM: the program holds only what VCF_SLIM lists (one temporary, float binaries, the hardware's exp / log / sqrt,
// rounding, loads and stores): the arms of everything else are left out, and with them most of the registers.
template <int SL, bool SLIM>
__device__ __forceinline__ void run_epilogue(typename SlabVec<SL>::type acc, const uint32_t *prog32, const EpiArgs &h, const SlabRows &rows,
                                             uint32_t col, uint32_t ncol) {
  typedef typename SlabVec<SL>::type Slabs;
  const uint32_t *code32 = prog32 + 2 * h.code_off;
  static_assert(NTEMP == 4, "temporaries are named registers");
  auto mem_desc = [&](uint32_t a, uint64_t &addr, uint32_t &dtype, uint32_t &sn, uint32_t &sm, uint64_t &boff) {
    const uint32_t *d = prog32 + 2 * h.mem_off + a * (sizeof(VCubeMem) / 4);
    addr = static_cast<uint64_t>(uni(d[0])) | (static_cast<uint64_t>(uni(d[1])) << 32);
    dtype = uni(d[2]);
    sn = uni(d[4]);
    sm = uni(d[5]);
    boff = static_cast<uint64_t>(h.batch0) * uni(d[6]) + static_cast<uint64_t>(h.batch1) * uni(d[7]);
  };
  if (h.flags & VCF_PLAIN_STORE) {
    // [Add mem] [cast.round] store: three instructions at most, done here without the dispatch loop
    uint32_t at = h.first;
    uint32_t w0 = __builtin_amdgcn_readlane(h.w0v, at);
    uint64_t addr, boff;
    uint32_t dtype, sn, sm;
    if ((w0 & 0xffu) == VOP_BINF) {
      mem_desc(w0 >> 24, addr, dtype, sn, sm, boff);
      acc = acc + epi_load<SL>(addr, dtype, sn, sm, boff, rows, col, ncol);
      w0 = __builtin_amdgcn_readlane(h.w0v, ++at);
    }
    if ((w0 & 0xffu) == VOP_CAST) {
      apply_rnd<SL>(acc, (w0 >> 20) & 0x3u);
      w0 = __builtin_amdgcn_readlane(h.w0v, ++at);
    }
    mem_desc(w0 >> 24, addr, dtype, sn, sm, boff);
    epi_store<SL>(addr, dtype, sn, sm, boff, rows, col, ncol, acc);
    return;
  }
  Slabs t0, t1, t2, t3;  // never read before written (the emitter parks a value before it names the register)
  uint32_t mask = 0;
  (void)t1;
  (void)t2;
  (void)t3;
  (void)mask;
  uint32_t pc = h.first;
  while (true) {
    // the program sits in two registers, one instruction per lane: no memory access to fetch one
    uint32_t w0, imm;
    if (pc < 64u) {
      w0 = __builtin_amdgcn_readlane(h.w0v, pc);
      imm = __builtin_amdgcn_readlane(h.immv, pc);
    } else {
      w0 = uni(code32[2 * pc]);
      imm = uni(code32[2 * pc + 1]);
    }
    ++pc;
    const uint32_t op = w0 & 0xffu;
    if (op == VOP_END) break;
    const uint32_t sub = (w0 >> 8) & 0xffu, a = w0 >> 24, rnd = (w0 >> 20) & 0x3u;
    if (op >= VOP_SRC_BASE || op == VOP_ST) {
      const uint32_t kind = op == VOP_ST ? static_cast<uint32_t>(VK_MEM) : ((w0 >> 16) & 0xfu);
      Slabs src;
      if (kind == VK_MEM) {
        const uint32_t *d = prog32 + 2 * h.mem_off + a * (sizeof(VCubeMem) / 4);
        const uint64_t addr = static_cast<uint64_t>(uni(d[0])) | (static_cast<uint64_t>(uni(d[1])) << 32);
        const uint32_t dtype = uni(d[2]), sn = uni(d[4]), sm = uni(d[5]), sb0 = uni(d[6]), sb1 = uni(d[7]);
        const uint64_t boff = static_cast<uint64_t>(h.batch0) * sb0 + static_cast<uint64_t>(h.batch1) * sb1;
        if (op == VOP_ST) {
          epi_store<SL>(addr, dtype, sn, sm, boff, rows, col, ncol, acc);
          continue;
        }
        src = epi_load<SL>(addr, dtype, sn, sm, boff, rows, col, ncol);
      } else if (kind == VK_IMM) {
        src = __uint_as_float(imm);
      } else if (kind == VK_REG) {
        if constexpr (SLIM) src = t0;
        else src = a == 0 ? t0 : (a == 1 ? t1 : (a == 2 ? t2 : t3));
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
            // (v_rcp_f32 and a multiply; the library's __fdividef is the full IEEE division, ten instructions)
            case VB_DIV_APPROX: FOR_SE acc[q] = acc[q] * __builtin_amdgcn_rcpf(src[q]); break;
            case VB_RDIV_APPROX: FOR_SE acc[q] = src[q] * __builtin_amdgcn_rcpf(acc[q]); break;
            case VB_MIN: FOR_SE acc[q] = acc[q] < src[q] ? acc[q] : src[q]; break;
            case VB_MAX: FOR_SE acc[q] = acc[q] > src[q] ? acc[q] : src[q]; break;
            case VB_AND: if constexpr (!SLIM) FOR_SE acc[q] = (acc[q] != 0.0f && src[q] != 0.0f) ? 1.0f : 0.0f; break;
            case VB_OR: if constexpr (!SLIM) FOR_SE acc[q] = (acc[q] != 0.0f || src[q] != 0.0f) ? 1.0f : 0.0f; break;
            case VB_POW: if constexpr (!SLIM) acc = slab_pow<SL>(acc, src); break;
            default: if constexpr (!SLIM) acc = slab_pow<SL>(src, acc); break;
          }
          apply_rnd<SL>(acc, rnd);
          break;
        case VOP_BINI:
          if constexpr (!SLIM) switch (sub & 0x3fu) {
            case VBI_ADD: FOR_SE acc[q] = __uint_as_float(__float_as_uint(acc[q]) + __float_as_uint(src[q])); break;
            case VBI_SUB: FOR_SE acc[q] = __uint_as_float(__float_as_uint(acc[q]) - __float_as_uint(src[q])); break;
            case VBI_RSUB: FOR_SE acc[q] = __uint_as_float(__float_as_uint(src[q]) - __float_as_uint(acc[q])); break;
            case VBI_MUL: FOR_SE acc[q] = __uint_as_float(__float_as_uint(acc[q]) * __float_as_uint(src[q])); break;
            case VBI_MIN: FOR_SE acc[q] = __int_as_float(min(__float_as_int(acc[q]), __float_as_int(src[q]))); break;
            default: FOR_SE acc[q] = __int_as_float(max(__float_as_int(acc[q]), __float_as_int(src[q]))); break;
          }
          break;
        case VOP_CMP: if constexpr (!SLIM) {
          const uint32_t t = sub & 0x7u;
          if (sub & VCMP_INT) {
            FOR_SE {
              const int32_t x = __float_as_int(acc[q]), y = __float_as_int(src[q]);
              const bool c = t == VCMP_EQ ? x == y : t == VCMP_NE ? x != y : t == VCMP_GT ? x > y : t == VCMP_GE ? x >= y : t == VCMP_LT ? x < y : x <= y;
              acc[q] = __int_as_float(c ? 1 : 0);
            }
          } else {
            FOR_SE {
              const float x = acc[q], y = src[q];
              const bool c = t == VCMP_EQ ? x == y : t == VCMP_NE ? x != y : t == VCMP_GT ? x > y : t == VCMP_GE ? x >= y : t == VCMP_LT ? x < y : x <= y;
              acc[q] = c ? 1.0f : 0.0f;
            }
          }
        }
          break;
        case VOP_MSK:
          if constexpr (!SLIM) {
            mask = 0;
            FOR_SE mask |= ((__float_as_uint(src[q]) << 1) != 0 ? 1u : 0u) << q;
          }
          break;
        default:  // VOP_MOVM
          if constexpr (!SLIM) FOR_SE acc[q] = ((mask >> q) & 1u) ? src[q] : acc[q];
          break;
      }
      continue;
    }
    switch (op) {
      case VOP_LDR:
        if constexpr (SLIM) acc = t0;
        else acc = a == 0 ? t0 : (a == 1 ? t1 : (a == 2 ? t2 : t3));
        break;
      case VOP_LDI:
        acc = __uint_as_float(imm);
        break;
      case VOP_STR:
        if (SLIM || a == 0) t0 = acc;
        else if (a == 1) t1 = acc;
        else if (a == 2) t2 = acc;
        else t3 = acc;
        break;
      case VOP_UN:
        switch (sub) {
          case VU_SQRT: if constexpr (!SLIM) acc = by_halves<SL>(acc, math_sqrt); break;
          case VU_SQRT_APPROX: FOR_SE acc[q] = __builtin_amdgcn_sqrtf(acc[q]); break;
          case VU_ABS: FOR_SE acc[q] = fabsf(acc[q]); break;
          case VU_LOG: if constexpr (!SLIM) acc = by_halves<SL>(acc, math_log); break;
          case VU_LOG_APPROX: FOR_SE acc[q] = __builtin_amdgcn_logf(acc[q]) * 0.6931471805599453f; break;  // (v_log_f32 is log2; the library's __logf is the exact one)
          case VU_EXP: if constexpr (!SLIM) acc = by_halves<SL>(acc, math_exp); break;
          case VU_EXP_SCALED:  // the product is a value of its own: rounded to fp32, never contracted into what follows
            if constexpr (!SLIM) {
              FOR_SE {
                float y = acc[q] * __uint_as_float(imm);
                asm volatile("" : "+v"(y));
                acc[q] = y;
              }
              acc = by_halves<SL>(acc, math_exp);
            }
            break;
          case VU_EXP_APPROX: FOR_SE acc[q] = __expf(acc[q]); break;
          case VU_EXP_SCALED_APPROX:
            FOR_SE {
              float y = acc[q] * __uint_as_float(imm);
              asm volatile("" : "+v"(y));
              acc[q] = __expf(y);
            }
            break;
          case VU_SILU_APPROX:
          case VU_SIGMOID_APPROX:
            FOR_SE {
              float y = acc[q] * __uint_as_float(imm);
              asm volatile("" : "+v"(y));  // (the product is a value of its own, as in the separate instructions)
              float d = __expf(y) + 1.0f;
              asm volatile("" : "+v"(d));
              const float r = __builtin_amdgcn_rcpf(d);
              acc[q] = sub == VU_SILU_APPROX ? acc[q] * r : r;
            }
            break;
          case VU_ISFINITE: if constexpr (!SLIM) FOR_SE acc[q] = isfinite(acc[q]) ? 1.0f : 0.0f; break;
          case VU_ROUND: if constexpr (!SLIM) FOR_SE acc[q] = rintf(acc[q]); break;
          case VU_FLOOR: if constexpr (!SLIM) FOR_SE acc[q] = floorf(acc[q]); break;
          case VU_CEIL: if constexpr (!SLIM) FOR_SE acc[q] = ceilf(acc[q]); break;
          case VU_TRUNC: if constexpr (!SLIM) FOR_SE acc[q] = truncf(acc[q]); break;
          default:
            if constexpr (!SLIM) FOR_SE {
              const uint32_t x = __float_as_uint(acc[q]);
              acc[q] = __uint_as_float(static_cast<int32_t>(x) < 0 ? 0u - x : x);
            }
            break;
        }
        apply_rnd<SL>(acc, rnd);
        break;
      case VOP_CAST:
        if (SLIM) {
          apply_rnd<SL>(acc, rnd);
        } else if (sub == VC_F2I) {
          FOR_SE acc[q] = __int_as_float(static_cast<int32_t>(acc[q]));
        } else if (sub == VC_I2F) {
          FOR_SE acc[q] = static_cast<float>(__float_as_int(acc[q]));
          apply_rnd<SL>(acc, rnd);
        } else if (sub == VC_RND) {
          apply_rnd<SL>(acc, rnd);
        } else {
          FOR_SE acc[q] = acc[q] != 0.0f ? 1.0f : 0.0f;
        }
        break;
      default:
        break;
    }
  }
}

// The epilogue of a plain product, [Add mem] [cast.round] store (VCF_PLAIN_STORE), for one wave's slabs of a pass: when
// they all lie inside the output and the operands take 128-bit accesses, every slab is read, finished and stored here
// (the descriptors are decoded once, the bias row is fetched once: a lane's column does not change) and the function
// returns true; otherwise the caller sends the slabs through epilogue_pass, which does the same with every guard.
// A function of its own, and a small one: what a call costs is the registers the callee has to save (the interpreter's
// pass saves and restores some hundred per lane through scratch memory, 12 us per tile and launch on MI355X).
template <int ROWS, int BN, int TM, int WM, int D16>
__device__ __attribute__((noinline)) bool epilogue_plain_pass(const void *dump, const uint32_t *prog32, EpiArgs ea, uint32_t m0, uint32_t n0,
                                                              uint32_t pass, uint32_t m, uint32_t n, uint32_t m_lo, uint32_t n_lo) {
  constexpr int NTHR = WM * 2 * 64;
  constexpr int GROUPS = BN / 8;
  constexpr int PER_THREAD = ROWS * GROUPS / NTHR;
  constexpr int ROWS_PER_STEP = NTHR / GROUPS;
  constexpr int HALF = ROWS / WM;
  const uint32_t tid = threadIdx.x;
  const uint32_t g = tid % GROUPS, r0 = tid / GROUPS;
  const uint32_t col = n0 + g * 8;
  const uint32_t ncol = (col >= n || col < n_lo) ? 0u : (n - col < 8u ? n - col : 8u);
  // [Add mem] [cast.round] store, the epilogue of a plain product: when the wave's slabs are all inside the output and
  // the operands take 128-bit accesses, every slab of the pass is read, finished and stored here in one go (the
  // descriptors are decoded once, the bias row is fetched once: a lane's column does not change); otherwise the
  // slabs go through run_epilogue below, which does the same three instructions with every guard.
  const uint32_t *code32 = prog32 + 2 * ea.code_off;
  auto desc = [&](uint32_t a, uint64_t &addr, uint32_t &dtype, uint32_t &sn, uint32_t &sm, uint64_t &boff) {
    const uint32_t *d = prog32 + 2 * ea.mem_off + a * (sizeof(VCubeMem) / 4);
    addr = static_cast<uint64_t>(uni(d[0])) | (static_cast<uint64_t>(uni(d[1])) << 32);
    dtype = uni(d[2]);
    sn = uni(d[4]);
    sm = uni(d[5]);
    boff = static_cast<uint64_t>(ea.batch0) * uni(d[6]) + static_cast<uint64_t>(ea.batch1) * uni(d[7]);
  };
  uint32_t at = ea.first, w0 = uni(code32[2 * at]);
  bool has_bias = false;
  uint64_t b_addr = 0, b_boff = 0, s_addr, s_boff;
  uint32_t b_dtype = 0, b_sn = 0, b_sm = 0, s_dtype, s_sn, s_sm, rnd = VRND_NONE;
  if ((w0 & 0xffu) == VOP_BINF) {
    has_bias = true;
    desc(w0 >> 24, b_addr, b_dtype, b_sn, b_sm, b_boff);
    w0 = uni(code32[2 * ++at]);
  }
  if ((w0 & 0xffu) == VOP_CAST) {
    rnd = (w0 >> 20) & 0x3u;
    w0 = uni(code32[2 * ++at]);
  }
  desc(w0 >> 24, s_addr, s_dtype, s_sn, s_sm, s_boff);
  const uint32_t s_esz = elem_size(s_dtype);
  bool fast = ncol == 8u && s_sn == 1u && s_esz != 1u && ((static_cast<uint64_t>(s_sm) * s_esz) & 15u) == 0u &&
              ((s_addr + (s_boff + col) * s_esz) & 15u) == 0u;
  if (has_bias) {  // a row of fp32 biases (the same for every row of the output), 128-bit loads
    fast = fast && b_dtype == VDT_F32 && b_sn == 1u && b_sm == 0u && ((b_addr + (b_boff + col) * 4u) & 15u) == 0u;
  }
  auto row_of = [&](int q) -> uint32_t {
    const uint32_t lr = q * ROWS_PER_STEP + r0;
    return m0 + (lr / HALF) * (TM * 32) + pass * HALF + lr % HALF;
  };
  {  // the lane's rows grow with q: the first and the last bound them all
    const uint32_t first = row_of(0), last = row_of(PER_THREAD - 1);
    fast = fast && first >= m_lo && last < m && first <= last;
  }
  if (wave_all(fast)) {
    vf4 blo = {0.0f, 0.0f, 0.0f, 0.0f}, bhi = blo;
    if (has_bias) {
      const DVM_GLOBAL vf4 *bp = reinterpret_cast<const DVM_GLOBAL vf4 *>(b_addr + (b_boff + col) * 4u);
      blo = bp[0];
      bhi = bp[1];
    }
    constexpr int CH = PER_THREAD < 4 ? PER_THREAD : 4;  // slabs in flight: few, so that the function stays small in registers
#pragma unroll
    for (int c0 = 0; c0 < PER_THREAD; c0 += CH) {
      vf4 lo[CH], hi[CH];
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        dump_read_slab<D16, BN>(dump, (c0 + q) * ROWS_PER_STEP + r0, g, lo[q], hi[q]);
      }
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        vf4 x = lo[q] + blo, y = hi[q] + bhi;
        if (rnd == VRND_F16) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            x[e] = round_f16(x[e]);
            y[e] = round_f16(y[e]);
          }
        } else if (rnd == VRND_BF16) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            x[e] = round_bf16(x[e]);
            y[e] = round_bf16(y[e]);
          }
        }
        const uint64_t o = (s_boff + col + static_cast<uint64_t>(row_of(c0 + q)) * s_sm) * s_esz;
        if (s_esz == 4u) {
          vu4 a, b;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            a[e] = __float_as_uint(x[e]);
            b[e] = __float_as_uint(y[e]);
          }
          *reinterpret_cast<DVM_GLOBAL vu4 *>(s_addr + o) = a;
          *reinterpret_cast<DVM_GLOBAL vu4 *>(s_addr + o + 16) = b;
        } else if (s_dtype == VDT_F16) {
          const vu4 a = {pack_f16(x[0], x[1]), pack_f16(x[2], x[3]), pack_f16(y[0], y[1]), pack_f16(y[2], y[3])};
          *reinterpret_cast<DVM_GLOBAL vu4 *>(s_addr + o) = a;
        } else {
          const vu4 a = {pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(y[0], y[1]), pack_bf16(y[2], y[3])};
          *reinterpret_cast<DVM_GLOBAL vu4 *>(s_addr + o) = a;
        }
      }
    }
    return true;
  }
  return false;
}

// Second half of a pass: the half tile sits in local memory, row major with PITCH floats per row;
// every lane takes slabs of 8 columns and walks the epilogue program over them.
template <int ROWS, int BN, int TM, int WM, bool SLIM, int D16>
__device__ __forceinline__ void epilogue_pass_body(const void *dump, const uint32_t *prog32, EpiArgs ea, uint32_t m0, uint32_t n0,
                                                        uint32_t pass, uint32_t m, uint32_t n, uint32_t m_lo, uint32_t n_lo) {
  constexpr int NTHR = WM * 2 * 64;
  constexpr int GROUPS = BN / 8;               // slabs per row
  constexpr int PER_THREAD = ROWS * GROUPS / NTHR;  // slabs per thread
  // four slabs per walk of the program where a wave may use all 512 registers; with two waves per SIMD two slabs
  constexpr int SL = (PER_THREAD % 4 == 0 && (WM == 2 || SLIM)) ? 4 : 2;
  static_assert(PER_THREAD % SL == 0, "slab count per thread");
  constexpr int ROWS_PER_STEP = NTHR / GROUPS;  // rows one step of all threads covers
  const uint32_t tid = threadIdx.x;
  const uint32_t g = tid % GROUPS, r0 = tid / GROUPS;
  constexpr int HALF = ROWS / WM;  // local rows [i * HALF, (i + 1) * HALF) belong to the i-th row of waves
  const uint32_t col = n0 + g * 8;
  // (a tile moved back from the edge starts its columns a whole number of slabs before n_lo)
  const uint32_t ncol = (col >= n || col < n_lo) ? 0u : (n - col < 8u ? n - col : 8u);
  {
    const uint32_t *code32 = prog32 + 2 * ea.code_off;
    const uint32_t li = (tid & 63u) < ea.w0v ? (tid & 63u) : 0u;  // w0v arrives holding the instruction count
    ea.w0v = code32[2 * li];
    ea.immv = code32[2 * li + 1];
  }
  for (int it = 0; it < PER_THREAD / SL; ++it) {
    typename SlabVec<SL>::type acc;
    SlabRows rows;
    rows.ok = 0;
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const uint32_t lr = (it * SL + s) * ROWS_PER_STEP + r0;  // local row of the dump
      const uint32_t wm = lr / HALF, rr = lr % HALF;
      rows.row[s] = m0 + wm * (TM * 32) + pass * HALF + rr;
      rows.ok |= ((rows.row[s] < m && rows.row[s] >= m_lo) ? 1u : 0u) << s;
      vf4 lo, hi;
      dump_read_slab<D16, BN>(dump, lr, g, lo, hi);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[s * 8 + e] = lo[e];
        acc[s * 8 + 4 + e] = hi[e];
      }
    }
    if (wave_all(rows.ok == 0u || ncol == 0u)) continue;  // nothing of these slabs is inside the tile's part of the output
    run_epilogue<SL, SLIM>(acc, prog32, ea, rows, col, ncol);
  }
}

template <int ROWS, int BN, int TM, int WM, bool SLIM, int D16>
__device__ __attribute__((noinline)) void epilogue_pass(const void *dump, const uint32_t *prog32, EpiArgs ea, uint32_t m0, uint32_t n0,
                                                        uint32_t pass, uint32_t m, uint32_t n, uint32_t m_lo, uint32_t n_lo) {
  epilogue_pass_body<ROWS, BN, TM, WM, SLIM, D16>(dump, prog32, ea, m0, n0, pass, m, n, m_lo, n_lo);
}

// TM x TN 32x32 MFMA tiles per wave, 2 x 2 waves per workgroup; A_KC / B_KC: the operand's k axis is
// contiguous in memory.
// COMB: the build for the second launch of a product with a split k axis (it sums the partial tiles and runs the
// epilogue; no operand is read). A kernel of its own, so that the registers the sum holds in flight do not weigh on
// the allocation of the tile loop (in one kernel with it the 256-tile product without a split lost 5 %).
template <bool IS_BF16, int TM, int TN, bool A_KC, bool B_KC, int WM, bool COMB = false>
__device__ __forceinline__ void vm_cube(const VmParam &p) {
  constexpr int NTHR = WM * 2 * 64;  // WM x 2 waves
  constexpr int BM = WM * TM * 32, BN = 2 * TN * 32;
  constexpr int PASSES = TM >= 2 ? 2 : 1;
  constexpr int PROWS = BM / PASSES;  // rows of the tile one epilogue pass covers
  constexpr int PITCH = BN + 4;
  extern __shared__ double lds_raw[];
  __shared__ uint32_t prog32[DVM_PARAM_BYTES / 4];
  {
    // only the words the program occupies are read: the argument segment is far away
    const uint32_t *src = reinterpret_cast<const uint32_t *>(p.w);
    const VCubeHeader *hp = reinterpret_cast<const VCubeHeader *>(p.w);
    uint32_t used = (hp->code_off + hp->n_code) * 2;
    used = used < DVM_PARAM_BYTES / 4 ? used : DVM_PARAM_BYTES / 4;
    const uint32_t trips = (used + NTHR - 1) / NTHR;
    for (uint32_t t = 0; t < trips; ++t) {
      uint32_t i = t * NTHR + threadIdx.x;
      i = i < used ? i : used - 1;
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
  float *dump = reinterpret_cast<float *>(lds_raw);
  // A grouped product (VCG_*): the upper bounds of the groups' ranges, read once from the list in memory (its sizes
  // summed up, every value clipped into the axis the groups split), behind the tile buffers in local memory. Groups of
  // rows get a second table behind the first: how many rows of tiles the groups up to and including g touch (a tile a
  // bound runs through counts for both sides), so that the work items are exactly the tiles that have rows to store.
  uint32_t *gtab = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(lds_raw) + DVM_CUBE_LDS_BYTES(static_cast<uint32_t>(BM)));
  const uint32_t gmode = COMB ? static_cast<uint32_t>(VCG_NONE) : h.group_mode;
  const bool g_rows = gmode == VCG_M_BOUND || gmode == VCG_M_SIZE;
  uint32_t *gpre = gtab + h.nb1;
  if (gmode != VCG_NONE) {
    const bool sizes = gmode == VCG_M_SIZE || gmode == VCG_K_SIZE;
    const uint32_t limit = g_rows ? h.m : h.k, groups = h.nb1;
    auto entry = [&](uint32_t i) -> uint32_t {
      long long v = h.group_i32 ? static_cast<long long>(reinterpret_cast<const DVM_GLOBAL int32_t *>(h.group_addr)[i])
                                : reinterpret_cast<const DVM_GLOBAL long long *>(h.group_addr)[i];
      v = v < 0 ? 0 : v;
      return v > static_cast<long long>(limit) ? limit : static_cast<uint32_t>(v);
    };
    // the first wave sums values up, 64 at a time (an inclusive scan across its lanes, the total carried on), never past `cap`
    auto running_sum = [&](uint32_t *table, auto value, uint32_t cap) {
      if (threadIdx.x >= 64u) return;
      uint32_t carry = 0;
      for (uint32_t c0 = 0; c0 < groups; c0 += 64u) {
        const uint32_t i = c0 + threadIdx.x;
        uint32_t v = i < groups ? value(i) : 0u;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const uint32_t up = __shfl_up(v, d, 64);
          if (static_cast<int>(threadIdx.x) >= d) v = v + up < cap ? v + up : cap;  // (both at most cap, cap below 2^31)
        }
        v = v + carry < cap ? v + carry : cap;
        if (i < groups) table[i] = v;
        carry = __shfl(v, 63, 64);
      }
    };
    if (!sizes) {
      for (uint32_t i = threadIdx.x; i < groups; i += NTHR) gtab[i] = entry(i);
    } else {
      running_sum(gtab, entry, limit);
    }
    __syncthreads();
    if (g_rows) {
      running_sum(gpre, [&](uint32_t g) -> uint32_t {
        const uint32_t lo = g != 0u ? gtab[g - 1u] : 0u, hi = gtab[g];
        return hi > lo ? (hi + BM - 1u) / BM - lo / BM : 0u;
      }, 0x7fffffffu);
      __syncthreads();
    }
  }
  // [A buffer 0 | A buffer 1 | B buffer 0 | B buffer 1], offsets in elements
  constexpr uint32_t kABuf = BM * BK, kBBuf = BN * BK, kBBase = 2 * kABuf;

  const uint32_t tid = threadIdx.x;
  const uint32_t wave = tid >> 6, lane = tid & 63u;
  const uint32_t wm = wave >> 1, wn = wave & 1u;
  // (groups of rows: the rows of tiles the groups touch, one after the other, stand in for the tile rows of one matrix)
  const uint32_t tile_rows = g_rows ? uni(gpre[h.nb1 - 1u]) : h.tiles_m;
  const uint32_t tiles_per_batch = tile_rows * h.tiles_n;
  const uint32_t n_tiles = g_rows ? tiles_per_batch : tiles_per_batch * h.nb0 * h.nb1;
  // Split k (VCF_SPLITK_*): the first launch has k_split workgroups per tile, each walks k_chunk of the k axis and
  // leaves its fp32 accumulators in the partials buffer, register by register as the lanes hold them; the second
  // launch has one workgroup per tile, adds the partials in ascending k order and runs the epilogue.
  const bool split_part = !COMB && (h.epi_flags & VCF_SPLITK_PARTIAL) != 0u;
  const uint32_t n_work = split_part ? n_tiles * h.k_split : n_tiles;
  constexpr uint32_t kPartVecs = TM * TN * 4;  // 16-byte vectors a lane holds of the tile

  // Fragment reads: fragment i of this wave is rows r0 + 32*i of the staged tile (r0 = the lane's row
  // in fragment 0), and step kk wants chunk 2*kk + lane/32 of that row. With the swizzle of tile_off
  // the element offset is (r0 + 32*i) * 64 + ((x ^ c) ), x = ((lane/32) ^ swz(r0)) * 8 per lane and
  // c = (kk * 16) ^ ((i & 1) * 32) a constant: one XOR per read instead of one register per address.
  const uint32_t a_r0 = wm * TM * 32 + (lane & 31u), b_r0 = wn * TN * 32 + (lane & 31u);
  const uint32_t a_x = ((lane >> 5) ^ ((a_r0 ^ (a_r0 >> 3)) & 7u)) << 3, b_x = ((lane >> 5) ^ ((b_r0 ^ (b_r0 >> 3)) & 7u)) << 3;
  const uint32_t a_row = a_r0 * BK, b_row = kBBase + b_r0 * BK;
  auto frag_off = [](uint32_t row, uint32_t x, int f, int kk) -> uint32_t {
    return row + static_cast<uint32_t>(f) * 32u * BK + (x ^ static_cast<uint32_t>((kk << 4) ^ ((f & 1) << 5)));
  };

  for (uint32_t t0 = blockIdx.x; t0 < n_work; t0 += gridDim.x) {
    // Tile order. Workgroups are dealt to the 8 XCDs round robin, each XCD has its own L2: workgroup w
    // takes position (w % 8) * (n_tiles / 8) + w / 8, so an XCD works through one contiguous eighth of the
    // order; the order itself walks 8-tile-wide column bands row by row, which makes the 32 tiles an XCD has
    // in flight a 4 x 8 block (12 operand panels to fetch instead of 18 for two full rows of 16).
    uint32_t t = t0;
    if ((n_work & 7u) == 0 && gridDim.x >= n_work) t = (t0 & 7u) * (n_work >> 3) + (t0 >> 3);
    const uint32_t ksplit = t / n_tiles;  // which part of the k axis (0 unless the launch writes partials)
    t -= ksplit * n_tiles;
    const uint32_t tile_id = t;
    uint32_t k_lo = ksplit * h.k_chunk;
    uint32_t k_hi = split_part ? (k_lo + h.k_chunk < h.k ? k_lo + h.k_chunk : h.k) : h.k;
    const uint32_t batch = t / tiles_per_batch, tt = t % tiles_per_batch;
    uint32_t bi0 = batch / h.nb1, bi1 = batch % h.nb1;
    const uint32_t band = tt / (tile_rows * 8u), in_band = tt % (tile_rows * 8u);
    const uint32_t band_w = h.tiles_n - band * 8u < 8u ? h.tiles_n - band * 8u : 8u;
    uint32_t tm = in_band / band_w;
    const uint32_t tn = band * 8u + in_band % band_w;
    if (g_rows) {
      // which group the row of tiles belongs to (the first whose running count exceeds its number), and which of the
      // group's rows of tiles it is
      uint32_t lo = 0, hi = h.nb1 - 1u;
      while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (uni(gpre[mid]) > tm) hi = mid;
        else lo = mid + 1u;
      }
      bi0 = 0;
      bi1 = lo;
      const uint32_t first_row = lo != 0u ? uni(gtab[lo - 1u]) : 0u;
      tm = first_row / BM + (tm - (lo != 0u ? uni(gpre[lo - 1u]) : 0u));
    }
    // A ragged tile at the bottom or right edge is moved back inside the output (it overlaps its neighbour) so that
    // it can take the vector path like any full tile; its epilogue covers only the rows from m_lo and the columns
    // from n_lo on, the part no other tile writes. (Columns move in whole 8-element slabs only; an operand whose
    // rows are the contiguous axis needs the new origin 16-byte aligned.)
    uint32_t m0 = tm * BM, n0 = tn * BN;
    uint32_t m_lo = m0, m_end = h.m;  // the rows of the output this tile stores
    const uint32_t n_lo = n0;
    bool k_fast = true;
    if (gmode != VCG_NONE) {
      const uint32_t g_lo = bi1 != 0u ? uni(gtab[bi1 - 1u]) : 0u;
      uint32_t g_hi = uni(gtab[bi1]);
      g_hi = g_hi > g_lo ? g_hi : g_lo;
      if (gmode == VCG_M_BOUND || gmode == VCG_M_SIZE) {
        // the rows of the tile that belong to this group; none: the tile is another group's
        const uint32_t t_hi = m0 + BM < h.m ? m0 + BM : h.m;
        m_lo = m0 > g_lo ? m0 : g_lo;
        m_end = t_hi < g_hi ? t_hi : g_hi;
        if (m_lo >= m_end) continue;
      } else {
        // the group's part of the k axis; the vector path takes it when it is whole steps from an aligned start
        k_lo = g_lo;
        k_hi = g_hi;
        k_fast = (k_lo & 7u) == 0u && k_hi > k_lo && ((k_hi - k_lo) & 63u) == 0u;
      }
    }
    if (h.fast) {
      if (m0 + BM > h.m && h.m >= BM && (A_KC || (h.m & 7u) == 0)) m0 = h.m - BM;
      if (n0 + BN > h.n && h.n >= BN && (h.n & 7u) == 0) n0 = h.n - BN;
    }
    const uint64_t a_base = h.a_addr + (static_cast<uint64_t>(bi0) * h.a_sb0 + static_cast<uint64_t>(bi1) * h.a_sb1) * 2;
    const uint64_t b_base = h.b_addr + (static_cast<uint64_t>(bi0) * h.b_sb0 + static_cast<uint64_t>(bi1) * h.b_sb1) * 2;

    vf16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = 0.0f;

    constexpr bool RING = BM == 256 && BN == 256;  // the ring of 32-deep stages
    // The smallest tile also takes the vector path when an operand with contiguous k has fewer rows than the tile
    // (one to 63 rows of A against a weight matrix): the rows past the end fetch the last valid row.
    constexpr bool a_clamps = !RING && A_KC && (BM * BK / 8 / NTHR) <= 2, b_clamps = !RING && B_KC && (BN * BK / 8 / NTHR) <= 2;
    const uint32_t a_rows = h.m - m0 < static_cast<uint32_t>(BM) ? h.m - m0 : static_cast<uint32_t>(BM);
    const uint32_t b_rows = h.n - n0 < static_cast<uint32_t>(BN) ? h.n - n0 : static_cast<uint32_t>(BN);
    // The guarded walk over a part of the k axis: any start, any length, rows and columns past the edges read as zero.
    const uint32_t a_vec = ((h.lda & 7u) == 0u && (a_base & 15u) == 0u) ? 1u : 0u;
    const uint32_t b_vec = ((h.ldb & 7u) == 0u && (b_base & 15u) == 0u) ? 1u : 0u;
    auto guarded_walk = [&](uint32_t from, uint32_t to) {
      for (uint32_t k0 = from; k0 < to; k0 += BK) {
        stage_generic<BM, NTHR>(lds, a_base, h.lda, m0, k0, h.m, to, A_KC ? 1u : 0u, a_vec, tid);
        stage_generic<BN, NTHR>(lds + kBBase, b_base, h.ldb, n0, k0, h.n, to, B_KC ? 1u : 0u, b_vec, tid);
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
          vu4 af[TM], bf[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const vu4 *>(lds + frag_off(a_row, a_x, i, kk));
#pragma unroll
          for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const vu4 *>(lds + frag_off(b_row, b_x, j, kk));
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma<IS_BF16>(af[i], bf[j], acc[i][j]);
        }
        __syncthreads();
      }
    };
    // A group's part of the k axis that is not whole steps from an aligned start: the vector path takes the steps in
    // its middle, the guarded walk the few k in front (up to the next multiple of 8) and behind (less than a step).
    uint32_t tail_lo = 0, tail_hi = 0;
    if constexpr (!COMB) {
      if (!g_rows && gmode != VCG_NONE && !k_fast && h.fast && k_hi > k_lo && (m0 + BM <= h.m || a_clamps) && (n0 + BN <= h.n || b_clamps)) {
        const uint32_t up8 = (k_lo + 7u) & ~7u;
        const uint32_t f_lo = up8 < k_hi ? up8 : k_hi;
        const uint32_t f_hi = f_lo + ((k_hi - f_lo) & ~63u);
        if (f_hi > f_lo) {
          if (f_lo > k_lo) guarded_walk(k_lo, f_lo);
          tail_lo = f_hi;
          tail_hi = k_hi;
          k_lo = f_lo;
          k_hi = f_hi;
          k_fast = true;
        }
      }
    }
    const uint32_t nk = (k_hi - k_lo + BK - 1) / BK;
    // address of element (row0, k_lo) of each operand
    const uint64_t a_org = a_base + (A_KC ? static_cast<uint64_t>(m0) * h.lda + k_lo : static_cast<uint64_t>(k_lo) * h.lda + m0) * 2;
    const uint64_t b_org = b_base + (B_KC ? static_cast<uint64_t>(n0) * h.ldb + k_lo : static_cast<uint64_t>(k_lo) * h.ldb + n0) * 2;
    if constexpr (COMB) {
      const DVM_GLOBAL vf4 *src = reinterpret_cast<const DVM_GLOBAL vf4 *>(h.part_addr) + static_cast<uint64_t>(tile_id) * kPartVecs * NTHR + tid;
      const uint64_t split_stride = static_cast<uint64_t>(n_tiles) * kPartVecs * NTHR;
      // One fragment (16 registers) at a time, its vectors of four or eight parts in flight together: a trip to memory
      // per fragment and group of parts instead of several per part (a single workgroup per tile is latency bound);
      // the parts are still added in ascending order.
      constexpr int PC = TM * TN == 4 ? 8 : 4;  // (fewer where the accumulators take half the registers, or two workgroups share a compute unit)
      for (uint32_t sp0 = 0; sp0 < h.k_split; sp0 += PC) {
        const uint32_t n_here = h.k_split - sp0 < static_cast<uint32_t>(PC) ? h.k_split - sp0 : static_cast<uint32_t>(PC);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            vf4 v[PC][4];
            const DVM_GLOBAL vf4 *frag = src + sp0 * split_stride + static_cast<uint32_t>((i * TN + j) * 4) * NTHR;
#pragma unroll
            for (int pp = 0; pp < PC; ++pp) {
              if (static_cast<uint32_t>(pp) < n_here) {
#pragma unroll
                for (int q = 0; q < 4; ++q) v[pp][q] = frag[pp * split_stride + static_cast<uint32_t>(q) * NTHR];
              }
            }
#pragma unroll
            for (int pp = 0; pp < PC; ++pp) {
              if (static_cast<uint32_t>(pp) < n_here) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                  for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += v[pp][q][e];
              }
            }
          }
      }
    } else {
    if (h.fast && k_fast && (m0 + BM <= h.m || a_clamps) && (n0 + BN <= h.n || b_clamps)) {
     if constexpr (RING) {
      tile_loop_ring<IS_BF16, A_KC, B_KC, WM>(acc, lds, a_org, b_org, h.lda, h.ldb, (k_hi - k_lo) / SK, tid);
     } else {
      Stage<BM, A_KC, NTHR> sa;
      Stage<BN, B_KC, NTHR> sb;
      // k advances by BK per step
      const uint64_t a_step = (A_KC ? static_cast<uint64_t>(BK) : static_cast<uint64_t>(BK) * h.lda) * 2;
      const uint64_t b_step = (B_KC ? static_cast<uint64_t>(BK) : static_cast<uint64_t>(BK) * h.ldb) * 2;
      LaneOffsets a_voff, b_voff;
      if constexpr (A_KC) a_voff = Stage<BM, A_KC, NTHR>::lane_offset(h.lda, tid, a_rows);
      else a_voff = Stage<BM, A_KC, NTHR>::lane_offset(h.lda, tid);
      if constexpr (B_KC) b_voff = Stage<BN, B_KC, NTHR>::lane_offset(h.ldb, tid, b_rows);
      else b_voff = Stage<BN, B_KC, NTHR>::lane_offset(h.ldb, tid);
      sa.fetch(a_org, h.lda, a_voff, tid, lds);
      sb.fetch(b_org, h.ldb, b_voff, tid, lds + kBBase);
      sa.commit(lds, tid);
      sb.commit(lds + kBBase, tid);
      if (nk > 1) {
        sa.fetch(a_org + a_step, h.lda, a_voff, tid, lds + kABuf);
        sb.fetch(b_org + b_step, h.ldb, b_voff, tid, lds + kBBase + kBBuf);
      }
      __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0): direct loads are not waited for by the barrier itself
      __syncthreads();
      vu4 af[2][TM], bf[2][TN];
      auto read_frags = [&](int fb, uint32_t buf, int kk) {
        const uint16_t *ab = lds + buf * kABuf, *bb = lds + buf * kBBuf;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[fb][i] = *reinterpret_cast<const vu4 *>(ab + frag_off(a_row, a_x, i, kk));
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[fb][j] = *reinterpret_cast<const vu4 *>(bb + frag_off(b_row, b_x, j, kk));
      };
      auto mfmas = [&](int fb) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = mfma<IS_BF16>(af[fb][i], bf[fb][j], acc[i][j]);
      };
      // One k tile (4 steps of 16). Step s runs its MFMAs on fragment buffer s&1 while the reads of
      // step s+1 land in the other one. A k-strided operand's tile kt+1 is written to the other
      // local-memory buffer during step 1 (its global loads were issued three steps earlier) and the
      // global loads of its tile kt+2 follow in step 2; the workgroup meets before step 3, which overlaps
      // the first fragment reads of tile kt+1 and sends the direct loads of tile kt+2 of a k-contiguous
      // operand into the buffer that has just been read for the last time (a whole tile of slack).
      // The group barriers pin that interleaving: the scheduler would otherwise serialise each read
      // against its use to save registers, and with one wave per SIMD nothing else hides the latency.
      auto k_tile = [&](uint32_t kt, auto has_next, auto has_next2) {
        constexpr bool NEXT = decltype(has_next)::value, NEXT2 = decltype(has_next2)::value;
        constexpr int NF = TM + TN, NM = TM * TN;
        const uint32_t cur = kt & 1u;
        constexpr int NREST = NM - NF > 0 ? NM - NF : 1;  // MFMAs left in a step after the fragment reads
        // staging instructions per such MFMA: ds_write of a k-strided operand (step 1), its global loads
        // (step 2), direct-to-LDS loads of a k-contiguous operand (step 3)
        constexpr int NW = ((A_KC ? 0 : Stage<BM, false, NTHR>::N_WRITES) + (B_KC ? 0 : Stage<BN, false, NTHR>::N_WRITES) + NREST - 1) / NREST;
        constexpr int NL = ((A_KC ? 0 : 8) + (B_KC ? 0 : 8) + NREST - 1) / NREST;
        constexpr int ND = ((A_KC ? Stage<BM, true, NTHR>::N : 0) + (B_KC ? Stage<BN, true, NTHR>::N : 0) + NREST - 1) / NREST;
        // step 0
        __builtin_amdgcn_sched_barrier(0);
        read_frags(1, cur, 1);
        mfmas(0);
#pragma unroll
        for (int q = 0; q < NF; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, NM - NF > 0 ? NM - NF : 0, 0);
        // step 1: tile kt+1 (loaded during the previous tile) goes to the other buffer
        __builtin_amdgcn_sched_barrier(0);
        read_frags(0, cur, 2);
        if constexpr (NEXT) {
          sa.commit(lds + (cur ^ 1u) * kABuf, tid);
          sb.commit(lds + kBBase + (cur ^ 1u) * kBBuf, tid);
        }
        mfmas(1);
#pragma unroll
        for (int q = 0; q < NF; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        if constexpr (NEXT && NW > 0) {
#pragma unroll
          for (int q = 0; q < NREST; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x200, NW, 0);
          }
        }
        // step 2: the staging registers are free again: tile kt+2 starts its way from memory
        __builtin_amdgcn_sched_barrier(0);
        read_frags(1, cur, 3);
        if constexpr (NEXT2 && !A_KC) sa.fetch(a_org + (kt + 2) * a_step, h.lda, a_voff, tid, lds);
        if constexpr (NEXT2 && !B_KC) sb.fetch(b_org + (kt + 2) * b_step, h.ldb, b_voff, tid, lds);
        mfmas(0);
#pragma unroll
        for (int q = 0; q < NF; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        if constexpr (NEXT2 && NL > 0) {
#pragma unroll
          for (int q = 0; q < NREST; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, NL, 0);
          }
        }
        // step 3: every wave has read its last fragments of this buffer and written its share of the
        // next one a step ago; meet, then start on the next tile's fragments under the last MFMAs
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NEXT) {
          // the direct loads of tile kt+1 (issued a tile ago) must have landed before anyone reads them; the
          // only younger memory operations of this wave are the step-2 loads of a k-strided operand
          if constexpr (A_KC || B_KC) {
            constexpr int YOUNGER = (BM == 256 && BN == 256 && NEXT2) ? ((A_KC ? 0 : 8) + (B_KC ? 0 : 8)) : 0;
            __builtin_amdgcn_s_waitcnt((YOUNGER & 0xf) | ((YOUNGER >> 4) << 14) | (7 << 4) | (15 << 8));
          }
          __syncthreads();
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NEXT) read_frags(0, cur ^ 1u, 0);
        // this buffer has been read for the last time: tile kt+2 of a k-contiguous operand starts its way into it
        if constexpr (NEXT2 && A_KC) sa.fetch(a_org + (kt + 2) * a_step, h.lda, a_voff, tid, lds + cur * kABuf);
        if constexpr (NEXT2 && B_KC) sb.fetch(b_org + (kt + 2) * b_step, h.ldb, b_voff, tid, lds + kBBase + cur * kBBuf);
        mfmas(1);
        if constexpr (NEXT) {
#pragma unroll
          for (int q = 0; q < NF; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
        }
        if constexpr (NEXT2 && ND > 0) {
#pragma unroll
          for (int q = 0; q < NREST; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, ND, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      read_frags(0, 0, 0);
      uint32_t kt = 0;
      for (; kt + 2 < nk; ++kt) k_tile(kt, std::true_type{}, std::true_type{});
      if (kt + 1 < nk) {
        k_tile(kt, std::true_type{}, std::false_type{});
        ++kt;
      }
      k_tile(kt, std::false_type{}, std::false_type{});
      __syncthreads();
     }
    } else {
      guarded_walk(k_lo, k_hi);
    }
    if (tail_hi > tail_lo) guarded_walk(tail_lo, tail_hi);
    }

    if (split_part) {
      DVM_GLOBAL vf4 *dst = reinterpret_cast<DVM_GLOBAL vf4 *>(h.part_addr) +
                            (static_cast<uint64_t>(ksplit) * n_tiles + tile_id) * kPartVecs * NTHR + tid;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const vf16 &c = acc[i][j];
            const vf4 v = {c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
            dst[static_cast<uint32_t>((i * TN + j) * 4 + q) * NTHR] = v;
          }
      continue;
    }
    // epilogue: accumulators -> local memory (row major), then slabs through the program
    if (h.epi_flags & VCF_DUMP16) {
      // The program starts with [add of a bias row] [rounding to the operand type]: done here, where a lane's column
      // is fixed (one bias value per fragment column). The rounded values are kept as their 16 bits, so the whole
      // tile fits local memory and goes through the epilogue in one pass, with no accumulator left alive across it.
      constexpr int D16K = IS_BF16 ? 1 : 2;
      constexpr int P16 = BN + 8;
      const uint32_t *code32 = prog32 + 2 * h.code_off;
      const uint32_t w_first = uni(code32[0]);
      uint32_t first = 0;
      float bias[TN];
#pragma unroll
      for (int j = 0; j < TN; ++j) bias[j] = 0.0f;
      if ((w_first & 0xffu) == VOP_BINF) {
        first = 1;
        const uint32_t *d = prog32 + 2 * h.mem_off + (w_first >> 24) * (sizeof(VCubeMem) / 4);
        const uint64_t addr = static_cast<uint64_t>(uni(d[0])) | (static_cast<uint64_t>(uni(d[1])) << 32);
        const uint32_t dtype = uni(d[2]);
        const uint64_t boff = static_cast<uint64_t>(bi0) * uni(d[6]) + static_cast<uint64_t>(bi1) * uni(d[7]);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const uint32_t col = n0 + (wn * TN + j) * 32 + (lane & 31u);
          const uint64_t at = boff + (col < h.n ? col : 0u);  // (columns past the edge are never stored)
          bias[j] = dtype == VDT_F32 ? reinterpret_cast<const DVM_GLOBAL float *>(addr)[at]
                                     : cvt_in(dtype, reinterpret_cast<const DVM_GLOBAL uint16_t *>(addr)[at]);
        }
      }
      // (the rounding is the next instruction, or what the program's one store does anyway)
      if ((uni(code32[2 * first]) & 0xffu) == VOP_CAST) ++first;
      const EpiArgs ea = {h.mem_off, h.code_off, bi0, bi1, h.epi_flags, h.n_code, 0, first};
      uint16_t *tile16 = reinterpret_cast<uint16_t *>(lds_raw);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const vf16 &c = acc[i][j];
          // lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4 of the fragment
          uint16_t *dst = tile16 + (wm * (TM * 32) + i * 32 + (lane >> 5) * 4) * P16 + (wn * TN + j) * 32 + (lane & 31u);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float v = c[r] + bias[j];
            uint16_t bits;
            if constexpr (IS_BF16) bits = static_cast<uint16_t>(__float_as_uint(round_bf16(v)) >> 16);
            else bits = __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
            dst[(8 * (r / 4) + (r % 4)) * P16] = bits;
          }
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (!(h.epi_flags & VCF_PLAIN_STORE) || !epilogue_plain_pass<BM, BN, TM, WM, D16K>(tile16, prog32, ea, m0, n0, 0, m_end, h.n, m_lo, n_lo)) {
        if (h.epi_flags & VCF_SLIM) {
          epilogue_pass_body<BM, BN, TM, WM, true, D16K>(tile16, prog32, ea, m0, n0, 0, m_end, h.n, m_lo, n_lo);
        }
        else epilogue_pass<BM, BN, TM, WM, false, D16K>(tile16, prog32, ea, m0, n0, 0, m_end, h.n, m_lo, n_lo);
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      continue;
    }
    const EpiArgs ea = {h.mem_off, h.code_off, bi0, bi1, h.epi_flags, h.n_code, 0, 0};
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      constexpr int FR = TM / PASSES;  // fragment rows of a wave per pass
#pragma unroll
      for (int fi = 0; fi < FR; ++fi) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const vf16 &c = acc[ps * FR + fi][j];
          // lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4 of the fragment
          float *dst = dump + (wm * (PROWS / WM) + fi * 32 + (lane >> 5) * 4) * PITCH + (wn * TN + j) * 32 + (lane & 31u);
#pragma unroll
          for (int r = 0; r < 16; ++r) dst[(8 * (r / 4) + (r % 4)) * PITCH] = c[r];
        }
      }
      // The two meetings of a pass order local-memory accesses only (the dump before the slabs are read, the reads
      // before the next dump): they wait for this wave's local-memory operations and not, as __syncthreads() would,
      // for its stores to memory as well, which stay in flight under the next pass and the next tile's loop.
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (!(h.epi_flags & VCF_PLAIN_STORE) || !epilogue_plain_pass<PROWS, BN, TM, WM, 0>(dump, prog32, ea, m0, n0, ps, m_end, h.n, m_lo, n_lo)) {
        if (h.epi_flags & VCF_SLIM) epilogue_pass<PROWS, BN, TM, WM, true, 0>(dump, prog32, ea, m0, n0, ps, m_end, h.n, m_lo, n_lo);
        else epilogue_pass<PROWS, BN, TM, WM, false, 0>(dump, prog32, ea, m0, n0, ps, m_end, h.n, m_lo, n_lo);
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
  }
}

}  // namespace

// `occ` = waves per SIMD the register budget must leave room for (two workgroups of the 64x64 tile share a compute unit:
// 256 registers a lane, vector and accumulation registers together)
#define DVM_CUBE_KERNEL(name, bf, tm, tn, wm, occ, akc, bkc) \
  extern "C" __global__ void __launch_bounds__(wm * 128, occ) name(const VmParam p) { vm_cube<bf, tm, tn, akc, bkc, wm>(p); }
#define DVM_CUBE_LAYOUTS(prefix, bf, tm, tn, wm, occ)            \
  DVM_CUBE_KERNEL(prefix##_nn, bf, tm, tn, wm, occ, true, false) \
  DVM_CUBE_KERNEL(prefix##_nt, bf, tm, tn, wm, occ, true, true)  \
  DVM_CUBE_KERNEL(prefix##_tn, bf, tm, tn, wm, occ, false, false) \
  DVM_CUBE_KERNEL(prefix##_tt, bf, tm, tn, wm, occ, false, true)

#define DVM_CUBE_COMB(name, bf, tm, tn, wm, occ) \
  extern "C" __global__ void __launch_bounds__(wm * 128, occ) name(const VmParam p) { vm_cube<bf, tm, tn, true, false, wm, true>(p); }
DVM_CUBE_COMB(dvm_vm_cube_bf16_big_comb, true, 4, 4, 2, 1)
DVM_CUBE_COMB(dvm_vm_cube_f16_big_comb, false, 4, 4, 2, 1)
DVM_CUBE_COMB(dvm_vm_cube_bf16_mid_comb, true, 2, 2, 2, 1)
DVM_CUBE_COMB(dvm_vm_cube_f16_mid_comb, false, 2, 2, 2, 1)
DVM_CUBE_COMB(dvm_vm_cube_bf16_small_comb, true, 1, 1, 2, 2)
DVM_CUBE_COMB(dvm_vm_cube_f16_small_comb, false, 1, 1, 2, 2)
DVM_CUBE_COMB(dvm_vm_cube_bf16_big8_comb, true, 2, 4, 4, 2)
DVM_CUBE_COMB(dvm_vm_cube_f16_big8_comb, false, 2, 4, 4, 2)
DVM_CUBE_LAYOUTS(dvm_vm_cube_bf16_big, true, 4, 4, 2, 1)
DVM_CUBE_LAYOUTS(dvm_vm_cube_f16_big, false, 4, 4, 2, 1)
DVM_CUBE_LAYOUTS(dvm_vm_cube_bf16_mid, true, 2, 2, 2, 1)
DVM_CUBE_LAYOUTS(dvm_vm_cube_f16_mid, false, 2, 2, 2, 1)
DVM_CUBE_LAYOUTS(dvm_vm_cube_bf16_small, true, 1, 1, 2, 2)
DVM_CUBE_LAYOUTS(dvm_vm_cube_f16_small, false, 1, 1, 2, 2)
// the 256x256 tile on eight waves (4 x 2, 64x128 accumulators each): two waves per SIMD
DVM_CUBE_LAYOUTS(dvm_vm_cube_bf16_big8, true, 2, 4, 4, 2)
DVM_CUBE_LAYOUTS(dvm_vm_cube_f16_big8, false, 2, 4, 4, 2)
