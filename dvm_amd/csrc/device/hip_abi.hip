// C ABI of the device layer: VM init / launch geometry / launch, and the thin
// runtime wrappers the host emitter needs (see include/dvm_hip.h for the
// reference interfaces each entry point replaces).
#include <hip/hip_runtime.h>
#include <algorithm>
#include <stdint.h>
#include <string.h>

#include <vector>

#include "../../../include/dvm_hip.h"
#include "../isa_gfx950.h"

extern "C" __global__ void dvm_vm_vec_pw(const VmParam p);
extern "C" __global__ void dvm_vm_vec_rx(const VmParam p);
extern "C" __global__ void dvm_vm_vec_ry(const VmParam p);
extern "C" __global__ void dvm_vm_vec_rx_parts(const VmParam p);
extern "C" __global__ void dvm_vm_vec_ry_parts(const VmParam p);
extern "C" __global__ void dvm_vm_vec_rx_sw(const VmParam p);
extern "C" __global__ void dvm_vm_vec_rx_sw_parts(const VmParam p);
extern "C" __global__ void dvm_vm_vec_pw_u4(const VmParam p);
extern "C" __global__ void dvm_vm_vec_rx_u4(const VmParam p);
extern "C" __global__ void dvm_vm_vec_ry_u4(const VmParam p);
#define DVM_CUBE_DECL(prefix)                                \
  extern "C" __global__ void prefix##_nn(const VmParam p); \
  extern "C" __global__ void prefix##_nt(const VmParam p); \
  extern "C" __global__ void prefix##_tn(const VmParam p); \
  extern "C" __global__ void prefix##_tt(const VmParam p);
DVM_CUBE_DECL(dvm_vm_cube_bf16_big)
DVM_CUBE_DECL(dvm_vm_cube_f16_big)
DVM_CUBE_DECL(dvm_vm_cube_bf16_mid)
DVM_CUBE_DECL(dvm_vm_cube_f16_mid)
DVM_CUBE_DECL(dvm_vm_cube_bf16_small)
DVM_CUBE_DECL(dvm_vm_cube_f16_small)
DVM_CUBE_DECL(dvm_vm_cube_bf16_big8)
DVM_CUBE_DECL(dvm_vm_cube_f16_big8)
// the builds that sum the partial tiles of a split k axis (second launch), [tile][bf16] below
extern "C" __global__ void dvm_vm_cube_f16_big_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_bf16_big_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_f16_mid_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_bf16_mid_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_f16_small_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_bf16_small_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_f16_big8_comb(const VmParam p);
extern "C" __global__ void dvm_vm_cube_bf16_big8_comb(const VmParam p);

extern "C" __global__ void dvm_vm_attn_f16(const VmParam p);
extern "C" __global__ void dvm_vm_attn_bf16(const VmParam p);
extern "C" __global__ void dvm_vm_attn_f16_w8(const VmParam p);
extern "C" __global__ void dvm_vm_attn_bf16_w8(const VmParam p);
extern "C" __global__ void dvm_vm_attn_f16_d64(const VmParam p);
extern "C" __global__ void dvm_vm_attn_bf16_d64(const VmParam p);
extern "C" __global__ void dvm_vm_attn_f16_w8_d64(const VmParam p);
extern "C" __global__ void dvm_vm_attn_bf16_w8_d64(const VmParam p);

typedef void (*CubeKernel)(const VmParam);
#define DVM_CUBE_ROW(prefix) {prefix##_nn, prefix##_nt, prefix##_tn, prefix##_tt}
// [tile][bf16][trans_a * 2 + trans_b]
static const CubeKernel kCubeKernels[4][2][4] = {
    {DVM_CUBE_ROW(dvm_vm_cube_f16_big), DVM_CUBE_ROW(dvm_vm_cube_bf16_big)},
    {DVM_CUBE_ROW(dvm_vm_cube_f16_mid), DVM_CUBE_ROW(dvm_vm_cube_bf16_mid)},
    {DVM_CUBE_ROW(dvm_vm_cube_f16_small), DVM_CUBE_ROW(dvm_vm_cube_bf16_small)},
    {DVM_CUBE_ROW(dvm_vm_cube_f16_big8), DVM_CUBE_ROW(dvm_vm_cube_bf16_big8)}};
static const CubeKernel kCubeCombKernels[4][2] = {{dvm_vm_cube_f16_big_comb, dvm_vm_cube_bf16_big_comb},
                                                  {dvm_vm_cube_f16_mid_comb, dvm_vm_cube_bf16_mid_comb},
                                                  {dvm_vm_cube_f16_small_comb, dvm_vm_cube_bf16_small_comb},
                                                  {dvm_vm_cube_f16_big8_comb, dvm_vm_cube_bf16_big8_comb}};

// The workspace of dvm_hip_launch_vm_static_ws: device memory that belongs to the library's code object, one copy
// per device. Host code never uses this name as an address: it asks the runtime for the array's address on the
// current device (hipGetSymbolAddress) and passes that.
static __device__ __align__(256) unsigned char dvm_static_ws[DVM_HIP_STATIC_WS_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void *g_static_ws[kMaxDevices] = {nullptr};  // address of dvm_static_ws on each device, looked up once per device

// Address of the static workspace on the current device (no allocation: the array exists since the code object
// was loaded there).
int static_ws_address(void **out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return static_cast<int>(err);
  if (dev < 0 || dev >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
  if (g_static_ws[dev] == nullptr) {
    void *p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(dvm_static_ws));
    if (err != hipSuccess) return static_cast<int>(err);
    if (p == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    g_static_ws[dev] = p;
  }
  *out = g_static_ws[dev];
  return 0;
}

struct DeviceInfo {
  bool ready = false;
  int dev = -1;
  uint32_t cus = 256;
  uint32_t lds_per_cu = 160 * 1024;
  uint32_t lds_per_wg = 64 * 1024;
};
DeviceInfo g_dev;

__global__ void dvm_fill_u32_kernel(uint32_t *dst, uint32_t value, size_t n) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (; i < n; i += stride) dst[i] = value;
}

// waves per SIMD each interpreter kernel fits at (from its VGPR count, allocated in blocks of 8: 92, 102 and 127
// registers). The grid is a multiple of what is resident: one workgroup too many per CU costs a whole extra pass.
uint32_t kernel_waves_per_simd(uint64_t kind) {
  if (kind & VS_WIDE) return 2;
  switch (kind & VS_KIND_MASK) {
    case VS_POINTWISE: return 5;
    case VS_REDX: return 4;
    case VS_REDY: return 4;
    default: return 2;
  }
}

}  // namespace

extern "C" {

int dvm_hip_init_vm(int dev_id, dvm_hip_sysconfig *conf) {
  int count = 0;
  hipError_t err = hipGetDeviceCount(&count);
  if (err != hipSuccess) return static_cast<int>(err);
  if (dev_id < 0 || dev_id >= count) return static_cast<int>(hipErrorInvalidDevice);
  // The limits below (compute units, local memory) are one set per process: a second call has to name the same
  // device. (One process drives one GPU; another device's limits would silently replace the first's otherwise.)
  if (g_dev.ready && g_dev.dev != dev_id) return DVM_HIP_ERROR_OTHER_DEVICE;
  err = hipSetDevice(dev_id);
  if (err != hipSuccess) return static_cast<int>(err);
  hipDeviceProp_t prop;
  err = hipGetDeviceProperties(&prop, dev_id);
  if (err != hipSuccess) return static_cast<int>(err);
  g_dev.dev = dev_id;
  g_dev.cus = static_cast<uint32_t>(prop.multiProcessorCount);
  g_dev.lds_per_cu = static_cast<uint32_t>(prop.maxSharedMemoryPerMultiProcessor);
  if (g_dev.lds_per_cu == 0) g_dev.lds_per_cu = 64 * 1024;
  g_dev.lds_per_wg = static_cast<uint32_t>(prop.sharedMemPerBlock);
  // gfx950 lets one workgroup use the CU's whole 160 KB; the kernels must opt in.
  std::vector<const void *> kernels = {reinterpret_cast<const void *>(dvm_vm_vec_pw), reinterpret_cast<const void *>(dvm_vm_vec_rx),
                                       reinterpret_cast<const void *>(dvm_vm_vec_ry), reinterpret_cast<const void *>(dvm_vm_vec_rx_parts),
                                       reinterpret_cast<const void *>(dvm_vm_vec_ry_parts),
                                       reinterpret_cast<const void *>(dvm_vm_vec_rx_sw), reinterpret_cast<const void *>(dvm_vm_vec_rx_sw_parts),
                                       reinterpret_cast<const void *>(dvm_vm_vec_pw_u4), reinterpret_cast<const void *>(dvm_vm_vec_rx_u4),
                                       reinterpret_cast<const void *>(dvm_vm_vec_ry_u4)};
  for (const auto &tile : kCubeKernels)
    for (const auto &dt : tile)
      for (CubeKernel k : dt) kernels.push_back(reinterpret_cast<const void *>(k));
  for (const auto &tile : kCubeCombKernels)
    for (CubeKernel k : tile) kernels.push_back(reinterpret_cast<const void *>(k));
  for (const void *k : {reinterpret_cast<const void *>(dvm_vm_attn_f16), reinterpret_cast<const void *>(dvm_vm_attn_bf16),
                        reinterpret_cast<const void *>(dvm_vm_attn_f16_w8), reinterpret_cast<const void *>(dvm_vm_attn_bf16_w8),
                        reinterpret_cast<const void *>(dvm_vm_attn_f16_d64), reinterpret_cast<const void *>(dvm_vm_attn_bf16_d64),
                        reinterpret_cast<const void *>(dvm_vm_attn_f16_w8_d64), reinterpret_cast<const void *>(dvm_vm_attn_bf16_w8_d64)})
    kernels.push_back(k);
  for (const void *k : kernels) {
    if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(g_dev.lds_per_cu)) ==
        hipSuccess) {
      g_dev.lds_per_wg = g_dev.lds_per_cu;
    } else {
      (void)hipGetLastError();
    }
  }
  {
    // the static workspace of dvm_hip_launch_vm_static_ws: its address on this device, looked up once, here
    void *ws = nullptr;
    const int rc = static_ws_address(&ws);
    if (rc != 0) return rc;
  }
  g_dev.ready = true;
  if (conf != nullptr) {
    conf->core_num = g_dev.cus;
    conf->local_mem_size = g_dev.lds_per_wg;
    conf->default_threads = 256;
    conf->wave_size = static_cast<uint64_t>(prop.warpSize);
    conf->l2_bytes = static_cast<uint64_t>(prop.l2CacheSize);
    conf->xcd_num = 8;
  }
  return 0;
}

uint64_t dvm_hip_select_block_thread(uint64_t kind, uint64_t item_num, uint64_t threads, uint32_t lds_bytes) {
  if (threads == 0) threads = 256;
  const uint64_t waves_per_wg = (threads + 63) / 64;
  uint64_t wg_per_cu = (4ull * kernel_waves_per_simd(kind)) / waves_per_wg;
  if (lds_bytes > 0) {
    const uint64_t by_lds = g_dev.lds_per_cu / lds_bytes;
    if (by_lds < wg_per_cu) wg_per_cu = by_lds;
  }
  if (wg_per_cu == 0) wg_per_cu = 1;
  uint64_t blocks = static_cast<uint64_t>(g_dev.cus) * wg_per_cu;
  if (blocks > item_num) blocks = item_num;
  if (blocks == 0) blocks = 1;
  return (blocks << 32) | threads;
}

// The sweep build decodes a sweep as [VOP_SWEEP] [VOP_LD] [body of at most DVM_VEC_SWEEP_BODY words, the last one
// flagged VI_ENDS] without looking for anything else: a blob that carries VS_SWEEPS must have that shape. (The
// table offsets have been checked by the caller.)
static bool sweeps_flag_holds(const VmParam &p) {
  const VVecHeader *h = reinterpret_cast<const VVecHeader *>(p.w);
  const uint64_t *code = p.w + h->code_off;
  const VMemDesc *mems = reinterpret_cast<const VMemDesc *>(p.w + h->mem_off);
  if (h->n_kdim > 2 || h->n_rdim > 2) return false;
  // an operand of a sweep is accessed without guards in the interior rounds: contiguous and 16-byte aligned, or one
  // fp32 element per slab
  auto unguarded_ok = [&](uint32_t a, bool must_be_wide) {
    const VMemDesc &m = mems[a];
    constexpr uint32_t kWide = VMF_VEC | VMF_ALIGNED;
    if ((m.flags & (kWide | VMF_GATHER)) == kWide) return (m.addr & 15u) == 0;
    return !must_be_wide && (m.flags & (VMF_VEC | VMF_GATHER)) == 0 && m.dtype == VDT_F32;
  };
  for (uint32_t i = 0; i < h->n_code; ++i) {
    const uint32_t op = VI_OP(code[i]);
    if (op == VOP_LDR || op == VOP_STR || op == VOP_RED || op == VOP_LDX) return false;  // (outside a sweep)
    if (op >= VOP_SRC_BASE || op == VOP_ST) {
      if ((op >= VOP_SRC_BASE && VI_KIND(code[i]) == VK_REG) || ((VI_KIND(code[i]) == VK_MEM || op == VOP_ST) && VI_A(code[i]) >= h->n_mem)) return false;
    }
    if (op != VOP_SWEEP) continue;
    if (i + 2 >= h->n_code || VI_OP(code[i + 1]) != VOP_LD || VI_A(code[i + 1]) >= h->n_mem || !unguarded_ok(VI_A(code[i + 1]), true)) return false;
    uint32_t j = i + 2;
    for (;; ++j) {
      if (j >= h->n_code || j - (i + 2) >= DVM_VEC_SWEEP_BODY) return false;
      const uint32_t bop = VI_OP(code[j]);
      if (bop != VOP_BINF && bop != VOP_RED && bop != VOP_ST && bop != VOP_UN && bop != VOP_CAST && bop != VOP_ENDSWEEP && bop != VOP_LD) return false;
      if (bop == VOP_LD && VI_KIND(code[j]) != VK_MEM) return false;
      if ((bop == VOP_ST || bop == VOP_LD || (bop == VOP_BINF && VI_KIND(code[j]) == VK_MEM)) &&
          (VI_A(code[j]) >= h->n_mem || !unguarded_ok(VI_A(code[j]), bop == VOP_ST))) return false;
      if (bop == VOP_BINF && VI_KIND(code[j]) == VK_REG) return false;
      if (static_cast<uint32_t>(code[j]) & VI_ENDS) break;
    }
    i = j;
  }
  return true;
}

// Checks one program blob against the launch it is to get and launches the interpreter kernel its entry type names.
static int launch_checked(const VmParam &p, uint32_t block_dim, uint32_t threads, uint32_t lds_bytes, void *stream, bool check_only = false) {
  if (block_dim == 0 || threads == 0 || threads > 1024 || (threads & 63u) != 0) {
    return static_cast<int>(hipErrorInvalidValue);
  }
  if (lds_bytes > g_dev.lds_per_wg) return static_cast<int>(hipErrorInvalidValue);
  const VVecHeader *h = reinterpret_cast<const VVecHeader *>(p.w);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (h->entry == VE_VECTOR) {
    // Reject blobs whose tables would be read outside the 4 KB argument.
    const uint64_t mem_end = static_cast<uint64_t>(h->mem_off) + static_cast<uint64_t>(h->n_mem) * (sizeof(VMemDesc) / 8);
    const uint64_t code_end = static_cast<uint64_t>(h->code_off) + h->n_code;
    if (mem_end > DVM_PARAM_WORDS || code_end > DVM_PARAM_WORDS || h->n_code == 0 ||
        VI_OP(p.w[code_end - 1]) != VOP_END || h->n_kdim > DVM_VEC_MAXR || h->n_rdim > DVM_VEC_MAXR) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    {
      // an operand without memory behind it (VDT_IOTA) is read element by element only, and never written
      const VMemDesc *mems = reinterpret_cast<const VMemDesc *>(p.w + h->mem_off);
      for (uint32_t i = 0; i < h->n_mem; ++i)
        if (mems[i].dtype > VDT_IOTA || (mems[i].dtype == VDT_IOTA && (mems[i].flags & VMF_ALIGNED))) return static_cast<int>(hipErrorInvalidValue);
      for (uint64_t i = h->code_off; i < code_end; ++i)
        if (VI_OP(p.w[i]) == VOP_ST && (VI_A(p.w[i]) >= h->n_mem || mems[VI_A(p.w[i])].dtype == VDT_IOTA)) return static_cast<int>(hipErrorInvalidValue);
    }
    const bool wide = (h->sched & VS_WIDE) != 0;
    if (wide && threads > 512) return static_cast<int>(hipErrorInvalidValue);
    // (the kernels that keep the innermost axis are built for at most 512 lanes as well)
    if ((h->sched & VS_KIND_MASK) == VS_REDY && threads > 512) return static_cast<int>(hipErrorInvalidValue);
    // the sweep build trusts the flag: it is only defined for programs that reduce the innermost axis, two slabs a lane
    const bool sweeps = (h->sched & VS_SWEEPS) != 0;
    if (sweeps && (wide || (h->sched & VS_KIND_MASK) != VS_REDX || !sweeps_flag_holds(p))) return static_cast<int>(hipErrorInvalidValue);
    // a reduce shared between workgroups: its parts are the outermost kept axis and cover the reduced index space
    const bool parts = h->r_chunk != 0;
    if (parts) {
      const uint32_t kind = h->sched & VS_KIND_MASK;
      if (wide || (kind != VS_REDX && kind != VS_REDY) || h->k_per_chunk == 0 || h->n_kidx % h->k_per_chunk != 0 || h->n_kdim == 0 ||
          h->kdims[h->n_kdim - 1].extent != h->n_kidx / h->k_per_chunk ||
          static_cast<uint64_t>(h->r_chunk) * (h->n_kidx / h->k_per_chunk) < h->n_ridx) {
        return static_cast<int>(hipErrorInvalidValue);
      }
    }
    {
      // local memory the interpreter will touch: reduce scratch, V registers, rounds parked by a load
      const uint64_t u = wide ? DVM_VEC_U_WIDE : 2;
      uint64_t need = static_cast<uint64_t>(DVM_VEC_RED_SCRATCH_DOUBLES(h->sched, threads)) * 8 + static_cast<uint64_t>(h->n_vslot) * u * 16 * threads;
      uint64_t parked = 0;
      for (uint64_t i = h->code_off; i < code_end; ++i) {
        if (VI_OP(p.w[i]) != VOP_LD) continue;
        if (static_cast<uint32_t>(p.w[i]) & (VI_LD_KEEP_WR | VI_LD_KEEP_RD)) {
          if (wide) return static_cast<int>(hipErrorInvalidValue);
          // rounds x bytes per slab: two 16-byte planes for fp32 values, one for values parked as fp16 / bf16
          const uint64_t planes = ((VI_IMM(p.w[i]) >> 20) & 3u) == VF_F32 ? 2 : 1;
          parked = std::max<uint64_t>(parked, (VI_IMM(p.w[i]) & 0xffffu) * planes);
        }
      }
      need += parked * threads * u * 16;
      if (lds_bytes < need) return static_cast<int>(hipErrorInvalidValue);
    }
    if ((h->sched & VS_KIND_MASK) > VS_REDY) return static_cast<int>(hipErrorInvalidValue);
    if (check_only) return 0;
    switch (h->sched & VS_KIND_MASK) {
      case VS_POINTWISE:
        hipLaunchKernelGGL(wide ? dvm_vm_vec_pw_u4 : dvm_vm_vec_pw, dim3(block_dim), dim3(threads), lds_bytes, s, p);
        break;
      case VS_REDX:
        if (sweeps) {
          hipLaunchKernelGGL(parts ? dvm_vm_vec_rx_sw_parts : dvm_vm_vec_rx_sw, dim3(block_dim), dim3(threads), lds_bytes, s, p);
        } else {
          hipLaunchKernelGGL(parts ? dvm_vm_vec_rx_parts : (wide ? dvm_vm_vec_rx_u4 : dvm_vm_vec_rx), dim3(block_dim), dim3(threads), lds_bytes, s, p);
        }
        break;
      case VS_REDY:
        hipLaunchKernelGGL(parts ? dvm_vm_vec_ry_parts : (wide ? dvm_vm_vec_ry_u4 : dvm_vm_vec_ry), dim3(block_dim), dim3(threads), lds_bytes, s, p);
        break;
      default:
        return static_cast<int>(hipErrorInvalidValue);
    }
  } else if (h->entry == VE_CUBE) {
    const VCubeHeader *c = reinterpret_cast<const VCubeHeader *>(p.w);
    const uint64_t mem_end = static_cast<uint64_t>(c->mem_off) + static_cast<uint64_t>(c->n_mem) * (sizeof(VCubeMem) / 8);
    const uint64_t code_end = static_cast<uint64_t>(c->code_off) + c->n_code;
    const uint32_t bt = (c->tile == 0 || c->tile == 3) ? 256u : (c->tile == 1 ? 128u : 64u);
    const uint32_t want_threads = c->tile == 3 ? 512u : 256u;  // tile 3: the 256x256 tile on eight waves
    // The tile loop trusts the header: check it describes the launch it gets.
    if (mem_end > DVM_PARAM_WORDS || code_end > DVM_PARAM_WORDS || c->n_code == 0 || VI_OP(p.w[code_end - 1]) != VOP_END ||
        c->tile > 3 || threads != want_threads || c->m == 0 || c->n == 0 || c->nb0 == 0 || c->nb1 == 0 ||
        c->tiles_m != (c->m + bt - 1) / bt || c->tiles_n != (c->n + bt - 1) / bt || lds_bytes < DVM_CUBE_LDS_BYTES(bt) ||
        c->a_addr == 0 || c->b_addr == 0 || (c->dtype != VDT_F16 && c->dtype != VDT_BF16)) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    if (c->group_mode != VCG_NONE) {
      // a grouped product: one inner batch axis (the groups), its list in memory, its table of bounds behind the tile
      // buffers in local memory, and the whole k axis per workgroup
      const bool rows = c->group_mode == VCG_M_BOUND || c->group_mode == VCG_M_SIZE;
      if (c->group_mode > VCG_K_SIZE || c->group_addr == 0 || (c->group_addr & (c->group_i32 ? 3u : 7u)) != 0 || c->nb0 != 1 ||
          c->nb1 > DVM_CUBE_MAX_GROUPS || (c->epi_flags & (VCF_SPLITK_PARTIAL | VCF_SPLITK_COMBINE)) != 0 ||
          lds_bytes < DVM_CUBE_LDS_BYTES(bt) + 8u * c->nb1 || (rows && (c->a_sb0 != 0 || c->a_sb1 != 0))) {
        return static_cast<int>(hipErrorInvalidValue);
      }
    }
    const bool k_groups = c->group_mode == VCG_K_BOUND || c->group_mode == VCG_K_SIZE;
    if (c->fast && (c->lda >= (1u << 22) || c->ldb >= (1u << 22) || (c->k % 64 != 0 && !k_groups) || c->k == 0 || c->lda % 8 != 0 || c->ldb % 8 != 0 ||
                    (c->a_addr & 15u) != 0 || (c->b_addr & 15u) != 0)) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    const uint32_t split = c->epi_flags & (VCF_SPLITK_PARTIAL | VCF_SPLITK_COMBINE);
    if (split != 0) {
      const uint64_t tiles = static_cast<uint64_t>(c->tiles_m) * c->tiles_n * c->nb0 * c->nb1;
      if (split == (VCF_SPLITK_PARTIAL | VCF_SPLITK_COMBINE) || c->k_split < 2 || c->k_chunk == 0 || c->k_chunk % 64 != 0 ||
          static_cast<uint64_t>(c->k_chunk) * (c->k_split - 1) >= c->k || static_cast<uint64_t>(c->k_chunk) * c->k_split < c->k ||
          c->part_addr == 0 || (c->part_addr & 15u) != 0 || tiles * c->k_split >= (1ull << 31)) {
        return static_cast<int>(hipErrorInvalidValue);
      }
    }
    const CubeKernel kern = (c->epi_flags & VCF_SPLITK_COMBINE)
                                ? kCubeCombKernels[c->tile][c->dtype == VDT_BF16 ? 1 : 0]
                                : kCubeKernels[c->tile][c->dtype == VDT_BF16 ? 1 : 0][(c->trans_a ? 2 : 0) + (c->trans_b ? 1 : 0)];
    if (check_only) return 0;
    hipLaunchKernelGGL(kern, dim3(block_dim), dim3(want_threads), lds_bytes, s, p);
  } else if (h->entry == VE_ATTN) {
    const VAttnHeader *a = reinterpret_cast<const VAttnHeader *>(p.w);
    // the kernel has no guards of its own beyond the query tail: the header must fit it exactly
    if (!DVM_ATTN_D_OK(a->d) || a->skv == 0 || !(a->scale > 0.0f) || a->sq == 0 || a->nb == 0 ||
        a->q_blocks != (a->sq + DVM_ATTN_BQ - 1) / DVM_ATTN_BQ || static_cast<uint64_t>(a->nb) * a->q_blocks != block_dim || (threads != 256 && threads != 512) ||
        lds_bytes < DVM_ATTN_LDS_BYTES_D(a->d) || a->q_addr == 0 || a->k_addr == 0 || a->v_addr == 0 || a->o_addr == 0 ||
        ((a->q_addr | a->k_addr | a->v_addr | a->o_addr) & 15u) != 0 || (a->dtype != VDT_F16 && a->dtype != VDT_BF16) ||
        a->nb_inner == 0 || a->nb % a->nb_inner != 0) {
      return static_cast<int>(hipErrorInvalidValue);
    }
    for (int i = 0; i < 4; ++i) {  // rows of at least d elements, every stride on 16 bytes (the kernel has 128-bit accesses only)
      if (a->row_stride[i] < a->d || a->row_stride[i] >= (1u << 22) || ((a->row_stride[i] | a->outer_stride[i] | a->inner_stride[i]) & 7u) != 0) {
        return static_cast<int>(hipErrorInvalidValue);
      }
    }
    // 256 lanes: four waves of 64 queries; 512 lanes: eight waves of 32 queries (same tile of 256 queries)
    const bool bf = a->dtype == VDT_BF16, narrow = a->d != DVM_ATTN_D;
    if (check_only) return 0;
    if (threads == 512) {
      hipLaunchKernelGGL(narrow ? (bf ? dvm_vm_attn_bf16_w8_d64 : dvm_vm_attn_f16_w8_d64) : (bf ? dvm_vm_attn_bf16_w8 : dvm_vm_attn_f16_w8),
                         dim3(block_dim), dim3(512), lds_bytes, s, p);
    } else {
      hipLaunchKernelGGL(narrow ? (bf ? dvm_vm_attn_bf16_d64 : dvm_vm_attn_f16_d64) : (bf ? dvm_vm_attn_bf16 : dvm_vm_attn_f16), dim3(block_dim),
                         dim3(256), lds_bytes, s, p);
    }
  } else {
    return static_cast<int>(hipErrorInvalidValue);
  }
  return static_cast<int>(hipGetLastError());
}

int dvm_hip_launch_vm(const void *param, uint32_t block_dim, uint32_t threads, uint32_t lds_bytes, void *stream) {
  if (param == nullptr) return static_cast<int>(hipErrorInvalidValue);
  VmParam p;
  memcpy(&p, param, sizeof(p));
  return launch_checked(p, block_dim, threads, lds_bytes, stream);
}

int dvm_hip_launch_vm_static_ws(const void *params, uint32_t n_programs, const uint32_t *geometry, const uint32_t *ws_words,
                                uint32_t n_ws, size_t ws_bytes, void *stream) {
  if (params == nullptr || geometry == nullptr || (n_ws > 0 && ws_words == nullptr)) return static_cast<int>(hipErrorInvalidValue);
  if (ws_bytes > DVM_HIP_STATIC_WS_BYTES) return DVM_HIP_ERROR_WS_TOO_LARGE;
  for (uint32_t i = 0; i < n_ws; ++i) {
    if (ws_words[2 * i] >= n_programs || ws_words[2 * i + 1] >= DVM_PARAM_WORDS) return DVM_HIP_ERROR_BAD_WS_WORD;
    const VmParam *src = static_cast<const VmParam *>(params) + ws_words[2 * i];
    if (src->w[ws_words[2 * i + 1]] >= ws_bytes) return DVM_HIP_ERROR_BAD_WS_WORD;
    // a word listed twice would get the workspace address added twice
    for (uint32_t j = 0; j < i; ++j)
      if (ws_words[2 * j] == ws_words[2 * i] && ws_words[2 * j + 1] == ws_words[2 * i + 1]) return DVM_HIP_ERROR_BAD_WS_WORD;
  }
  void *ws = nullptr;
  int rc = static_ws_address(&ws);
  if (rc != 0) return rc;
  // Two passes over the programs: every blob is checked against its geometry before the first one is launched.
  // A program with nothing to do has the geometry {0, 0, 0} (the exporter's convention) and is passed over.
  for (int pass = 0; pass < 2; ++pass) {
    for (uint32_t prog = 0; prog < n_programs; ++prog) {
      const uint32_t *g = geometry + 3 * prog;
      if (g[0] == 0 && g[1] == 0 && g[2] == 0) continue;
      VmParam p;  // the caller's blob stays as it is: the offsets become addresses in this copy
      memcpy(&p, static_cast<const VmParam *>(params) + prog, sizeof(p));
      for (uint32_t i = 0; i < n_ws; ++i) {
        if (ws_words[2 * i] == prog) p.w[ws_words[2 * i + 1]] += reinterpret_cast<uint64_t>(ws);
      }
      rc = launch_checked(p, g[0], g[1], g[2], stream, pass == 0);
      if (rc != 0) return rc;
    }
  }
  return 0;
}

int dvm_hip_fill_u32(void *dst, uint32_t value, size_t bytes, void *stream) {
  if (bytes == 0) return 0;
  if (dst == nullptr || (bytes & 3u) != 0) return static_cast<int>(hipErrorInvalidValue);
  const size_t n = bytes / 4;
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(dvm_fill_u32_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), static_cast<uint32_t *>(dst), value, n);
  return static_cast<int>(hipGetLastError());
}

int dvm_hip_get_device_count(uint32_t *count) {
  int n = 0;
  hipError_t err = hipGetDeviceCount(&n);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  if (count != nullptr) *count = static_cast<uint32_t>(n);
  return static_cast<int>(err);
}
int dvm_hip_set_device(int device_id) { return static_cast<int>(hipSetDevice(device_id)); }
int dvm_hip_get_device(int *device_id) { return static_cast<int>(hipGetDevice(device_id)); }
int dvm_hip_create_stream(void **stream) { return static_cast<int>(hipStreamCreate(reinterpret_cast<hipStream_t *>(stream))); }
int dvm_hip_destroy_stream(void *stream) { return static_cast<int>(hipStreamDestroy(reinterpret_cast<hipStream_t>(stream))); }
int dvm_hip_synchronize_stream(void *stream) {
  hipError_t err = hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream));
  if (err != hipSuccess) (void)hipGetLastError();  // do not leave the error for the next call
  return static_cast<int>(err);
}
int dvm_hip_malloc(void **ptr, size_t size) { return static_cast<int>(hipMalloc(ptr, size)); }
int dvm_hip_free(void *ptr) { return static_cast<int>(hipFree(ptr)); }
int dvm_hip_malloc_host(void **ptr, size_t size) { return static_cast<int>(hipHostMalloc(ptr, size, hipHostMallocDefault)); }
int dvm_hip_free_host(void *ptr) { return static_cast<int>(hipHostFree(ptr)); }
int dvm_hip_mem_to_dev(void *dst, const void *src, size_t count) {
  return static_cast<int>(hipMemcpy(dst, src, count, hipMemcpyHostToDevice));
}
int dvm_hip_mem_from_dev(void *dst, const void *src, size_t count) {
  return static_cast<int>(hipMemcpy(dst, src, count, hipMemcpyDeviceToHost));
}
int dvm_hip_mem_to_dev_async(void *dst, const void *src, size_t count, void *stream) {
  return static_cast<int>(hipMemcpyAsync(dst, src, count, hipMemcpyHostToDevice, reinterpret_cast<hipStream_t>(stream)));
}
int dvm_hip_memset(void *dst, int value, size_t size) { return static_cast<int>(hipMemset(dst, value, size)); }
int dvm_hip_create_event(void **event) { return static_cast<int>(hipEventCreate(reinterpret_cast<hipEvent_t *>(event))); }
int dvm_hip_destroy_event(void *event) { return static_cast<int>(hipEventDestroy(reinterpret_cast<hipEvent_t>(event))); }
int dvm_hip_record_event(void *event, void *stream) {
  return static_cast<int>(hipEventRecord(reinterpret_cast<hipEvent_t>(event), reinterpret_cast<hipStream_t>(stream)));
}
int dvm_hip_synchronize_event(void *event) { return static_cast<int>(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event))); }
int dvm_hip_event_elapsed_time(float *ms, void *start, void *end) {
  return static_cast<int>(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(end)));
}
const char *dvm_hip_error_string(int code) {
  if (code == DVM_HIP_ERROR_WS_TOO_LARGE) return "the programs need more workspace than the static workspace holds (DVM_HIP_STATIC_WS_BYTES)";
  if (code == DVM_HIP_ERROR_OTHER_DEVICE) return "dvm_hip_init_vm was called for another device before: one process drives one device";
  if (code == DVM_HIP_ERROR_BAD_WS_WORD) return "a workspace word names no program, no word of its blob, or an offset outside the workspace";
  return hipGetErrorString(static_cast<hipError_t>(code));
}

}  // extern "C"
