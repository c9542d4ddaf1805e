/* C ABI of the gfx950 device layer (libdvm_hip.so).
 *
 * These are the entry points the reference's host code binds for its device
 * backend: the three device-VM functions of src/vm_gpu.h:153-155 and the
 * runtime wrappers of src/runtime.h:34-84. Plain C types only, so the host
 * emitter (or any other caller) needs no HIP headers. Every function returns
 * 0 on success or the HIP error code, unless stated otherwise. No function
 * throws.
 */
#ifndef DVM_HIP_H_
#define DVM_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Limits of the device the VM was initialised on.
 * Replaces dvm::gpu::SysConfig (src/vm_gpu.h:147-151). */
typedef struct {
  uint64_t core_num;        /* compute units */
  uint64_t local_mem_size;  /* LDS bytes one workgroup may use */
  uint64_t default_threads; /* default workgroup size */
  uint64_t wave_size;       /* 64 on gfx950 */
  uint64_t l2_bytes;        /* L2 size per XCD */
  uint64_t xcd_num;         /* accelerator dies (L2 domains) */
} dvm_hip_sysconfig;

/* Queries device `dev_id`, loads the VM kernels and fills `conf`.
 * The limits it finds are one set per process: a later call has to name the same device, another one gets
 * DVM_HIP_ERROR_OTHER_DEVICE (one process drives one GPU, as the reference's runtime does after SetDevice).
 * Replaces dvm::gpu::InitVM (src/vm_gpu.h:153). */
#define DVM_HIP_ERROR_OTHER_DEVICE (-4)
int dvm_hip_init_vm(int dev_id, dvm_hip_sysconfig *conf);

/* Launch geometry for a program of interpreter kind `kind` (the schedule id
 * of a vector program, or 16 + entry type for the matmul kernels) over
 * `item_num` work items, each workgroup having `threads` lanes and
 * `lds_bytes` of local memory: returns (workgroups << 32) | threads, the
 * number of workgroups that are resident at once, capped by `item_num`.
 * Replaces dvm::gpu::SelectBlockThread (src/vm_gpu.h:154). */
uint64_t dvm_hip_select_block_thread(uint64_t kind, uint64_t item_num, uint64_t threads, uint32_t lds_bytes);

/* Launches the device VM on one 4096-byte program blob (`param` is host
 * memory, copied into the kernel arguments). The entry type in the blob's
 * first word selects the interpreter kernel.
 * Replaces dvm::gpu::LaunchVM (src/vm_gpu.h:155). */
int dvm_hip_launch_vm(const void *param, uint32_t block_dim, uint32_t threads, uint32_t lds_bytes, void *stream);

/* Launches `n_programs` program blobs in order on `stream`, with the workspace they share (the values one launch
 * hands to a later one) placed in a workspace the library owns, and allocates nothing: no hipMalloc, no hipFree,
 * no allocating library routine. It has no counterpart in the reference; it is for callers that cannot allocate
 * device memory where they launch: code under HIP graph capture, tight serving loops, harnesses that forbid it.
 * The existing route is dvm_hip_launch_vm once per blob with workspace addresses the caller allocated.
 *   params     n_programs consecutive blobs of 4096 bytes (host memory), each as dvm_hip_launch_vm takes it,
 *              input and output addresses filled in by the caller;
 *   geometry   n_programs triples {workgroups, threads, lds_bytes};
 *   ws_words   n_ws pairs {program index, index of a 64-bit word of that blob}: the word holds a byte offset into
 *              the workspace instead of an address (a multiple of 16 for the matmul and attention operands);
 *   ws_bytes   size of the workspace the offsets were planned for.
 * The workspace is one array of DVM_HIP_STATIC_WS_BYTES bytes per device, 256-byte aligned, that lives in the
 * library's device code from load to process exit. A larger ws_bytes, or an offset outside ws_bytes, is refused
 * with DVM_HIP_ERROR_WS_TOO_LARGE / DVM_HIP_ERROR_BAD_WS_WORD before anything is launched. Nothing in it has to
 * start at zero: a launch writes all of a value before a later launch reads it. Every call on a device uses that
 * device's one array, which keeps what the last call left there: two calls that overlap on one device (different
 * streams, or two threads) race on it; calls on one stream are ordered and safe. */
#define DVM_HIP_STATIC_WS_BYTES (32u * 1024u * 1024u)
#define DVM_HIP_ERROR_WS_TOO_LARGE (-2)
#define DVM_HIP_ERROR_BAD_WS_WORD (-3)
int dvm_hip_launch_vm_static_ws(const void *params, uint32_t n_programs, const uint32_t *geometry, const uint32_t *ws_words,
                                uint32_t n_ws, size_t ws_bytes, void *stream);

/* Fills `bytes` bytes at device address `dst` with the 32-bit pattern `value`
 * on `stream` using a fill kernel (safe under graph capture, unlike a memset
 * node). Used where the reference launches its clean kernels
 * (src/ops.cc:551-606, src/kernel.cc:23-75). `bytes` must be a multiple of 4. */
int dvm_hip_fill_u32(void *dst, uint32_t value, size_t bytes, void *stream);

/* Runtime wrappers: the dvm::rt functions of src/runtime.h:34-84. */
int dvm_hip_get_device_count(uint32_t *count);
int dvm_hip_set_device(int device_id);
int dvm_hip_get_device(int *device_id);
int dvm_hip_create_stream(void **stream);
int dvm_hip_destroy_stream(void *stream);
int dvm_hip_synchronize_stream(void *stream);
int dvm_hip_malloc(void **ptr, size_t size);
int dvm_hip_free(void *ptr);
int dvm_hip_malloc_host(void **ptr, size_t size);
int dvm_hip_free_host(void *ptr);
int dvm_hip_mem_to_dev(void *dst, const void *src, size_t count);
int dvm_hip_mem_from_dev(void *dst, const void *src, size_t count);
int dvm_hip_mem_to_dev_async(void *dst, const void *src, size_t count, void *stream);
int dvm_hip_memset(void *dst, int value, size_t size);
int dvm_hip_create_event(void **event);
int dvm_hip_destroy_event(void *event);
int dvm_hip_record_event(void *event, void *stream);
int dvm_hip_synchronize_event(void *event);
int dvm_hip_event_elapsed_time(float *ms, void *start, void *end);

/* Text for an error code returned by any function above (static storage). */
const char *dvm_hip_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* DVM_HIP_H_ */
