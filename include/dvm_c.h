/* Flat C ABI over dvm::Kernel plus a small runner (device buffers, launch,
 * timing), bound by the Python package with ctypes.
 *
 * It stands where the reference's pybind module stands: the `Kernel` builder
 * methods of include/dvm_py.h:277-388 and the `PyKernel` runner of
 * src/pybind_api.cc:410-907 (input / codegen / run / output / perf / das).
 * Handles are opaque pointers owned by the runner they came from. Functions
 * that return a pointer return NULL on error, the others a non-zero code;
 * dvm_c_last_error() then holds the message (per thread).
 */
#ifndef DVM_C_H_
#define DVM_C_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

typedef struct dvm_rt dvm_rt;          /* a kernel plus its runner                        */
typedef struct dvm_obj dvm_obj;        /* an operator node (dvm::NDObject)                */
typedef struct dvm_shape dvm_shape;    /* an updatable shape (dvm::IntArrayRef + storage) */
typedef struct dvm_scalar dvm_scalar;  /* an updatable scalar (dvm::ScalarRef)            */

/* One operand of a binary operator. kind: 0 tensor (obj), 1 float immediate (f),
 * 2 int32 immediate (i), 3 scalar reference (ref). */
typedef struct {
  int kind;
  dvm_obj *obj;
  dvm_scalar *ref;
  double f;
  int64_t i;
} dvm_operand;

const char *dvm_c_last_error(void);

/* ker_type: "vector", "split", "mix", "cube" optionally followed by ":dyn" (src/pybind_api.cc:117-154).
 * run_mode: "dev" (needs a GPU) or "das" (code generation and disassembly only, fake addresses). */
dvm_rt *dvm_rt_new(const char *ker_type, const char *run_mode, int dev_id);
void dvm_rt_delete(dvm_rt *rt);
int dvm_rt_reset(dvm_rt *rt);

dvm_shape *dvm_rt_new_shape(dvm_rt *rt, const int64_t *dims, size_t n);
int dvm_shape_update(dvm_shape *s, const int64_t *dims, size_t n);
dvm_scalar *dvm_rt_new_scalar(dvm_rt *rt, int dtype);
int dvm_scalar_update_f(dvm_scalar *s, double v);
int dvm_scalar_update_i(dvm_scalar *s, int64_t v);

dvm_obj *dvm_rt_load(dvm_rt *rt, dvm_shape *shape, int dtype);
dvm_obj *dvm_rt_store(dvm_rt *rt, dvm_obj *x);
dvm_obj *dvm_rt_unary(dvm_rt *rt, int unary_type, dvm_obj *x);
dvm_obj *dvm_rt_binary(dvm_rt *rt, int binary_type, const dvm_operand *lhs, const dvm_operand *rhs);
dvm_obj *dvm_rt_select(dvm_rt *rt, dvm_obj *cond, dvm_obj *lhs, dvm_obj *rhs);
dvm_obj *dvm_rt_cast(dvm_rt *rt, dvm_obj *x, int dtype);
dvm_obj *dvm_rt_broadcast(dvm_rt *rt, dvm_obj *x, dvm_shape *shape);
dvm_obj *dvm_rt_full(dvm_rt *rt, const dvm_operand *value, dvm_shape *shape, int dtype);
dvm_obj *dvm_rt_reshape(dvm_rt *rt, dvm_obj *x, dvm_shape *shape);
dvm_obj *dvm_rt_reduce(dvm_rt *rt, int reduce_type, dvm_obj *x, dvm_shape *dims, int keepdims);
dvm_obj *dvm_rt_copy(dvm_rt *rt, dvm_obj *x);
dvm_obj *dvm_rt_matmul(dvm_rt *rt, dvm_obj *lhs, dvm_obj *rhs, int trans_a, int trans_b, dvm_obj *bias);
// Kernel::GlobalAccess / GatherLoad / PadStore / OneHot / ElemAny (include/dvm.h:284, 297-307, 344, 482-496 of the
// reference; KernelPy global_access / gather_load / pad_store / one_hot / element_any, include/dvm_py.h:302-327).
// global_access names an int32 index tensor (bound like a load); gather_load reads the tensor bound to the returned
// handle (like a load's input) at those indices along `axis` (gather_mode 0: NumPy take_along_axis, 1: NumPy take);
// pad_store writes into a buffer whose innermost rows are pad_size elements longer than the value's (the output is
// that larger buffer); one_hot's depth is a one-element shape; element_any gives one fp32 value, the maximum of x.
dvm_obj *dvm_rt_global_access(dvm_rt *rt, dvm_shape *shape, int dtype);
dvm_obj *dvm_rt_gather_load(dvm_rt *rt, dvm_shape *shape, dvm_obj *index, int dtype, int axis, int gather_mode);
dvm_obj *dvm_rt_pad_store(dvm_rt *rt, dvm_obj *x, long long pad_size);
dvm_obj *dvm_rt_one_hot(dvm_rt *rt, dvm_obj *indices, dvm_shape *depth, int axis, double on_value, double off_value, int dtype);
dvm_obj *dvm_rt_element_any(dvm_rt *rt, dvm_obj *x);
// Kernel::GroupedMatMul (include/dvm.h:510-522 of the reference; KernelPy grouped_matmul, include/dvm_py.h:198-205):
// group_type 0: the groups are ranges of lhs's rows, rhs is [groups, k, n] ([groups, n, k] transposed), the result
// [m, n]; group_type 2: ranges of the k axis, the result [groups, m, n]. group_list is a load of int64 (or int32)
// values, one per group, read on the device at every launch: the ranges' upper bounds (group_list_type 0, ascending)
// or their sizes (1). bias (may be null) is [groups, n]. Rows past the last bound are not written.
dvm_obj *dvm_rt_grouped_matmul(dvm_rt *rt, dvm_obj *lhs, dvm_obj *rhs, int trans_a, int trans_b, dvm_obj *bias, dvm_obj *group_list,
                               int group_type, int group_list_type);
int dvm_rt_set_store_inplace(dvm_rt *rt, dvm_obj *store);
// Kernel::SetStoreTemp / SetLoadBind / SpecNext (include/dvm.h:352-353, 544 of the reference; KernelPy set_store_temp /
// set_load_bind, include/dvm_py.h:207-208, RtKernelPy spec_next): a Store that is no output of the kernel, a Load that
// reads what a Store of the same kernel writes (bind before the Load's first use), the stage marker of a kernel
// created as "vector:spec".
int dvm_rt_set_store_temp(dvm_rt *rt, dvm_obj *store);
int dvm_rt_set_load_bind(dvm_rt *rt, dvm_obj *load, dvm_obj *store);
int dvm_rt_spec_next(dvm_rt *rt);
// Strided views (Kernel::Load / Store with a stride list, SliceLoad, StridedSliceLoad: include/dvm.h:195-201, 214 of the
// reference; KernelPy view_load / slice_load / stridedslice_load, include/dvm_py.h). Strides are in elements, the
// innermost one may be anything (0 broadcasts, 1 is the fast path, others go element by element). A view store writes into a zero-initialised buffer of extent_elems elements;
// dvm_obj_set_view_offset moves the first element of a view that many elements into its buffer.
dvm_obj *dvm_rt_view_load(dvm_rt *rt, dvm_shape *shape, dvm_shape *stride, int dtype);
dvm_obj *dvm_rt_slice_load(dvm_rt *rt, dvm_shape *shape, dvm_shape *start, dvm_shape *size, int dtype);
dvm_obj *dvm_rt_stridedslice_load(dvm_rt *rt, dvm_shape *shape, dvm_shape *start, dvm_shape *end, dvm_shape *step, int dtype);
dvm_obj *dvm_rt_view_store(dvm_rt *rt, dvm_obj *x, dvm_shape *stride, size_t extent_elems);
int dvm_obj_set_view_offset(dvm_obj *io, long long elems);
// Views of values (Kernel::Permute / Slice / Split, include/dvm.h:434,443,453,479 of the reference; KernelPy permute /
// slice / slice_dim / split, include/dvm_py.h:347-358): dims[i] names the input dim that becomes result dim i; a slice
// keeps `size` elements from `start` in every dim, or [begin, end) of one dim (negative bounds count from the end,
// both are clipped; the scalars are re-read at every code generation); split writes `num` handles to `out`, chunks
// of `chunk` along `dim`, the last one possibly smaller.
dvm_obj *dvm_rt_permute(dvm_rt *rt, dvm_obj *x, dvm_shape *dims);
dvm_obj *dvm_rt_slice(dvm_rt *rt, dvm_obj *x, dvm_shape *start, dvm_shape *size);
dvm_obj *dvm_rt_slice_dim(dvm_rt *rt, dvm_obj *x, int dim, dvm_scalar *begin, dvm_scalar *end);
int dvm_rt_split(dvm_rt *rt, dvm_obj *x, int dim, long long chunk, size_t num, dvm_obj **out);
// Kernel::Concat (include/dvm.h:470 of the reference; KernelPy concat, include/dvm_py.h:173-181): the n inputs joined along `dim`.
dvm_obj *dvm_rt_concat(dvm_rt *rt, dvm_obj **inputs, size_t n, int dim);
// Group markers of "seq" and "parallel" kernels (KernelPy::SequenceAdd / ParallelAdd, include/dvm_py.h:369-371; Kernel::SequenceAdd /
// ParallelAdd, include/dvm.h:250-251): operators built after the call belong to the next sub-kernel group.
int dvm_rt_seq_add(dvm_rt *rt, int ktype, unsigned flags);
// RtKernelPy::Clone (src/pybind_api.cc:923-993; Kernel::Clone, include/dvm.h:188): `rt` becomes a copy of `base`'s
// graph with shapes, axis lists and scalars of its own. items[i] (kinds[i]: 0 dvm_obj*, 1 dvm_shape*, 2 dvm_scalar*)
// are handles of `base`; out[i] receives the corresponding handle of `rt`.
int dvm_rt_clone(dvm_rt *rt, dvm_rt *base, const int *kinds, void *const *items, size_t n, void **out);
int dvm_rt_parallel_add(dvm_rt *rt, int ktype, unsigned flags, size_t core_limit);

int dvm_obj_rank(const dvm_obj *o);
int dvm_obj_shape(const dvm_obj *o, int64_t *dims, size_t cap);
int dvm_obj_dtype(const dvm_obj *o);

/* Copies `bytes` of host data into a device buffer owned by the runner and binds it to the load. */
int dvm_rt_input(dvm_rt *rt, dvm_obj *load, const void *host, size_t bytes);
/* Binds a caller-owned device buffer to a load or store (no copy, no ownership). */
int dvm_rt_bind_device(dvm_rt *rt, dvm_obj *io, void *device_ptr);
/* Binds a caller-owned device buffer to a load that reads it through element strides (a tensor that is not
 * contiguous: a transposed or sliced view), `strides[rank]` against the load's shape; NULL makes the load dense
 * again. The reference takes such tensors through Load with a stride list (include/dvm.h:294); its torch adapter
 * passes a tensor's strides the same way (docs/pytorch.md:209-262). */
int dvm_rt_bind_device_view(dvm_rt *rt, dvm_obj *load, void *device_ptr, const int64_t *strides, size_t rank);
/* The workspace of the kernel's launches comes from `alloc(bytes, user)` (device memory that stays valid until the
 * launches of the next dvm_rt_run have finished) instead of the runner's own allocation: the counterpart of the
 * WsAllocator argument of Kernel::CodeGen (include/dvm.h:208-210), so that a framework's caching allocator can
 * own it. NULL restores the runner's allocation. */
typedef void *(*dvm_ws_alloc_fn)(size_t bytes, void *user);
int dvm_rt_set_workspace_allocator(dvm_rt *rt, dvm_ws_alloc_fn alloc, void *user);
/* Forgets every binding made by dvm_rt_bind_device (the memory stays the caller's); loads and stores get
 * buffers of the runner again at the next dvm_rt_input / dvm_rt_codegen. */
int dvm_rt_unbind_device(dvm_rt *rt);
/* Normalize + allocate unbound outputs + CodeGen with relocations. */
// Shape inference only (what dvm_rt_codegen does first): afterwards dvm_obj_shape of a store is what the bound
// inputs imply, so a caller can allocate its own output memory and bind it before code generation.
int dvm_rt_normalize(dvm_rt *rt);
int dvm_rt_codegen(dvm_rt *rt);
/* Host wall time of the last Normalize + CodeGen in microseconds. */
double dvm_rt_jit_us(const dvm_rt *rt);
/* Launch and, with DVM_RUN_WAIT, wait for the stream. The stream is `stream` when that is not NULL or when
 * DVM_RUN_ON_GIVEN_STREAM is set (then NULL names the device's default stream), else the runner's own. */
#define DVM_RUN_WAIT 1
#define DVM_RUN_ON_GIVEN_STREAM 2
int dvm_rt_run(dvm_rt *rt, void *stream, int flags);
int dvm_rt_output(dvm_rt *rt, dvm_obj *store, void *host, size_t bytes);
void *dvm_rt_device_ptr(dvm_rt *rt, dvm_obj *io);
/* warmup + iters timed launches with events: out = {min, max, mean} microseconds (src/pybind_api.cc:751-767). */
int dvm_rt_perf(dvm_rt *rt, int warmup, int iters, double out[3]);
/* The same measurement, every launch's microseconds written to samples[0..iters) (for medians). */
int dvm_rt_perf_samples(dvm_rt *rt, int warmup, int iters, double *samples);
/* The matmul tuner (Config::SetOnlineTuner / SetLazyTuner of include/dvm.h; the reference's table of tuned tile
 * parameters, src/ops_m.h:174-263): with either switched on, the first code generation of a product shape on a
 * machine with a device times every (block tile, parts of the k axis) candidate there and remembers the fastest for
 * the process. dvm_tuner_stats: shapes measured so far and entries of the table; dvm_tuner_clear empties the table. */
void dvm_set_online_tuner(int enable);
void dvm_set_lazy_tuner(int enable);
void dvm_tuner_stats(uint64_t *shapes_measured, uint64_t *table_size);
void dvm_tuner_clear(void);
/* Number of device launches one run() issues. */
int dvm_rt_num_launches(const dvm_rt *rt);
size_t dvm_rt_workspace_bytes(const dvm_rt *rt);

/* The compiled launches of the kernel, for a caller that drives the device layer (include/dvm_hip.h) itself:
 * after dvm_rt_codegen, launch i of dvm_rt_program_count() is copied out as its 4096-byte blob with the bound
 * input / output addresses in place, its geometry {workgroups, threads, lds_bytes} (all zero for a launch that
 * has nothing to do) and the indices of the blob's 64-bit words that address the kernel's workspace. Those words
 * hold byte offsets into the workspace (of dvm_rt_workspace_bytes() bytes) instead of addresses, which is the
 * form dvm_hip_launch_vm_static_ws takes; adding a workspace address to each gives what dvm_hip_launch_vm
 * takes. Returns the number of workspace words (at most `cap` are written), or -1. Kernels whose launches need a
 * buffer cleared first (an output of a reduce over no elements) are refused. */
int dvm_rt_program_count(const dvm_rt *rt);
int dvm_rt_program(dvm_rt *rt, int i, void *blob, uint32_t geometry[3], uint32_t *ws_words, size_t cap);

const char *dvm_rt_das(dvm_rt *rt);
const char *dvm_rt_dump(dvm_rt *rt);
const char *dvm_rt_dump_r(dvm_rt *rt);
const char *dvm_rt_inspect(dvm_rt *rt);

/* Host codecs used for bf16 numpy round trips (src/pybind_api.cc:584-609). */
void dvm_c_f32_to_bf16(const float *src, uint16_t *dst, size_t n);
void dvm_c_bf16_to_f32(const uint16_t *src, float *dst, size_t n);

int dvm_c_has_device(void);
int dvm_c_core_num(void);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* DVM_C_H_ */
