// Host-side IR of the gfx950 backend: operator nodes, the kernel object behind
// dvm::Kernel, and the compiled sub-kernel programs.
//
// Role in the reference: NDObject hierarchy (src/ops.h:444-554), VKernel and
// its subclasses (src/kernel.h:52-104, src/xkernel.h), Code (src/code.h:90-286).
// Here one node class covers every operator kind and one kernel class covers
// the vector / split / mix kernel types; the graph is cut into sub-kernels by
// fusability on the gfx950 VM, not by the reference's local-memory tile model.
#ifndef DVM_AMD_HOST_IR_H_
#define DVM_AMD_HOST_IR_H_

#include <cstdint>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "../../../include/dvm.h"
#include "../isa_gfx950.h"

namespace dvm {

constexpr int kMaxRank = 10;  // same limit as the reference (src/ops.h:165)

enum ObjKind : uint8_t {
  kObjLoad = 0,
  kObjStore,
  kObjUnary,
  kObjBinary,
  kObjBinaryS,   // tensor (op) scalar
  kObjCompare,
  kObjCompareS,  // tensor (cmp) scalar
  kObjSelect,
  kObjCast,
  kObjBroadcast,
  kObjBroadcastS,  // scalar fill
  kObjReduce,
  kObjReshape,
  kObjCopy,
  kObjMatMul,
  kObjPermute,   // view: dims reordered (aux_ref = source dim of every result dim)
  kObjSlice,     // view: a box of the input (slice_start + aux_ref sizes, or one dim with begin / end)
  kObjConcatPart,  // writes its input into its place in the buffer of a Concat (a store through strides)
  kObjConcat,      // the buffer the parts wrote, read by the consumers like any value kept in memory
  // int64 tensors are pairs of int32 tensors (the reference's lowering, src/dvm.cc:478-760): the low and the high
  // words of every element. An int64 value the API hands out is a kObjPack64 (in[0] = low words, in[1] = high
  // words; a handle only, nothing computes it), or a Load of that type, whose words are read through two views:
  kObjPack64,
  kObjHalf64,      // view of an int64 Load: every second 32-bit word of its memory (op = 0 low words, 1 high words)
  // OneHot (src/ops.h:1333 of the reference): in[0] = int32 indices; the result has one more dim, of extent aux_ref[0],
  // at position slice_dim; scalar where the position along that dim equals the index, scalar2 elsewhere. The positions
  // are a memory operand without memory (VDT_IOTA) that walks the result's index space with the strides in vstride_.
  kObjOneHot,
  // GatherLoad (src/ops.h:632): the node is the source tensor (addr; full_shape_ref = its shape) read at positions an
  // int32 index tensor names along dim slice_dim. in[0] = the index values. op = 0: the index has the result's shape,
  // result[i..] = source[i.. with the index value in place of the coordinate along the dim] (NumPy take_along_axis);
  // op = 1: the index's dims replace the dim (NumPy take). vstride_ = the source's strides seen from the result's
  // index space, 0 along the gathered dims.
  kObjGather,
};

// A scalar operand: an immediate fixed at build time or a ScalarRef re-read at every code generation.
struct ScalarOperand {
  ScalarRef imm;
  ScalarRef *ref = nullptr;
  const ScalarRef &Get() const { return ref != nullptr ? *ref : imm; }
};

class NDObject {
 public:
  NDObject(ObjKind k, DataType t) : kind(k), type_id_(t) {
    own_ref_.data = shape_;
    own_ref_.size = 0;
    shape_ref_ = &own_ref_;
  }
  ObjKind kind;
  DataType type_id_;
  uint8_t op = 0;          // UnaryType / BinaryType / ReduceType
  bool scalar_left = false;  // kObjBinaryS / kObjCompareS: scalar is the left operand
  bool keepdims = false;
  bool trans_a = false, trans_b = false;
  bool inplace = false;
  bool temp = false;            // a Store marked by SetStoreTemp: no output of the kernel, only what bound loads read
  NDObject *bound = nullptr;    // a Load bound to a Store of the same kernel by SetLoadBind: it reads the stored value
  int part_split = 0;           // kObjReduce, during code generation only: the reduce is shared between workgroups, its result
                                // has one more (outermost) dim that numbers the parts (Compiler::SplitLongReduces)
  bool noloss_cast = false;
  uint8_t half64 = 0;           // kObjBroadcastS of an int64 scalar as int32 words: 1 = its low word, 2 = its high word
  NDObject *hi_view = nullptr;  // kObjStore of an int64 value (in[0] low, in[1] high words): where the high words go
                                // (owned; the Store itself says where the low words go)
  int nin = 0;
  NDObject *in[3] = {nullptr, nullptr, nullptr};
  ScalarOperand scalar;
  ScalarOperand scalar2;           // kObjOneHot: the value where the index does not match
  // kObjMatMul made by GroupedMatMul (src/ops_m.h:143-159 of the reference): 1 = the groups split the rows of the left
  // operand (right operand [groups, k, n], result [m, n]), 2 = they split the k axis (result [groups, m, n]);
  // group_list = the Load of the int64 (or int32) list of bounds (gmm_sizes: of sizes); a bias is [groups, n]
  uint8_t gmm_type = 0;
  bool gmm_sizes = false;
  NDObject *group_list = nullptr;
  bool elem_any = false;           // kObjReduce made by ElemAny: a reduce to one element, result of shape [1]
  int64_t pad_size = -1;           // kObjStore made by PadStore: rows of the buffer are this many elements longer than the value's
  int64_t gather_extent = 0, gather_stride = 0;  // kObjGather: extent and element stride of the gathered dim of the source
  // storage for a list of dims an operator made for itself (the reduce behind ElemAny): aux_ref points here then
  int64_t own_axes_[10] = {0};
  IntArrayRef own_axes_ref_;
  IntArrayRef *aux_ref = nullptr;  // reduce axes / broadcast target / reshape target / user shape of a load
  void *addr = nullptr;            // load / store address (may arrive later through a RelocEntry)
  // A load or store that walks its buffer with strides of its own (Kernel::Load / Store with a stride list,
  // SliceLoad, StridedSliceLoad; src/ops.h ViewLoad family): element strides per dim and the element offset of
  // the first element, refreshed from the references below at every Normalize().
  bool strided = false;
  int64_t vstride_[10] = {0};
  int64_t view_offset = 0;         // fixed part of the offset (set by the runner for views into a larger array)
  int64_t view_base_ = 0;          // view_offset plus what a slice's start adds
  IntArrayRef *stride_ref = nullptr;                 // explicit strides
  IntArrayRef *full_shape_ref = nullptr;             // slices: shape of the whole tensor
  IntArrayRef *slice_start = nullptr, *slice_end = nullptr, *slice_step = nullptr;  // end/step only for strided slices
  // kObjSlice along one dim (Slice(input, dim, begin, end) and the chunks of Split): bounds from the
  // references when set, else the fixed values; negative bounds count from the end, both are clipped
  NDObject *cat = nullptr;          // kObjConcatPart: the Concat it belongs to
  std::vector<NDObject *> parts;    // kObjConcat: its parts, in order along slice_dim
  int slice_dim = -1;
  ScalarRef *dim_begin_ref = nullptr, *dim_end_ref = nullptr;
  int64_t dim_begin = 0, dim_end = 0;
  int id = -1;                     // position in the kernel's operator list
  int stage = 0;                   // sub-kernel group opened by Kernel::ParallelAdd / SequenceAdd

  // Shape as the API sees it, outermost first. Loads point at the caller's
  // IntArrayRef (dynamic shapes), every other node at its own storage.
  IntArrayRef *shape_ref_;
  IntArrayRef own_ref_;
  int64_t shape_[kMaxRank];

  int rank() const { return static_cast<int>(shape_ref_->size); }
  int64_t dim(int i) const { return shape_ref_->data[i]; }
  int64_t numel() const {
    int64_t n = 1;
    for (size_t i = 0; i < shape_ref_->size; ++i) n *= shape_ref_->data[i];
    return n;
  }
  void SetShape(const int64_t *d, size_t n) {
    std::memcpy(shape_, d, sizeof(int64_t) * n);
    own_ref_.size = n;
  }
  bool IsLoad() const { return kind == kObjLoad; }
};

inline size_t DTypeSize(DataType t) {
  switch (t) {
    case kBool: return 1;
    case kFloat16:
    case kBFloat16: return 2;
    case kInt64: return 8;
    default: return 4;
  }
}

// One launch of the device VM.
struct Program {
  VmParam blob;
  uint32_t grid = 0;
  uint32_t threads = 0;
  uint32_t lds_bytes = 0;
  bool skip = false;       // nothing to do (an extent is zero)
  // addresses inside the blob that depend on relocation: (word offset, op) pairs
  struct Patch {
    uint32_t word;   // 64-bit word of the blob that receives the address
    int op_id;       // load/store node whose address goes there, or -1
    int ws_slot;     // or the workspace slot
    int64_t byte_offset = 0;  // added to the operator's address (strided views start inside their buffer)
    uint8_t role;    // kPatchVecMem: a VMemDesc (alignment flag follows the address); kPatchIota: a VMemDesc without
                     // memory, whose address word is its first value (byte_offset / 4); kPatchCubeOperand:
                     // a matmul operand (the fast path needs 16-byte alignment); kPatchPlain: nothing else;
                     // kPatchAligned16: an operand of the fused attention kernel, which only has 128-bit accesses
  };
  enum : uint8_t { kPatchVecMem = 0, kPatchCubeOperand = 1, kPatchPlain = 2, kPatchAligned16 = 3, kPatchIota = 4 };
  std::vector<Patch> patches;
  // What binding an unaligned address takes away from the blob (the alignment flag of a memory operand, the sweep
  // build of a vector program, the fast path of a matmul), as code generation left it: (32-bit word of the blob,
  // value) pairs that every bind writes back first, so that a later bind of aligned addresses gets the fast paths back.
  std::vector<std::pair<uint32_t, uint32_t>> bind_dependent;
  void RememberBindDependent() {
    bind_dependent.clear();
    const uint32_t *w32 = reinterpret_cast<const uint32_t *>(blob.w);
    auto keep = [&](size_t byte_offset) { bind_dependent.emplace_back(static_cast<uint32_t>(byte_offset / 4), w32[byte_offset / 4]); };
    const uint32_t entry = w32[0];
    if (entry == VE_VECTOR) {
      keep(offsetof(VVecHeader, sched));
      for (const Patch &pt : patches)
        if (pt.role == kPatchVecMem) keep(static_cast<size_t>(pt.word) * 8 + offsetof(VMemDesc, flags));
    } else if (entry == VE_CUBE) {
      keep(offsetof(VCubeHeader, fast));
    }
  }
  // pre-launch fills (zero-size reduce identities, clean kernels)
  struct Fill {
    int op_id;
    int ws_slot;
    uint32_t value;
    size_t bytes;
  };
  std::vector<Fill> fills;
};

// Host fp16 / bf16 codecs (same results as the reference's, src/dvm.cc:78-186).
uint16_t F32ToF16Bits(float f);
float F16BitsToF32(uint16_t h);
uint16_t F32ToBF16Bits(float f);
float BF16BitsToF32(uint16_t h);

// Value of a scalar operand as the 32-bit register pattern of a tensor of
// type `t`: the value is first converted to `t` exactly like the reference's
// EncodeScalar (src/dvm.cc:186-223), then widened to the VM's container
// (fp32 bits for bool/f16/bf16/f32 tensors, two's complement for int32).
uint32_t ScalarToContainer(const ScalarRef &s, DataType t, int half64 = 0);

struct DeviceApi;  // bound C ABI of libdvm_hip.so (system.cc)
class Compiler;    // compiler.h

// Tuning switches from the environment, read once when a kernel object is made (code generation runs in
// microseconds; a getenv per switch per compile is a measurable part of that). -1: not set.
struct Tuning {
  int vec_wide = -1;    // DVM_VEC_WIDE=1: four slabs per lane in the vector VM
  int vec_team = -1;    // DVM_VEC_TEAM=n: at most n lanes per output in reduces along the innermost axis
  int vec_runs = -1;    // DVM_VEC_RUNS=1: per-output runs only when the team is the whole workgroup
  int vec_pair = -1;   // DVM_VEC_PAIR=0: a load never takes the binary instruction behind it along
  int vec_fuse = -1;    // DVM_VEC_FUSE=0: the instruction stream stays as emitted (no fused sweep instructions)
  int vec_unirun = -1;  // DVM_VEC_UNIRUN=0: every wave executes the per-output runs
  int vec_reread = -1;  // DVM_VEC_REREAD=0: nothing parked, no reversed sweeps; 2: parked rounds only; 3: reversed sweeps only
  int vec_sweeps = -1;  // DVM_VEC_SWEEPS=0: never the sweep build of the vector VM
  int vec_gather_tile = -1;  // DVM_VEC_GATHER_TILE=0: pointwise programs with a gathered operand keep the plain slab order
  int cube_tile = -1;   // DVM_CUBE_TILE=256|128|64
  int cube_waves = -1;  // DVM_CUBE_WAVES=4|8
  int red_split_turn = -1;  // DVM_RED_SPLIT_TURN=0: the reduce over the parts of a shared reduce walks them outermost, as they lie in memory
  int red_split = -1;    // DVM_RED_SPLIT=0: never share a reduce between workgroups; N >= 2: N parts whenever the graph allows
  int cube_splitk = -1;  // DVM_CUBE_SPLITK=0: never split the k axis; N >= 2: split it N ways whenever the shape allows
  int cube_dump16 = -1; // DVM_CUBE_DUMP16=0: the matmul epilogue always reads the tile back as fp32, half a tile per pass
  int cube_fuse_act = -1;  // DVM_CUBE_FUSE_ACT=0: x / (exp(x * c) + 1) and 1 / (exp(x * c) + 1) of a matmul epilogue stay separate instructions
  int cube_exact = -1;  // DVM_CUBE_EXACT=1: never the hardware approximations of exp, log, sqrt, division in a matmul epilogue
  int attn_waves = -1;  // DVM_ATTN_WAVES=4
  bool debug = false;   // DVM_DEBUG: node dump in compile errors
  bool in_tuner = false;  // the kernel is a candidate the online tuner is timing: it is not tuned itself
  void Read();
};

class VKernel {
 public:
  VKernel(KernelType t, uint32_t f) : ktype_(t), flags_(f) { tuning_.Read(); }
  ~VKernel();
  Tuning tuning_;

  KernelType KType() const { return ktype_; }
  uint32_t Flags() const { return flags_; }
  bool IsDynamic() const { return (flags_ & kDynamic) != 0; }

  NDObject *Append(NDObject *op);
  // Opens the next group of a parallel / sequence kernel: operators appended from now on never share
  // a launch with earlier ones (src/xkernel.h: SeqKernel / ParallelKernel stages).
  void NextStage() { ++cur_stage_; }
  int Stage() const { return cur_stage_; }
  void SetStage(int s) { cur_stage_ = s; }
  void Normalize();
  // Compiles every sub-kernel. With `pre` set no addresses are needed yet; returns the workspace size.
  size_t CodeGen(bool pre);
  void BindAddresses(const RelocEntry *relocs, size_t n, WsAllocator *alloc, void *workspace);
  int Launch(void *stream);

  std::string &DumpGraph(bool ref_shapes);
  std::string &DisAssemble();
  std::string &Inspect();

  std::vector<NDObject *> ops_;
  // arrays handed to the caller (the chunks of a Split); they live as long as the kernel's operators
  NDObject **NewObjectArray(size_t n) {
    obj_arrays_.emplace_back(n, nullptr);
    return obj_arrays_.back().data();
  }
  std::vector<std::vector<NDObject *>> obj_arrays_;
  std::vector<Program> programs_;
  size_t ws_bytes_ = 0;
  std::vector<size_t> ws_offsets_;  // per workspace slot
  std::vector<size_t> ws_sizes_;
  void *ws_base_ = nullptr;
  std::string name_, fullname_;
  int part_mode_ = 0;             // partition mode that compiled last time (see Compiler::Run)
  int ops_limit_ = 0;             // ... and, when that took fewer operators per sub-kernel or pointwise workgroups of
  uint32_t pw_cap_ = 0;           // fewer lanes than the defaults, those (0: the defaults)
  double last_codegen_us_ = 0.0;  // wall time of the last Normalize+CodeGen, for JIT latency reports

 private:
  KernelType ktype_;
  uint32_t flags_;
  bool normalized_ = false;
  bool compiled_ = false;
  int cur_stage_ = 0;
  Compiler *compiler_ = nullptr;  // kept between code generations of a dynamic kernel: its tables keep their storage
  std::string dump_str_;
  friend class Compiler;
};

[[noreturn]] void Throw(const std::string &msg);

}  // namespace dvm

#endif  // DVM_AMD_HOST_IR_H_
