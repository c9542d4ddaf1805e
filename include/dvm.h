// Public C++ graph-building API of the DVM fused-operator JIT, gfx950 backend.
//
// This header is the drop-in boundary towards frameworks: it declares the same
// names, signatures, enum values and ownership rules as the reference's
// include/dvm.h (enums :27-117, Float16/BFloat16 :123-147, IntArrayRef :149-159,
// ScalarRef :161-199, RelocEntry :201-206, WsAllocator/CloneHelper :208-217,
// Kernel :236-722, Config :727-741, DvmException :752), so code written against
// that header compiles and links against this backend unchanged. Everything
// behind it (IR, passes, tile-bytecode emitter, device VM) is specific to
// MI355X.
//
// Ownership and lifetime rules kept from the reference:
//  * a Kernel owns every NDObject it returns;
//  * IntArrayRef* / ScalarRef* arguments are borrowed and re-read at every
//    Normalize()/CodeGen(), which is how dynamic shapes and scalars work;
//  * tensor addresses may be null at build time and supplied through
//    RelocEntry at CodeGen()/Launch();
//  * strings returned by Dump/DumpR/Das/Inspect belong to the Kernel and share
//    one buffer (the next call overwrites the previous result).
#ifndef _DVM_H_
#define _DVM_H_

#include <cstddef>
#include <cstdint>
#include <vector>

#define DVM_API __attribute__((visibility("default")))

namespace dvm {

enum DataType { kBool = 0, kFloat16, kBFloat16, kFloat32, kInt32, kInt64, kDataTypeEnd };

enum GatherMode { kElementGather = 0, kSliceGather = 1 };

enum UnaryType {
  kSqrt = 0, kAbs, kLog, kExp, kReciprocal, kIsFinite, kLogicalNot, kRound, kFloor, kCeil, kTrunc, kUnaryTypeEnd,
};

enum BinaryType {
  kEqual = 0, kNotEqual, kGreater, kGreaterEqual, kLess, kLessEqual,
  kAdd, kSub, kMul, kDiv, kPow, kMaximum, kMinimum, kLogicalAnd, kLogicalOr, kBinaryTypeEnd,
};

enum ReduceType { kSum = 0, kMax, kMin, kReduceTypeEnd };

enum GmmSplitType { kSplit_M = 0, kSplit_N, kSplit_K, kGroupTypeEnd };

enum GmmListType { kListBound = 0, kListSize, kEnd };

// What Kernel::Reset() builds.
enum KernelType {
  kVector = 0,  // element-wise / broadcast / reduce operators only
  kCube,        // one matmul
  kMix,         // one matmul plus vector operators fused behind it
  kParallel,    // several sub-kernels side by side
  kSequence,    // several sub-kernels one after another
  kSplit,       // the graph is cut into sub-kernels automatically
  kEager,       // operators are appended and run incrementally
  kKernelTypeEnd,
};

// Flag bits for Kernel::Reset().
enum KernelFlag {
  kDynamic = 0x1,      // shapes behind IntArrayRef may change between CodeGen calls
  kUnifyWS = 0x2,      // one workspace allocation for the whole kernel
  kSpeculate = 0x4,
  kLazyCodeGen = 0x8,
  kOptFractalTrans = 1u << 29,
  kPrivate1 = 1u << 30,
  kPrivate2 = 1u << 31,
};

class NDObject;
class VKernel;
class Communicator;

// IEEE binary16 value carried as its bit pattern.
class DVM_API Float16 {
 public:
  explicit Float16(uint16_t bits) : value_(bits) {}
  explicit Float16(float v);
  explicit Float16(int32_t v);
  explicit operator float() const;
  explicit operator int32_t() const;
  uint16_t int_value() const { return value_; }

 private:
  uint16_t value_;
};

// bfloat16 value carried as its bit pattern.
class DVM_API BFloat16 {
 public:
  explicit BFloat16(uint16_t bits) : value_(bits) {}
  explicit BFloat16(float v);
  explicit BFloat16(int32_t v);
  explicit operator float() const;
  explicit operator int32_t() const;
  uint16_t int_value() const { return value_; }

 private:
  uint16_t value_;
};

// Borrowed view of an int64 array (a shape, a stride list, a list of axes).
struct DVM_API IntArrayRef {
  IntArrayRef() {}
  explicit IntArrayRef(const std::vector<int64_t> &v) : data(v.data()), size(v.size()) {}
  IntArrayRef &operator=(const std::vector<int64_t> &v) {
    data = v.data();
    size = v.size();
    return *this;
  }
  const int64_t *data;
  size_t size;
};

// A scalar operand whose value is read again at every code generation.
struct DVM_API ScalarRef {
  ScalarRef() = default;
  template <typename T>
  ScalarRef(T v) {
    *this = v;
  }
  ScalarRef &operator=(float v) { type = kFloat32; f32 = v; return *this; }
  ScalarRef &operator=(int32_t v) { type = kInt32; i32 = v; return *this; }
  ScalarRef &operator=(Float16 v) { type = kFloat16; f16 = v.int_value(); return *this; }
  ScalarRef &operator=(BFloat16 v) { type = kBFloat16; f16 = v.int_value(); return *this; }
  ScalarRef &operator=(int64_t v) { type = kInt64; i64 = v; return *this; }
  DataType type;
  union {
    float f32;
    int32_t i32;
    uint16_t f16;
    int64_t i64;
  };
};

// Binds a load/store operation to a device address at code generation or launch.
struct DVM_API RelocEntry {
  RelocEntry() {}
  RelocEntry(NDObject *op, void *address) : io(op), addr(address) {}
  NDObject *io;
  void *addr;
};

// Callback that provides workspace (device) memory during CodeGen.
struct DVM_API WsAllocator {
  virtual void *Alloc(size_t size) = 0;
};

// Callback set used by Kernel::Clone to map the objects of the base kernel.
struct DVM_API CloneHelper {
  virtual IntArrayRef *GetClone(IntArrayRef *shape) = 0;
  virtual ScalarRef *GetClone(ScalarRef *scalar) = 0;
  virtual NDObject *GetClone(NDObject *op) = 0;
  virtual void SetClone(NDObject *op, NDObject *clone) = 0;
};

// Communicator handle for the in-kernel collectives. This backend drives one
// GPU: Init() succeeds only for a single rank and the collective operators
// are rejected when a graph is built.
class DVM_API Comm {
 public:
  enum { kMemory, kHccl, kDummy };
  Comm() = default;
  ~Comm();
  bool Init(int rank_id, int rank_size, int comm_type, const uint32_t *group_ranks = nullptr);
  bool Init(int rank_id, int rank_size) { return Init(rank_id, rank_size, kMemory); }
  void Init(void *hccl_comm);
  inline const Communicator *GetImpl() const { return comm_; }

 protected:
  Communicator *comm_{nullptr};
};

class DVM_API Kernel {
 public:
  Kernel();
  ~Kernel();
  // Copying moves the implementation: only one Kernel holds it afterwards.
  Kernel &operator=(Kernel &other);
  explicit Kernel(Kernel &other);

  // (Re)creates the kernel as `type` with KernelFlag bits `flags`.
  void Reset(KernelType type, uint32_t flags);
  // Rebuilds the graph of `base` (which must be constructed) with objects mapped by `helper`.
  void Clone(const Kernel &base, CloneHelper &helper);
  // Names used in dumps and profiles.
  void SetNameHint(const char *name, const char *fullname);

  // ---- tensor access ----
  NDObject *Load(void *addr, IntArrayRef *shape, DataType type);                         // contiguous input
  NDObject *GlobalAccess(void *addr, IntArrayRef *shape, DataType type);                 // handle only, no load
  NDObject *Load(void *addr, IntArrayRef *shape, IntArrayRef *stride, DataType type);    // strided input
  NDObject *GatherLoad(void *addr, IntArrayRef *shape, NDObject *index, int axis, DataType type,
                       GatherMode gather_mode = kElementGather);
  NDObject *SliceLoad(void *addr, IntArrayRef *shape, IntArrayRef *start, IntArrayRef *size, DataType type);
  NDObject *StridedSliceLoad(void *addr, IntArrayRef *shape, IntArrayRef *start, IntArrayRef *end, IntArrayRef *step,
                             DataType type);
  NDObject *MultiLoad(void *addr, IntArrayRef *shape, DataType type, const Comm *comm);
  NDObject *Store(void *addr, NDObject *input);                                          // contiguous output
  NDObject *Store(void *addr, NDObject *input, IntArrayRef *stride);                     // strided output
  NDObject *PadStore(void *addr, NDObject *input, int64_t pad_size);
  void SetStoreInplace(NDObject *store);  // the output aliases an input: never reuse it as workspace
  void SetStoreTemp(NDObject *store);
  void SetLoadBind(NDObject *load, NDObject *access);

  // ---- operators ----
  template <UnaryType op_type>
  NDObject *Unary(NDObject *input);
  // lhs / rhs: NDObject*, float, int32_t, Float16, BFloat16, ScalarRef*, or int64_t (compares only).
  template <BinaryType op_type, typename L, typename R>
  NDObject *Binary(L lhs, R rhs);
  template <ReduceType op_type>
  NDObject *Reduce(NDObject *input, IntArrayRef *dims, bool keepdims) {
    return _Reduce(op_type, input, dims, keepdims);
  }
  NDObject *Select(NDObject *cond, NDObject *lhs, NDObject *rhs);
  NDObject *Cast(NDObject *input, DataType type);
  NDObject *Broadcast(NDObject *input, IntArrayRef *shape);
  // val: float, int32_t, int64_t, Float16, BFloat16 or ScalarRef*.
  template <typename T>
  NDObject *Broadcast(T val, IntArrayRef *shape, DataType type);
  NDObject *Reshape(NDObject *input, IntArrayRef *shape);
  NDObject *Permute(NDObject *input, IntArrayRef *dims);
  NDObject *Slice(NDObject *input, IntArrayRef *start, IntArrayRef *size);
  NDObject *Slice(NDObject *input, int dim, ScalarRef *begin, ScalarRef *end);
  NDObject *Copy(NDObject *input);
  NDObject *Concat(NDObject **inputs, size_t input_num, int dim);
  NDObject **Split(NDObject *input, int dim, int64_t split_size, size_t split_num);
  template <typename T>
  NDObject *OneHot(NDObject *indices, IntArrayRef *depth, int axis, T on_value, T off_value);
  NDObject *ElemAny(NDObject *input);
  // fp16 / bf16 matmul with fp32 accumulation; bias may be null.
  NDObject *MatMul(NDObject *lhs, NDObject *rhs, bool trans_a, bool trans_b, NDObject *bias);
  NDObject *GroupedMatMul(NDObject *lhs, NDObject *rhs, bool trans_a, bool trans_b, NDObject *bias,
                          NDObject *group_list, GmmSplitType group_type, GmmListType group_list_type);
  template <ReduceType op_type>
  NDObject *AllReduce(NDObject *input, const Comm *comm) {
    return _AllReduce(op_type, input, comm);
  }
  NDObject *AllGather(NDObject *input, const Comm *comm);
  NDObject *AllGatherV2(NDObject *input, const Comm *comm);
  NDObject *ReduceScatter(NDObject *input, const Comm *comm);
  NDObject *ExtOut(NDObject *op, int index);

  // ---- kernel structure ----
  void SpecNext();
  void ParallelAdd(KernelType type, uint32_t flags, size_t thread_limit = 0);
  void SequenceAdd(KernelType type, uint32_t flags);

  // ---- compile and run ----
  void Normalize();  // re-infer every shape; call before CodeGen when an input shape changed
  void CodeGen(const RelocEntry *relocs, size_t reloc_size, WsAllocator *ws_alloc);
  int Launch(void *stream);  // 0 on success
  void Clear();
  size_t PreCodeGen();       // code generation before addresses are known; returns the workspace size
  int Launch(const RelocEntry *relocs, size_t reloc_size, void *workspace, void *stream);

  // ---- introspection ----
  static IntArrayRef *GetShape(NDObject *op);  // valid after Normalize / PreCodeGen
  static DataType GetDType(NDObject *op);
  const char *Dump() const;     // graph with compute shapes
  const char *DumpR() const;    // graph with reference (API) shapes
  const char *Das() const;      // disassembled bytecode; valid after CodeGen / PreCodeGen
  const char *Inspect() const;  // validation report
  VKernel *GetImpl() const { return kernel_; }

 protected:
  NDObject *_Reduce(int op_type, NDObject *input, IntArrayRef *dims, bool keepdims);
  NDObject *_AllReduce(int op_type, NDObject *input, const Comm *comm);
  NDObject *_Unary(int op_type, NDObject *input);
  template <typename L, typename R>
  NDObject *_Binary(int op_type, L lhs, R rhs);

  VKernel *kernel_;

 public:
  // Older spellings kept for source compatibility.
  NDObject *Unary(int op_type, NDObject *input) { return _Unary(op_type, input); }
  template <typename L, typename R>
  NDObject *Binary(int op_type, L lhs, R rhs) {
    return _Binary<L, R>(op_type, lhs, rhs);
  }
  NDObject *Reduce(int op_type, NDObject *input, IntArrayRef *dims, bool keepdims) {
    return _Reduce(op_type, input, dims, keepdims);
  }
  NDObject *AllReduce(int op_type, NDObject *input, const Comm *comm) { return _AllReduce(op_type, input, comm); }
  void ParallelNext() { return ParallelAdd(KernelType::kVector, 0); }
  void Infer() { Normalize(); }
  size_t CodeGen() { return PreCodeGen(); }
};

// Process-wide switches.
class DVM_API Config {
 public:
  Config() = default;
  ~Config() = default;
  static Config &Instance();
  bool IsInitialized() const;
  virtual Config &SetDeterm() = 0;
  virtual Config &UnsetDeterm() = 0;
  virtual Config &SetOnlineTuner() = 0;
  virtual Config &UnsetOnlineTuner() = 0;
  virtual Config &SetLazyTuner() = 0;
  virtual Config &UnsetLazyTuner() = 0;
  virtual Config &SetVfFusion(int mode = 1) = 0;
  virtual Config &UnsetVfFusion() = 0;
};

using DType = DataType;
using UnaryOpType = UnaryType;
using BinaryOpType = BinaryType;
using ReduceOpType = ReduceType;
using GroupType = GmmSplitType;
using GroupListType = GmmListType;
using ShapeRef = IntArrayRef;

// Every error is reported by throwing std::runtime_error("DVM EXCEPTION. reason: ...").
[[noreturn]] DVM_API void DvmException(const char *error_str);

}  // namespace dvm
#endif  // _DVM_H_
