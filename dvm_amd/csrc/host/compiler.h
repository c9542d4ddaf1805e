// The gfx950 code generator behind VKernel::CodeGen: one Compiler object turns the operator list of a kernel into
// launches of the device VM. Its steps live in separate translation units:
//   partition.cc    which operators share a launch, which values cross launches (workspace), attention detection
//   schedule.cc     nodes of one sub-kernel, unification of tensor dims into domain axes, order / merge, schedule
//   emit_vector.cc  accumulator-machine code for vector sub-kernels, registers, memory operand descriptors
//   peephole.cc     passes over the emitted instruction words
//   emit_cube.cc    matmul sub-kernels: tile choice, operand descriptors, epilogue program
//   emit_attn.cc    the fused attention launch
//   kernel.cc       VKernel::CodeGen / BindAddresses / Launch and the partition-mode loop
// Role in the reference: the split kernel's graph cutter (src/xkernel.cc:1980-2119), domain / tiling
// (src/kernel.cc:765-1194), liveness + buffer allocation (src/kernel.cc:196-317, 1285-1332) and the Emit methods
// (src/ops.cc). The gfx950 target differs in what a sub-kernel may contain: a reduce and its consumers stay in one
// launch (consecutive sweeps of one workgroup-resident program), broadcasts are stride-0 operands, and intermediate
// values live in lane registers, so the "tiling" step is an index-space analysis instead of a local-memory planner:
//   1. every tensor dim of every value is unified into domain axes;
//   2. axes are ordered, merged where all memory operands allow it, and split into a kept list and a reduced list;
//   3. a schedule (pointwise / reduce over the innermost axis / reduce with the innermost axis kept) and its launch
//      geometry are chosen;
//   4. the operator DAG is linearised into accumulator-machine code, section by section (code outside sweeps works
//      on the kept space, a sweep walks the reduce space), values that cannot stay in a register across a sweep are
//      recomputed from their loads.
#ifndef DVM_AMD_HOST_COMPILER_H_
#define DVM_AMD_HOST_COMPILER_H_

#include <cstdint>
#include <string>
#include <vector>

#include "ir.h"
#include "system.h"

namespace dvm {

constexpr int kMaxNodes = 160;     // nodes of one sub-kernel
constexpr int kMaxAreaOps = 100;   // operators the partitioner puts into one sub-kernel
constexpr int kMaxAxes = 24;       // domain axes before merging
constexpr int E = DVM_VEC_E;

enum AKind : uint8_t { AK_MEM, AK_SCALAR, AK_OP, AK_ALIAS, AK_REDUCE, AK_OUT };

struct ANode {
  AKind kind;
  NDObject *op;         // originating operator (for AK_MEM of a cross-kernel value: the producer or the reshape view)
  DataType dtype;
  int nin;
  int in[3];
  int rank;
  const int64_t *dims;  // API shape, outermost first
  int axis[kMaxRank];   // domain axis per dim, -1 for extent 1
  // memory leaves / outputs
  int addr_op;          // load/store operator supplying the address, or -1
  int ws_slot;          // workspace slot, or -1
  int mem_idx;          // descriptor index in the program
  const NDObject *view; // load / store that walks its buffer with strides of its own, or nullptr (dense)
  // emission state
  bool has_inner;       // varies along the innermost domain axis
  bool fd;              // has a reduced axis
  int level;
  int sec;              // section the value is computed in
  int uses;             // remaining uses in the section being emitted
  int reg;              // S register (has_inner false) or V slot, -1 when not in a register
  uint8_t reg_fmt;
  bool in_cone;
  int last_sec;         // last section with a consumer
  int slot;             // AK_REDUCE: reduce slot of its sweep
  bool slot_ready;      // AK_REDUCE: the combined result sits in its slot (from the end of its sweep to the next sweep)
};

struct Axis {
  int64_t extent;
  bool reduced;
  uint32_t before;  // axes that must be outside (more significant than) this one
};

struct Dim {  // merged domain dim
  int64_t extent;
  bool reduced;
  int first_axis, last_axis;  // merged range in ordered-axis space (outer .. inner)
};

inline uint32_t FloatBits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

inline VDim MakeVDim(uint32_t d) {
  VDim v;
  v.extent = d;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  v.shift = s;
  v.magic = static_cast<uint32_t>((((1ull << 32) * ((1ull << s) - d)) / (d == 0 ? 1 : d)) + 1);
  v.pad = 0;
  return v;
}

inline uint32_t MemDType(DataType t) {
  switch (t) {
    case kBool: return VDT_BOOL;
    case kFloat16: return VDT_F16;
    case kBFloat16: return VDT_BF16;
    case kFloat32: return VDT_F32;
    case kInt32: return VDT_I32;
    default: Throw("tensor type without a device form");
  }
}

inline uint32_t RndOf(DataType t) { return t == kFloat16 ? VRND_F16 : (t == kBFloat16 ? VRND_BF16 : VRND_NONE); }

inline bool IsPointwiseKind(ObjKind k) {
  switch (k) {
    case kObjUnary:
    case kObjBinary:
    case kObjBinaryS:
    case kObjCompare:
    case kObjCompareS:
    case kObjSelect:
    case kObjCast:
    case kObjCopy:
    case kObjBroadcast:
    case kObjStore:
    case kObjConcatPart:
      return true;
    default:
      return false;
  }
}

// A reshape that only inserts or removes extent-1 dims keeps every element's coordinates.
inline bool IsSqueezeReshape(const NDObject *o) {
  const NDObject *x = o->in[0];
  int i = 0, j = 0;
  const int ri = x->rank(), ro = o->rank();
  while (true) {
    while (i < ri && x->dim(i) == 1) ++i;
    while (j < ro && o->dim(j) == 1) ++j;
    if (i == ri || j == ro) break;
    if (x->dim(i) != o->dim(j)) return false;
    ++i;
    ++j;
  }
  return i == ri && j == ro;
}


// ---------- online tuner of matmul launches (host/tuner.cc) ----------
struct CubeProblem {
  int64_t m = 0, n = 0, k = 0, nb0 = 1, nb1 = 1;
  DataType dtype = kFloat16;
  bool trans_a = false, trans_b = false;
};
struct CubeChoice {
  int tile = 0;    // 256, 128 or 64; 0: nothing measured
  int split = 1;   // parts of the k axis (1: one launch)
  double us = 0.0;
};
// The measured choice for a product shape, measuring it first when the shape is new and a tuner is switched on
// (Config::SetOnlineTuner / SetLazyTuner). False: no tuner, no device, or the shape could not be measured.
bool CubeTunerLookup(const CubeProblem &q, CubeChoice *out);
void CubeTunerStats(uint64_t *shapes_measured, uint64_t *table_size);
void CubeTunerClear();

class Compiler {
 public:
  explicit Compiler(VKernel *k) : k_(k), n_(static_cast<int>(k->ops_.size())) {}

  // Partition modes, tried in order until every sub-kernel compiles: 0 joins an operator to its
  // producers' sub-kernel whenever the hard rules allow, 1 also requires broadcast-compatible
  // shapes, 2 additionally ends a sub-kernel after every reduce (the reference's rule), 3 gives
  // every operator its own sub-kernel.
  size_t Run();

  size_t RunOnce(int mode);

 private:
  size_t RunModes();

  // ---------- reduces shared between workgroups ----------
  // A reduce with few outputs gives the schedules few workgroups (one per output, or per 512 outputs along the
  // innermost axis): a column sum of a [4096, 4096] tensor would run on 8 of 256 compute units, a sum of a whole
  // tensor on one. The reference adds partial results across blocks with atomics (src/vm_gpu.cu:750-939); here, to
  // keep results the same on every run, such a reduce R = reduce(x, dims) becomes, for the duration of one code
  // generation, R' = the same reduce over each of S parts of the reduced index space (one more, outermost, dim of
  // extent S on its result: a kept axis that no input has) and reduce(R', dim 0), which every consumer of R reads.
  // Only reduces whose consumers work on the reduce's own output shape qualify (a consumer that walks x again would
  // be as short of workgroups in the second launch). SplitLongReduces rewrites the operator list and returns true
  // if it changed anything; UndoSplitReduces restores it and renumbers the operators the programs refer to.
  bool SplitLongReduces();
  void UndoSplitReduces(bool keep_programs);
  struct SplitRecord {
    NDObject *reduce;     // the user's reduce (holds part_split and the longer shape meanwhile)
    NDObject *second;     // the synthetic reduce over the parts (owned here)
    NDObject *turned = nullptr;  // the partial results seen with the parts innermost: what `second` reads (owned here)
    NDObject *layout = nullptr;  // strides the launch over the parts stores its results with: parts innermost (owned here)
    int64_t shape[kMaxRank];
    size_t rank;
    IntArrayRef axis0;    // what `second` reduces over: {0}, or the last dim of `turned`
    int64_t zero = 0;
    IntArrayRef turn_order;  // the permutation `turned` stands for
    int64_t turn_dims[kMaxRank];
  };
  std::vector<SplitRecord *> splits_;
  // The strides a shared reduce's partial results are stored with (nullptr: dense in their own shape).
  const NDObject *PartsLayout(const NDObject *o) const {
    if (o->kind != kObjReduce || o->part_split == 0) return nullptr;
    for (const SplitRecord *rec : splits_)
      if (rec->reduce == o) return rec->layout;
    return nullptr;
  }
  struct Repoint {
    NDObject *consumer;
    int slot;
    NDObject *was;
  };
  std::vector<Repoint> repoints_;
  std::vector<NDObject *> saved_ops_;
  VKernel *k_;
  int n_;
  std::vector<int> area_, ws_slot_, store_of_, level_;
  std::vector<char> live_, mat_;
  std::vector<char> absorbed_;  // stores of a Concat whose parts write the user's buffer themselves
  int n_areas_ = 0;
  struct AreaInfo {
    bool cube = false;
    bool has_reduce = false;
    const NDObject *reduce = nullptr;
    int rank = 0;
    int64_t dom[kMaxRank];
    const NDObject *cube_op = nullptr;
    int attn = -1;  // index into attn_groups_ when the sub-kernel is one fused attention
    int red_at_level[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // reduces per sweep: the interpreter has two reduce slots per sweep
    int stage = 0;  // the caller's group (parallel / sequence kernels); operators of different groups never share a launch
    int n_ops = 0;  // operators joined so far (a program has room for about 500 instruction words and 160 nodes)
    bool has_part = false;  // holds a reduce shared between workgroups: only operators of its input's index space join
    int64_t over_parts = 0;  // holds the reduce over the parts of a shared reduce: its output's elements (0: none); nothing larger joins
  };
  std::vector<AreaInfo> areas_;

  // softmax(Q K^T * scale) V written as matmul / mul / cast / max / sub / exp / sum / div / cast /
  // matmul (examples/03_attention.py:30-50): recognised as a whole and run by the fused kernel.
  struct AttnGroup {
    NDObject *m1, *m2, *q, *k, *v;
    float scale;
    int area;
    // The result goes straight into a Store through strides (a Store with a stride list, or the dense Store of a
    // Permute of the result that keeps the head dimension innermost): no dense copy of the result exists then.
    NDObject *out_store = nullptr;
    uint32_t out_row = 0, out_outer = 0, out_inner = 0, out_nb_inner = 1;
    int64_t out_base = 0;
  };
  // How an operand of a fused attention lies in memory (VAttnHeader: strides in elements). `ok`: the kernel can
  // read it in place (a load, or a permute / slice of a load; head dimension contiguous; at most two batch axes
  // unless it is dense; every stride a multiple of eight elements).
  struct AttnLayout {
    bool ok = false;
    const NDObject *root = nullptr;  // the load whose address the operand starts from
    int64_t base = 0;                // element offset of the view inside that buffer
    uint32_t row = 0, outer = 0, inner = 0, nb_inner = 1;
  };
  AttnLayout AttnOperandLayout(const NDObject *x) const;
  std::vector<AttnGroup> attn_groups_;
  std::vector<int> attn_of_;
  void DetectAttention();

  // ---------- liveness ----------
  void MarkLive();

  // ---------- partition into sub-kernels ----------
  static bool IsLeaf(const NDObject *o) { return o->kind == kObjLoad || o->kind == kObjBroadcastS; }
  static bool IsStoreLike(const NDObject *o) { return o->kind == kObjStore || o->kind == kObjConcatPart; }

  // A view: reshape of a materialised value (or of a load) that is read through its new shape.
  bool IsView(const NDObject *o) const {
    return (o->kind == kObjReshape && !IsSqueezeReshape(o)) || o->kind == kObjPermute || o->kind == kObjSlice || o->kind == kObjHalf64;
  }

  // The operator whose buffer a view chain ends at.
  const NDObject *ViewRoot(const NDObject *o) const {
    while (IsView(o)) o = o->in[0];
    return o;
  }

  bool DomCompatible(const AreaInfo &ai, const int64_t *dims, int rank) const;

  void DomMerge(AreaInfo &ai, const int64_t *dims, int rank);

  static bool SameReduce(const NDObject *a, const NDObject *b);

  // Sweep an operator would run in if it joined sub-kernel a: one more than the deepest reduce among the
  // operators of a it depends on.
  int LevelIn(int a, const NDObject *o) const;

  bool CanJoin(int a, const NDObject *o);

  void Join(int a, const NDObject *o);

  void Partition();

  // ---------- which values cross sub-kernels ----------
  void PlanMaterialisation();

  // ---------- one sub-kernel ----------
  ANode nodes_[kMaxNodes];
  int nn_ = 0;
  std::vector<int> node_of_;  // op id -> node (per area)
  Axis axes_[kMaxAxes];
  int n_axes_ = 0;
  int order_[kMaxAxes];       // ordered axes, outermost first
  int pos_[kMaxAxes];         // axis -> position in order_
  Dim dims_[kMaxAxes];
  int n_dims_ = 0;
  int dim_of_axis_[kMaxAxes]; // ordered position -> merged dim
  // kept / reduced lists, innermost first (indices into dims_)
  int klist_[DVM_VEC_MAXR], rlist_[DVM_VEC_MAXR];
  // Kept dims beyond the VM's DVM_VEC_MAXR (the outermost ones) are peeled: the program covers one index of
  // them and is launched once per index, every operand address moved by that index times its stride.
  static constexpr int kMaxPeel = 4;
  int n_peel_ = 0;
  int peel_dim_[kMaxPeel];
  int64_t peel_stride_[DVM_VEC_MAXMEM][kMaxPeel];
  int nk_ = 0, nr_ = 0;
  // program under construction
  Program *prog_ = nullptr;
  VVecHeader hdr_;
  VMemDesc mems_[DVM_VEC_MAXMEM];
  int n_mem_ = 0;
  std::vector<uint64_t> code_;
  bool conservative_ = false;
  int mode_ = 0;
  bool single_round_ = false;
  int held_[kMaxNodes];  // registers whose release waits for the end of the sweep
  int n_held_ = 0;
  bool split_inner_ = false;  // pointwise programs with a gathered operand walk the innermost axis in tiles of 64
  int acc_node_ = -1;
  uint32_t sreg_used_ = 0;
  uint32_t vslot_used_ = 0;
  int max_vslot_ = 0;
  int vslot_limit_ = 0;
  int cur_sec_ = 0;

  int AddNode(AKind kind, NDObject *op, DataType t, const int64_t *dims, int rank);

  // Leaf node for an operand coming from outside the sub-kernel.
  int LeafFor(NDObject *v);

  int cur_area_ = 0;
  void Fail(const char *why);

  void CompileArea(int a);
  void CompileCube(int a);
  uint32_t FuseCubeEpilogue();
  void CompileAttn(int g);
  void BuildNodes(int a);
  void UnifyAxes();
  void OrderAndMerge();
  void ChooseSchedule();
  void EmitProgram();
  void FinishProgram();
  void ReplicatePeeled();

  // tables of the passes: members, so that a kernel compiled again (dynamic shapes) allocates nothing
  std::vector<int> scratch_a_, scratch_b_;
  std::vector<char> scratch_c_;
  std::vector<uint64_t> scratch_code_;
  // union-find over (node, dim) variables
  std::vector<int> uf_;
  int Find(int x) {
    while (uf_[x] != x) {
      uf_[x] = uf_[uf_[x]];
      x = uf_[x];
    }
    return x;
  }
  void Union(int a, int b) {
    a = Find(a);
    b = Find(b);
    if (a != b) uf_[b] = a;
  }
  int Var(int node, int dim) const { return node * kMaxRank + dim; }
  void UnifyAligned(int out, int in);

  // emission helpers
  void Emit(uint32_t op, uint32_t sub, uint32_t kind, uint32_t rnd, uint32_t a, uint32_t imm);
  void DropCastBeforeStore(const uint32_t *mem_dtypes);
  void DropUnreadSRegStores();
  void FuseSweepInstructions();
  void MarkUniformRuns();
  void PairLoads();
  void PlanRereads();
  bool FitsSweepBuild();
  bool mem_is_view_[DVM_VEC_MAXMEM] = {false};  // memory operand i is a strided view
  int last_mem_ = -1;         // memory operand of the last memory instruction emitted in this round, or -1
  int u_ = 2;                 // slabs per lane per instruction of the program being compiled
  bool uniform_emit_ = false; // the value being computed is the same in every element of a lane's accumulator
  int Resolve(int v) const {
    while (nodes_[v].kind == AK_ALIAS) v = nodes_[v].in[0];
    return v;
  }
  int MemIndex(int v);
  int CubeMemIndex(int v);
  bool cube_mode_ = false;
  VCubeMem cmems_[DVM_CUBE_MAXMEM];
  const NDObject *cube_out_ = nullptr;
  uint32_t pw_threads_cap_ = 256;     // lanes of a pointwise workgroup in this attempt (128 doubles the V register slots a lane has)
  int area_ops_limit_ = kMaxAreaOps;  // operators per sub-kernel in this attempt (RunModes lowers it when a sub-kernel runs out of registers)
  int gmm_bias_node_ = -1;  // the [groups, n] bias of a grouped matmul (its row goes with the group, not with the output's dims)
  bool SimpleOperand(int v);
  void EmitOperandInsn(uint32_t op, uint32_t sub, uint32_t rnd, int v);
  void EmitValue(int v);
  void ComputeInto(int v);
  void BeforeOverwrite();
  void SaveAcc(int v);
  void ConsumeUse(int v);
  void ReleaseReg(int v);
  int AllocSReg();
  int AllocVSlot(int n);
  void CountCone(int v);
  void EmitSection(int sec);
  int n_sec_ = 1;
};

// small helpers shared by the translation units
uint32_t Pow2Ceil(uint64_t v);
uint32_t Log2(uint32_t v);

}  // namespace dvm

#endif  // DVM_AMD_HOST_COMPILER_H_
