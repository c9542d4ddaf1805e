// Graph -> sub-kernels -> gfx950 tile bytecode.
//
// Role in the reference: shape normalisation (src/ops.cc Normalize family),
// the split kernel's graph cutter (src/xkernel.cc:1980-2119), domain / tiling
// (src/kernel.cc:765-1194), liveness + buffer allocation (src/kernel.cc:196-317,
// 1285-1332) and the Emit methods (src/ops.cc). The gfx950 target differs in
// what a sub-kernel may contain: a reduce and its consumers stay in one launch
// (consecutive sweeps of one workgroup-resident program), broadcasts are
// stride-0 operands, and intermediate values live in lane registers, so the
// "tiling" step is an index-space analysis instead of a local-memory planner:
//   1. every tensor dim of every value is unified into domain axes;
//   2. axes are ordered, merged where all memory operands allow it, and split
//      into a kept list and a reduced list;
//   3. a schedule (pointwise / reduce over the innermost axis / reduce with
//      the innermost axis kept) and its launch geometry are chosen;
//   4. the operator DAG is linearised into accumulator-machine code, section
//      by section (code outside sweeps works on the kept space, a sweep walks
//      the reduce space), values that cannot stay in a register across a
//      sweep are recomputed from their loads.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "ir.h"
#include "system.h"

namespace dvm {

VKernel::~VKernel() {
  for (NDObject *o : ops_) delete o;
}

NDObject *VKernel::Append(NDObject *op) {
  op->id = static_cast<int>(ops_.size());
  op->stage = cur_stage_;
  ops_.push_back(op);
  normalized_ = false;
  compiled_ = false;
  return op;
}

// ---- shape inference -----------------------------------------------------------------

namespace {

void BroadcastShapes(const NDObject *a, const NDObject *b, int64_t *out, size_t *out_rank) {
  const size_t ra = a->shape_ref_->size, rb = b->shape_ref_->size;
  const size_t r = std::max(ra, rb);
  for (size_t i = 0; i < r; ++i) {
    const int64_t da = i + ra >= r ? a->shape_ref_->data[i + ra - r] : 1;
    const int64_t db = i + rb >= r ? b->shape_ref_->data[i + rb - r] : 1;
    if (da != db && da != 1 && db != 1) Throw("operands cannot be broadcast together");
    out[i] = da == 1 ? db : da;
  }
  *out_rank = r;
}

}  // namespace

void VKernel::Normalize() {
  // a slice bound below zero counts from the end of its axis; bounds past either end stop there
  // (src/dvm.cc:770-773,826-831 of the reference, which clips the end; NumPy's rule for both)
  auto bound = [](int64_t v, int64_t extent) {
    if (v < 0) v += extent;
    return std::min(std::max<int64_t>(v, 0), extent);
  };
  for (NDObject *o : ops_) {
    switch (o->kind) {
      case kObjLoad:
        if (o->strided) {
          if (o->slice_end != nullptr) {  // strided slice: the value's shape comes from start / end / step
            const size_t r = o->full_shape_ref->size;
            if (o->slice_start->size != r || o->slice_end->size != r || o->slice_step->size != r) Throw("slice lists do not match the tensor rank");
            for (size_t i = 0; i < r; ++i) {
              const int64_t st = o->slice_step->data[i];
              if (st <= 0) Throw("slice step has to be positive");
              const int64_t len = bound(o->slice_end->data[i], o->full_shape_ref->data[i]) -
                                  bound(o->slice_start->data[i], o->full_shape_ref->data[i]);
              o->shape_[i] = len > 0 ? (len + st - 1) / st : 0;
            }
            o->own_ref_.size = r;
          }
          const size_t r = o->shape_ref_->size;
          if (r > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
          o->view_base_ = o->view_offset;
          if (o->stride_ref != nullptr) {
            if (o->stride_ref->size != r) Throw("stride list does not match the tensor rank");
            for (size_t i = 0; i < r; ++i) o->vstride_[i] = o->stride_ref->data[i];
          } else {
            if (o->full_shape_ref->size != r || o->slice_start->size != r) Throw("slice lists do not match the tensor rank");
            int64_t dense = 1;
            for (size_t i = r; i-- > 0;) {
              const int64_t st = o->slice_step != nullptr ? o->slice_step->data[i] : 1;
              const int64_t first = bound(o->slice_start->data[i], o->full_shape_ref->data[i]);
              if (first + (o->shape_ref_->data[i] - 1) * st >= o->full_shape_ref->data[i]) {
                if (o->shape_ref_->data[i] > 0) Throw("slice reaches outside the tensor");
              }
              o->vstride_[i] = dense * st;
              o->view_base_ += first * dense;
              dense *= o->full_shape_ref->data[i];
            }
          }
        }
        if (o->shape_ref_->size > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
        break;
      case kObjStore:
        o->SetShape(o->in[0]->shape_ref_->data, o->in[0]->shape_ref_->size);
        if (o->strided) {
          if (o->stride_ref->size != o->in[0]->shape_ref_->size) Throw("stride list does not match the tensor rank");
          for (size_t i = 0; i < o->stride_ref->size; ++i) o->vstride_[i] = o->stride_ref->data[i];
          o->view_base_ = o->view_offset;
        }
        break;
      case kObjUnary:
      case kObjBinaryS:
      case kObjCompareS:
      case kObjCast:
      case kObjCopy:
        o->SetShape(o->in[0]->shape_ref_->data, o->in[0]->shape_ref_->size);
        break;
      case kObjBinary:
      case kObjCompare: {
        size_t r;
        BroadcastShapes(o->in[0], o->in[1], o->shape_, &r);
        o->own_ref_.size = r;
        break;
      }
      case kObjSelect: {
        NDObject tmp(kObjCopy, o->type_id_);
        size_t r;
        BroadcastShapes(o->in[0], o->in[1], tmp.shape_, &r);
        tmp.own_ref_.size = r;
        BroadcastShapes(&tmp, o->in[2], o->shape_, &r);
        o->own_ref_.size = r;
        break;
      }
      case kObjBroadcast: {
        const size_t r = o->aux_ref->size;
        const size_t ri = o->in[0]->shape_ref_->size;
        if (r > static_cast<size_t>(kMaxRank) || ri > r) Throw("bad broadcast target");
        for (size_t i = 0; i < r; ++i) {
          int64_t d = o->aux_ref->data[i];
          if (d == -1) {
            if (i + ri < r) Throw("bad broadcast target");
            d = o->in[0]->shape_ref_->data[i + ri - r];
          }
          o->shape_[i] = d;
        }
        o->own_ref_.size = r;
        break;
      }
      case kObjBroadcastS:
        if (o->aux_ref->size > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
        o->SetShape(o->aux_ref->data, o->aux_ref->size);
        break;
      case kObjReduce: {
        const NDObject *x = o->in[0];
        const size_t r = x->shape_ref_->size;
        bool red[kMaxRank] = {false};
        for (size_t i = 0; i < o->aux_ref->size; ++i) {
          int64_t d = o->aux_ref->data[i];
          if (d < 0) d += static_cast<int64_t>(r);
          if (d < 0 || d >= static_cast<int64_t>(r)) Throw("reduce axis out of range");
          red[d] = true;
        }
        size_t n = 0;
        for (size_t i = 0; i < r; ++i) {
          if (red[i]) {
            if (o->keepdims) o->shape_[n++] = 1;
          } else {
            o->shape_[n++] = x->shape_ref_->data[i];
          }
        }
        o->own_ref_.size = n;
        break;
      }
      case kObjConcatPart:
        o->SetShape(o->in[0]->shape_ref_->data, o->in[0]->shape_ref_->size);
        break;
      case kObjConcat: {
        const NDObject *first = o->parts[0];
        const size_t r = first->shape_ref_->size;
        int64_t dim = o->slice_dim;
        if (dim < 0) dim += static_cast<int64_t>(r);
        if (dim < 0 || dim >= static_cast<int64_t>(r)) Throw("concat dim out of range");
        for (size_t i = 0; i < r; ++i) o->shape_[i] = first->shape_ref_->data[i];
        o->shape_[dim] = 0;
        for (const NDObject *p : o->parts) {
          if (p->shape_ref_->size != r) Throw("concat inputs differ in rank");
          for (size_t i = 0; i < r; ++i)
            if (static_cast<int64_t>(i) != dim && p->shape_ref_->data[i] != first->shape_ref_->data[i]) Throw("concat inputs differ outside the concat dim");
          o->shape_[dim] += p->shape_ref_->data[dim];
        }
        o->own_ref_.size = r;
        int64_t dense[kMaxRank], acc = 1;
        for (size_t i = r; i-- > 0;) {
          dense[i] = acc;
          acc *= o->shape_[i];
        }
        int64_t at = 0;
        for (NDObject *p : o->parts) {  // where each part lands: the buffer's strides, its offset along the dim
          p->strided = true;
          for (size_t i = 0; i < r; ++i) p->vstride_[i] = dense[i];
          p->view_base_ = at * dense[dim];
          at += p->shape_ref_->data[dim];
        }
        break;
      }
      case kObjPermute:
      case kObjSlice: {
        // A view of the input's memory: element strides and offset of the input (its own when it is a view or a
        // strided load, those of a dense row-major tensor otherwise), reordered or moved by the slice's start.
        const NDObject *x = o->in[0];
        const size_t r = x->shape_ref_->size;
        int64_t xs[kMaxRank];
        if (x->strided && x->kind != kObjStore) {
          for (size_t i = 0; i < r; ++i) xs[i] = x->vstride_[i];
          o->view_base_ = x->view_base_;
        } else {
          int64_t dense = 1;
          for (size_t i = r; i-- > 0;) {
            xs[i] = dense;
            dense *= x->shape_ref_->data[i];
          }
          o->view_base_ = 0;
        }
        o->strided = true;
        if (o->kind == kObjPermute) {
          if (o->aux_ref->size != r) Throw("permutation does not match the tensor rank");
          bool seen[kMaxRank] = {false};
          for (size_t i = 0; i < r; ++i) {
            int64_t d = o->aux_ref->data[i];
            if (d < 0) d += static_cast<int64_t>(r);
            if (d < 0 || d >= static_cast<int64_t>(r) || seen[d]) Throw("permutation names a dim twice or out of range");
            seen[d] = true;
            o->shape_[i] = x->shape_ref_->data[d];
            o->vstride_[i] = xs[d];
          }
        } else if (o->slice_dim < 0 && o->slice_start != nullptr) {
          if (o->slice_start->size != r || o->aux_ref->size != r) Throw("slice lists do not match the tensor rank");
          for (size_t i = 0; i < r; ++i) {
            const int64_t ext = x->shape_ref_->data[i];
            int64_t st = o->slice_start->data[i];
            if (st < 0) st += ext;
            const int64_t n = o->aux_ref->data[i];
            if (st < 0 || n < 0 || st + n > ext) Throw("slice reaches outside the tensor");
            o->shape_[i] = n;
            o->vstride_[i] = xs[i];
            o->view_base_ += st * xs[i];
          }
        } else {
          int64_t dim = o->slice_dim;
          if (dim < 0) dim += static_cast<int64_t>(r);
          if (dim < 0 || dim >= static_cast<int64_t>(r)) Throw("slice dim out of range");
          auto as_int = [](const ScalarRef *s) -> int64_t {
            switch (s->type) {
              case kInt32: return s->i32;
              case kInt64: return s->i64;
              case kFloat32: return static_cast<int64_t>(s->f32);
              default: Throw("slice bounds have to be integers");
            }
            return 0;
          };
          const int64_t ext = x->shape_ref_->data[dim];
          const int64_t b = bound(o->dim_begin_ref != nullptr ? as_int(o->dim_begin_ref) : o->dim_begin, ext);
          const int64_t e = bound(o->dim_end_ref != nullptr ? as_int(o->dim_end_ref) : o->dim_end, ext);
          for (size_t i = 0; i < r; ++i) {
            o->shape_[i] = x->shape_ref_->data[i];
            o->vstride_[i] = xs[i];
          }
          o->shape_[dim] = e > b ? e - b : 0;
          o->view_base_ += b * xs[dim];
        }
        o->own_ref_.size = r;
        break;
      }
      case kObjReshape: {
        if (o->in[0]->strided && o->in[0]->kind != kObjStore && o->in[0]->kind != kObjLoad) {
          Throw("DVM EXCEPTION. reason: a reshape of a permuted or sliced value needs a Copy in between on the gfx950 backend");
        }
        const size_t r = o->aux_ref->size;
        if (r > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
        int64_t known = 1;
        int infer = -1;
        for (size_t i = 0; i < r; ++i) {
          o->shape_[i] = o->aux_ref->data[i];
          if (o->shape_[i] == -1) {
            infer = static_cast<int>(i);
          } else {
            known *= o->shape_[i];
          }
        }
        o->own_ref_.size = r;
        const int64_t total = o->in[0]->numel();
        if (infer >= 0) o->shape_[infer] = known == 0 ? 0 : total / known;
        if (o->numel() != total) Throw("reshape changes the number of elements");
        break;
      }
      case kObjMatMul: {
        const NDObject *a = o->in[0], *b = o->in[1];
        const size_t ra = a->shape_ref_->size, rb = b->shape_ref_->size;
        if (ra < 2 || rb < 2) Throw("matmul operands need rank >= 2");
        const int64_t m = o->trans_a ? a->dim(ra - 1) : a->dim(ra - 2);
        const int64_t ka = o->trans_a ? a->dim(ra - 2) : a->dim(ra - 1);
        const int64_t kb = o->trans_b ? b->dim(rb - 1) : b->dim(rb - 2);
        const int64_t n = o->trans_b ? b->dim(rb - 2) : b->dim(rb - 1);
        if (ka != kb) Throw("matmul inner dimensions differ");
        const size_t ba = ra - 2, bb = rb - 2, br = std::max(ba, bb);
        if (br + 2 > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
        for (size_t i = 0; i < br; ++i) {
          const int64_t da = i + ba >= br ? a->dim(i + ba - br) : 1;
          const int64_t db = i + bb >= br ? b->dim(i + bb - br) : 1;
          if (da != db && da != 1 && db != 1) Throw("matmul batch dimensions cannot be broadcast");
          o->shape_[i] = da == 1 ? db : da;
        }
        o->shape_[br] = m;
        o->shape_[br + 1] = n;
        o->own_ref_.size = br + 2;
        break;
      }
    }
  }
  normalized_ = true;
}

// ---- compiler ------------------------------------------------------------------------

namespace {

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

uint32_t FloatBits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

VDim MakeVDim(uint32_t d) {
  VDim v;
  v.extent = d;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  v.shift = s;
  v.magic = static_cast<uint32_t>((((1ull << 32) * ((1ull << s) - d)) / (d == 0 ? 1 : d)) + 1);
  v.pad = 0;
  return v;
}

uint32_t MemDType(DataType t) {
  switch (t) {
    case kBool: return VDT_BOOL;
    case kFloat16: return VDT_F16;
    case kBFloat16: return VDT_BF16;
    case kFloat32: return VDT_F32;
    case kInt32: return VDT_I32;
    default: Throw("tensor type without a device form");
  }
}

uint32_t RndOf(DataType t) { return t == kFloat16 ? VRND_F16 : (t == kBFloat16 ? VRND_BF16 : VRND_NONE); }

bool IsPointwiseKind(ObjKind k) {
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
bool IsSqueezeReshape(const NDObject *o) {
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

}  // namespace

class Compiler {
 public:
  explicit Compiler(VKernel *k) : k_(k), n_(static_cast<int>(k->ops_.size())) {}

  // Partition modes, tried in order until every sub-kernel compiles: 0 joins an operator to its
  // producers' sub-kernel whenever the hard rules allow, 1 also requires broadcast-compatible
  // shapes, 2 additionally ends a sub-kernel after every reduce (the reference's rule), 3 gives
  // every operator its own sub-kernel.
  size_t Run() {
    for (int mode = k_->part_mode_; mode < 3; ++mode) {
      try {
        const size_t ws = RunOnce(mode);
        k_->part_mode_ = mode;
        return ws;
      } catch (const std::runtime_error &) {
      }
    }
    k_->part_mode_ = 3;
    return RunOnce(3);
  }

  size_t RunOnce(int mode) {
    mode_ = mode;
    conservative_ = mode >= 2;
    area_.assign(n_, -1);
    level_.assign(n_, 0);
    live_.assign(n_, 0);
    mat_.assign(n_, 0);
    absorbed_.assign(n_, 0);
    ws_slot_.assign(n_, -1);
    store_of_.assign(n_, -1);
    MarkLive();
    attn_groups_.clear();
    attn_of_.assign(n_, -1);
    if (mode_ == 0) DetectAttention();
    Partition();
    k_->programs_.clear();
    k_->ws_sizes_.clear();
    k_->ws_offsets_.clear();
    PlanMaterialisation();
    for (int a = 0; a < n_areas_; ++a) CompileArea(a);
    size_t total = 0;
    for (size_t i = 0; i < k_->ws_sizes_.size(); ++i) {
      k_->ws_offsets_.push_back(total);
      total += (k_->ws_sizes_[i] + 255) & ~static_cast<size_t>(255);
    }
    k_->ws_bytes_ = total;
    return total;
  }

 private:
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
  };
  std::vector<AreaInfo> areas_;

  // softmax(Q K^T * scale) V written as matmul / mul / cast / max / sub / exp / sum / div / cast /
  // matmul (examples/03_attention.py:30-50): recognised as a whole and run by the fused kernel.
  struct AttnGroup {
    NDObject *m1, *m2, *q, *k, *v;
    float scale;
    int area;
  };
  std::vector<AttnGroup> attn_groups_;
  std::vector<int> attn_of_;
  void DetectAttention();

  // ---------- liveness ----------
  void MarkLive() {
    for (int i = n_ - 1; i >= 0; --i) {
      NDObject *o = k_->ops_[i];
      if (o->kind == kObjStore) live_[i] = 1;
      if (!live_[i]) continue;
      for (int j = 0; j < o->nin; ++j)
        if (o->in[j] != nullptr) live_[o->in[j]->id] = 1;
      for (NDObject *p : o->parts) live_[p->id] = 1;
    }
  }

  // ---------- partition into sub-kernels ----------
  static bool IsLeaf(const NDObject *o) { return o->kind == kObjLoad || o->kind == kObjBroadcastS; }
  static bool IsStoreLike(const NDObject *o) { return o->kind == kObjStore || o->kind == kObjConcatPart; }

  // A view: reshape of a materialised value (or of a load) that is read through its new shape.
  bool IsView(const NDObject *o) const {
    return (o->kind == kObjReshape && !IsSqueezeReshape(o)) || o->kind == kObjPermute || o->kind == kObjSlice;
  }

  // The operator whose buffer a view chain ends at.
  const NDObject *ViewRoot(const NDObject *o) const {
    while (IsView(o)) o = o->in[0];
    return o;
  }

  bool DomCompatible(const AreaInfo &ai, const int64_t *dims, int rank) const {
    const int r = std::max(ai.rank, rank);
    for (int i = 0; i < r; ++i) {
      const int64_t da = i + ai.rank >= r ? ai.dom[i + ai.rank - r] : 1;
      const int64_t db = i + rank >= r ? dims[i + rank - r] : 1;
      if (da != db && da != 1 && db != 1) return false;
    }
    return true;
  }

  void DomMerge(AreaInfo &ai, const int64_t *dims, int rank) {
    const int r = std::max(ai.rank, rank);
    int64_t out[kMaxRank];
    for (int i = 0; i < r; ++i) {
      const int64_t da = i + ai.rank >= r ? ai.dom[i + ai.rank - r] : 1;
      const int64_t db = i + rank >= r ? dims[i + rank - r] : 1;
      out[i] = da == 1 ? db : da;
    }
    std::memcpy(ai.dom, out, sizeof(int64_t) * r);
    ai.rank = r;
  }

  static bool SameReduce(const NDObject *a, const NDObject *b) {
    const NDObject *xa = a->in[0], *xb = b->in[0];
    if (xa->rank() != xb->rank()) return false;
    for (int i = 0; i < xa->rank(); ++i)
      if (xa->dim(i) != xb->dim(i)) return false;
    bool ra[kMaxRank] = {false}, rb[kMaxRank] = {false};
    for (size_t i = 0; i < a->aux_ref->size; ++i) {
      int64_t d = a->aux_ref->data[i];
      ra[d < 0 ? d + xa->rank() : d] = true;
    }
    for (size_t i = 0; i < b->aux_ref->size; ++i) {
      int64_t d = b->aux_ref->data[i];
      rb[d < 0 ? d + xb->rank() : d] = true;
    }
    for (int i = 0; i < xa->rank(); ++i)
      if (xa->dim(i) != 1 && ra[i] != rb[i]) return false;
    return true;
  }

  // Sweep an operator would run in if it joined sub-kernel a: one more than the deepest reduce among the
  // operators of a it depends on.
  int LevelIn(int a, const NDObject *o) const {
    int lvl = 0;
    for (int j = 0; j < o->nin; ++j) {
      const NDObject *v = o->in[j];
      if (v == nullptr || area_[v->id] != a) continue;
      lvl = std::max(lvl, level_[v->id] + (v->kind == kObjReduce ? 1 : 0));
    }
    return lvl;
  }

  bool CanJoin(int a, const NDObject *o) {
    if (a >= static_cast<int>(areas_.size())) return true;  // a fresh sub-kernel
    const AreaInfo &ai = areas_[a];
    if (ai.stage != o->stage) return false;
    // a store goes where the value it stores is computed (an operator's own output is never a reason to cut)
    if (IsStoreLike(o) && ai.attn < 0 && !ai.cube && area_[o->in[0]->id] == a) return true;
    if (o->kind == kObjReduce && LevelIn(a, o) < 8 && ai.red_at_level[LevelIn(a, o)] >= 2) return false;
    if (o->kind == kObjMatMul) return false;
    if (ai.n_ops >= kMaxAreaOps && !IsStoreLike(o)) return false;  // long graphs are cut into several launches
    if (ai.attn >= 0) return o->kind == kObjStore && o->in[0] == attn_groups_[ai.attn].m2;
    if (ai.cube) {
      if (!IsPointwiseKind(o->kind)) return false;
      if (mode_ >= 2 && !(o->kind == kObjStore && o->in[0] == ai.cube_op)) return false;  // plain matmul, epilogue on its own
      // the epilogue works on the matmul's own output domain
      const NDObject *c = ai.cube_op;
      if (o->rank() != c->rank()) return false;
      for (int i = 0; i < o->rank(); ++i)
        if (o->dim(i) != c->dim(i)) return false;
      return true;
    }
    if (o->kind == kObjReduce) {
      if (ai.has_reduce && !SameReduce(ai.reduce, o)) return false;
      return mode_ == 0 || DomCompatible(ai, o->in[0]->shape_ref_->data, o->in[0]->rank());
    }
    // A store of a value from outside (a load, a view, another launch's result) is a copy nothing else in the
    // sub-kernel relates to: it joins only one whose index space it fills, element for element.
    if (IsStoreLike(o) && ai.n_ops > 0) {  // same extents in the same order, dims of extent 1 aside
      int i = 0, j = 0;
      while (true) {
        while (i < ai.rank && ai.dom[i] == 1) ++i;
        while (j < o->rank() && o->dim(j) == 1) ++j;
        if (i == ai.rank || j == o->rank()) break;
        if (ai.dom[i] != o->dim(j)) return false;
        ++i;
        ++j;
      }
      if (i != ai.rank || j != o->rank()) return false;
    }
    return mode_ == 0 || DomCompatible(ai, o->shape_ref_->data, o->rank());
  }

  void Join(int a, const NDObject *o) {
    while (a >= static_cast<int>(areas_.size())) areas_.push_back(AreaInfo());
    AreaInfo &ai = areas_[a];
    if (ai.n_ops == 0) ai.stage = o->stage;
    ++ai.n_ops;
    level_[o->id] = LevelIn(a, o);
    if (o->kind == kObjReduce && level_[o->id] < 8) ++ai.red_at_level[level_[o->id]];
    if (o->kind == kObjMatMul) {
      ai.cube = true;
      ai.cube_op = o;
      return;
    }
    if (ai.cube) return;
    if (o->kind == kObjReduce) {
      if (!ai.has_reduce) {
        ai.has_reduce = true;
        ai.reduce = o;
      }
      DomMerge(ai, o->in[0]->shape_ref_->data, o->in[0]->rank());
    }
    DomMerge(ai, o->shape_ref_->data, o->rank());
  }

  void Partition() {
    areas_.clear();
    const bool fuse = !conservative_;
    // Operators that share no tensor (directly or through other operators) never share a
    // sub-kernel: connected components are numbered first, each gets its own range of areas.
    std::vector<int> comp(n_);
    for (int i = 0; i < n_; ++i) comp[i] = i;
    auto find = [&](int x) {
      while (comp[x] != x) x = comp[x] = comp[comp[x]];
      return x;
    };
    for (int i = 0; i < n_; ++i) {
      NDObject *o = k_->ops_[i];
      if (!live_[i]) continue;
      for (int j = 0; j < o->nin; ++j) {
        if (o->in[j] == nullptr || o->in[j]->kind == kObjBroadcastS) continue;
        comp[find(i)] = find(o->in[j]->id);
      }
    }
    std::vector<int> comp_base(n_, -1);
    for (int i = 0; i < n_; ++i) {
      NDObject *o = k_->ops_[i];
      if (!live_[i] || IsLeaf(o)) continue;
      if (IsView(o)) continue;  // read through by its consumers
      if (o->kind == kObjConcat) {  // complete once the last of its parts has run; never computed itself
        int a = 0;
        for (const NDObject *p : o->parts) a = std::max(a, area_[p->id]);
        area_[i] = a;
        continue;
      }
      const int c = find(i);
      if (comp_base[c] < 0) comp_base[c] = static_cast<int>(areas_.size());
      if (attn_of_[i] >= 0) {
        AttnGroup &g = attn_groups_[attn_of_[i]];
        if (g.area < 0) {
          g.area = static_cast<int>(areas_.size());
          areas_.push_back(AreaInfo());
          areas_.back().attn = attn_of_[i];
          areas_.back().stage = o->stage;
          areas_.back().n_ops = 1;
        }
        area_[i] = g.area;
        continue;
      }
      int a = comp_base[c];
      for (int j = 0; j < o->nin; ++j) {
        const NDObject *v = o->in[j];
        if (v == nullptr || IsLeaf(v)) continue;
        bool cut = false;
        if (IsView(v)) {
          v = ViewRoot(v);
          if (IsLeaf(v)) continue;
          cut = true;
        }
        if (o->kind == kObjMatMul || v->kind == kObjConcat) cut = true;
        if (!fuse && v->kind == kObjReduce && !IsStoreLike(o)) cut = true;  // the reference's rule: a reduce ends its sub-kernel
        a = std::max(a, area_[v->id] + (cut ? 1 : 0));
      }
      if (o->kind == kObjMatMul || (mode_ >= 3 && !IsStoreLike(o))) a = std::max(a, static_cast<int>(areas_.size()));
      while (!CanJoin(a, o)) ++a;
      area_[i] = a;
      Join(a, o);
    }
    n_areas_ = static_cast<int>(areas_.size());
  }

  // ---------- which values cross sub-kernels ----------
  void PlanMaterialisation() {
    for (int i = 0; i < n_; ++i) {
      NDObject *o = k_->ops_[i];
      if (!live_[i]) continue;
      // a value stored through a stride list is not read back from there by later launches: they expect
      // the dense layout, so such a value also goes to the workspace when it crosses launches
      if (o->kind == kObjStore && !o->strided) store_of_[o->in[0]->id] = i;
    }
    for (int i = 0; i < n_; ++i) {
      NDObject *o = k_->ops_[i];
      if (!live_[i] || IsLeaf(o)) continue;
      for (int j = 0; j < o->nin; ++j) {
        const NDObject *v = o->in[j];
        if (v == nullptr) continue;
        const NDObject *root = ViewRoot(v);
        if (IsLeaf(root) || root->kind == kObjLoad) continue;
        const int user_area = IsView(o) ? -2 : area_[i];
        if (IsView(v) || (user_area != -2 && area_[root->id] != user_area)) mat_[root->id] = 1;
      }
    }
    for (int i = 0; i < n_; ++i)
      if (live_[i] && k_->ops_[i]->kind == kObjConcat) mat_[i] = 1;  // its parts need the buffer whoever reads it
    for (int i = 0; i < n_; ++i) {
      if (!mat_[i]) continue;
      NDObject *o = k_->ops_[i];
      if (store_of_[i] >= 0 && area_[store_of_[i]] == area_[i]) continue;  // later kernels read the user's output
      if (o->kind == kObjConcat && store_of_[i] >= 0) {  // the parts write straight into the stored output
        absorbed_[store_of_[i]] = 1;
        continue;
      }
      ws_slot_[i] = static_cast<int>(k_->ws_sizes_.size());
      k_->ws_sizes_.push_back(static_cast<size_t>(std::max<int64_t>(o->numel(), 1)) * DTypeSize(o->type_id_));
    }
  }

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

  int AddNode(AKind kind, NDObject *op, DataType t, const int64_t *dims, int rank) {
    if (nn_ >= kMaxNodes) Throw("sub-kernel too large");
    ANode &n = nodes_[nn_];
    std::memset(&n, 0, sizeof(n));
    n.kind = kind;
    n.op = op;
    n.dtype = t;
    n.dims = dims;
    n.rank = rank;
    n.addr_op = -1;
    n.ws_slot = -1;
    n.mem_idx = -1;
    n.reg = -1;
    for (int i = 0; i < kMaxRank; ++i) n.axis[i] = -1;
    return nn_++;
  }

  // Leaf node for an operand coming from outside the sub-kernel.
  int LeafFor(NDObject *v) {
    if (node_of_[v->id] >= 0) return node_of_[v->id];
    int idx;
    if (v->kind == kObjBroadcastS) {
      idx = AddNode(AK_SCALAR, v, v->type_id_, v->shape_ref_->data, v->rank());
    } else {
      idx = AddNode(AK_MEM, v, v->type_id_, v->shape_ref_->data, v->rank());
      const NDObject *root = ViewRoot(v);
      // a permuted or sliced value carries the strides of the whole chain down to the root's memory
      if (v->kind == kObjPermute || v->kind == kObjSlice) nodes_[idx].view = v;
      if (root->kind == kObjLoad) {
        nodes_[idx].addr_op = root->id;
        if (root->strided && nodes_[idx].view == nullptr) {
          if (root != v) Throw("DVM EXCEPTION. reason: a reshape of a strided load is not supported by the gfx950 backend");
          nodes_[idx].view = root;
        }
      } else if (ws_slot_[root->id] >= 0) {
        nodes_[idx].ws_slot = ws_slot_[root->id];
      } else {
        nodes_[idx].addr_op = store_of_[root->id];
      }
    }
    node_of_[v->id] = idx;
    return idx;
  }

  int cur_area_ = 0;
  void Fail(const char *why) {
    std::string msg = "cannot compile sub-kernel " + std::to_string(cur_area_) + " (partition mode " +
                      std::to_string(mode_) + "): " + why;
    if (std::getenv("DVM_DEBUG") != nullptr) {
      msg += "\n nodes:";
      for (int i = 0; i < nn_; ++i) {
        msg += "\n  n" + std::to_string(i) + " kind=" + std::to_string(nodes_[i].kind) + " op=%" +
               std::to_string(nodes_[i].op != nullptr ? nodes_[i].op->id : -1) + " dims=[";
        for (int d = 0; d < nodes_[i].rank; ++d) msg += std::to_string(nodes_[i].dims[d]) + ":" + std::to_string(nodes_[i].axis[d]) + " ";
        msg += "] in=" + std::to_string(nodes_[i].in[0]) + "," + std::to_string(nodes_[i].in[1]);
      }
    }
    Throw(msg);
  }

  void CompileArea(int a);
  void CompileCube(int a);
  void CompileAttn(int g);
  void BuildNodes(int a);
  void UnifyAxes();
  void OrderAndMerge();
  void ChooseSchedule();
  void EmitProgram();
  void FinishProgram();
  void ReplicatePeeled();

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
  void Emit(uint32_t op, uint32_t sub, uint32_t kind, uint32_t rnd, uint32_t a, uint32_t imm) {
    uint64_t w = VI_MAKE(op, sub, kind, rnd, a, imm);
    if (op == VOP_ENDSWEEP) w |= VI_ENDS;
    if (!cube_mode_) {
      const bool mem = op == VOP_ST || (op >= VOP_SRC_BASE && kind == VK_MEM);
      if (mem) {
        // consecutive memory instructions of one round that walk memory identically share their offsets
        if (last_mem_ >= 0 && std::memcmp(mems_[last_mem_].kstride, mems_[a].kstride, sizeof(mems_[a].kstride)) == 0 &&
            std::memcmp(mems_[last_mem_].rstride, mems_[a].rstride, sizeof(mems_[a].rstride)) == 0) {
          w |= VI_SAME_OFFS;
        }
        last_mem_ = static_cast<int>(a);
      } else if (op == VOP_SWEEP || op == VOP_ENDSWEEP) {
        last_mem_ = -1;
      } else if (uniform_emit_ && (op == VOP_UN || op == VOP_CAST ||
                                   ((op == VOP_BINF || op == VOP_BINI || op == VOP_CMP) && (kind == VK_IMM || kind == VK_SREG || kind == VK_ACC)))) {
        w |= VI_UNIFORM;
      }
    }
    code_.push_back(w);
  }
  void DropCastBeforeStore(const uint32_t *mem_dtypes);
  void FuseSweepInstructions();
  void MarkUniformRuns();
  void PlanRereads();
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

// ---------- node construction ----------

void Compiler::BuildNodes(int a) {
  nn_ = 0;
  node_of_.assign(n_, -1);
  for (int i = 0; i < n_; ++i) {
    if (area_[i] != a) continue;
    NDObject *o = k_->ops_[i];
    if (o->kind == kObjConcat) continue;  // a buffer its parts fill, nothing to compute
    if (absorbed_[i]) continue;             // its value was written in place by the parts of a Concat
    int in_idx[3] = {-1, -1, -1};
    for (int j = 0; j < o->nin; ++j) {
      NDObject *v = o->in[j];
      if (v == nullptr) continue;
      if (node_of_[v->id] >= 0 && area_[v->id] == a) {
        in_idx[j] = node_of_[v->id];
      } else {
        in_idx[j] = LeafFor(v);
      }
    }
    AKind kind = AK_OP;
    if (o->kind == kObjCopy || o->kind == kObjBroadcast || o->kind == kObjReshape) kind = AK_ALIAS;
    if (o->kind == kObjReduce) {
      // a reduce over axes of extent 1 only (tests/ut/test_reduce.py:91: [120,20,1] over axis 2) computes
      // nothing: sum, max and min of one element are the element; it is a squeeze of its input
      const NDObject *x = o->in[0];
      bool nothing = true;
      for (size_t j = 0; j < o->aux_ref->size; ++j) {
        int64_t d = o->aux_ref->data[j];
        if (d < 0) d += x->rank();
        if (x->dim(static_cast<int>(d)) != 1) nothing = false;
      }
      kind = nothing ? AK_ALIAS : AK_REDUCE;
    }
    if (IsStoreLike(o)) kind = AK_OUT;
    if (o->kind == kObjCast) {
      // widening conversions do not change the register value
      const DataType s = o->in[0]->type_id_, d = o->type_id_;
      const bool nop = (d == kFloat32 && (s == kFloat16 || s == kBFloat16)) || (s == kBool && d != kInt32);
      if (nop) kind = AK_ALIAS;
    }
    const int idx = AddNode(kind, o, o->type_id_, o->shape_ref_->data, o->rank());
    ANode &n = nodes_[idx];
    n.nin = o->nin;
    for (int j = 0; j < 3; ++j) n.in[j] = in_idx[j];
    if (kind == AK_OUT) {
      if (o->kind == kObjConcatPart) {
        n.ws_slot = ws_slot_[o->cat->id];
        if (n.ws_slot < 0) n.addr_op = store_of_[o->cat->id];
        n.view = o;
      } else {
        n.addr_op = i;
        if (o->strided) n.view = o;
      }
    }
    node_of_[i] = idx;
    // a value later sub-kernels read and that the user does not store: write it to workspace
    if (mat_[i] && ws_slot_[i] >= 0) {
      const int out = AddNode(AK_OUT, o, o->type_id_, o->shape_ref_->data, o->rank());
      nodes_[out].nin = 1;
      nodes_[out].in[0] = idx;
      nodes_[out].ws_slot = ws_slot_[i];
    }
  }
}

// Unifies the dims of `in` with the right-aligned dims of `out` (NumPy broadcasting).
void Compiler::UnifyAligned(int out, int in) {
  const ANode &o = nodes_[out], &x = nodes_[in];
  for (int i = 0; i < x.rank; ++i) {
    const int oi = i + o.rank - x.rank;
    if (oi < 0) {
      if (x.dims[i] != 1) Fail("operand rank exceeds result rank");
      continue;
    }
    if (x.dims[i] != 1 && x.dims[i] == o.dims[oi]) Union(Var(out, oi), Var(in, i));
  }
}

void Compiler::UnifyAxes() {
  uf_.resize(static_cast<size_t>(nn_) * kMaxRank);
  for (size_t i = 0; i < uf_.size(); ++i) uf_[i] = static_cast<int>(i);
  std::vector<char> reduced_var(uf_.size(), 0);
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    switch (n.kind) {
      case AK_MEM:
      case AK_SCALAR:
        break;
      case AK_OUT:
        for (int d = 0; d < n.rank; ++d) Union(Var(i, d), Var(n.in[0], d));
        break;
      case AK_REDUCE: {
        const ANode &x = nodes_[n.in[0]];
        bool red[kMaxRank] = {false};
        for (size_t j = 0; j < n.op->aux_ref->size; ++j) {
          int64_t d = n.op->aux_ref->data[j];
          red[d < 0 ? d + x.rank : d] = true;
        }
        int od = 0;
        for (int d = 0; d < x.rank; ++d) {
          if (red[d]) {
            if (x.dims[d] != 1) reduced_var[Var(n.in[0], d)] = 1;
            if (n.op->keepdims) ++od;
          } else {
            Union(Var(i, od), Var(n.in[0], d));
            ++od;
          }
        }
        break;
      }
      case AK_ALIAS:
        if (n.op->kind == kObjReshape || n.op->kind == kObjReduce) {  // dims of extent 1 come and go, the rest keep their order
          const ANode &x = nodes_[n.in[0]];
          int a = 0, b = 0;
          while (true) {
            while (a < x.rank && x.dims[a] == 1) ++a;
            while (b < n.rank && n.dims[b] == 1) ++b;
            if (a == x.rank || b == n.rank) break;
            Union(Var(i, b), Var(n.in[0], a));
            ++a;
            ++b;
          }
        } else {
          UnifyAligned(i, n.in[0]);
        }
        break;
      case AK_OP:
        for (int j = 0; j < n.nin; ++j)
          if (n.in[j] >= 0) UnifyAligned(i, n.in[j]);
        break;
    }
  }
  // Reduces that share a sub-kernel have the same input shape and axes: their inputs walk the
  // same index space even when no operator relates them, so their dims are unified by position.
  {
    int first = -1;
    for (int i = 0; i < nn_; ++i) {
      if (nodes_[i].kind != AK_REDUCE) continue;
      if (first < 0) {
        first = nodes_[i].in[0];
        continue;
      }
      const ANode &x = nodes_[nodes_[i].in[0]], &f = nodes_[first];
      if (x.rank != f.rank) Fail("reduces of different rank in one sub-kernel");
      for (int d = 0; d < x.rank; ++d)
        if (x.dims[d] != 1 && x.dims[d] == f.dims[d]) Union(Var(nodes_[i].in[0], d), Var(first, d));
    }
  }
  // Parts of the sub-kernel that no operator relates to each other (consumers of two different views of one
  // buffer, each with its own store; a copy beside a reduce) walk the same index space too.
  {
    std::vector<int> comp(nn_);
    for (int i = 0; i < nn_; ++i) comp[i] = i;
    auto find = [&](int v) {
      while (comp[v] != v) v = comp[v] = comp[comp[v]];
      return v;
    };
    for (int i = 0; i < nn_; ++i)
      for (int j = 0; j < nodes_[i].nin; ++j)
        if (nodes_[i].in[j] >= 0) comp[find(i)] = find(nodes_[i].in[j]);
    // Each component is matched through its node with the most dims of extent > 1 (an output of a reduce has
    // fewer dims than the walk that produces it); the component of the widest output is the anchor.
    auto wide = [&](int v) {
      int c = 0;
      for (int d = 0; d < nodes_[v].rank; ++d) c += nodes_[v].dims[d] != 1;
      return c;
    };
    std::vector<int> rep(nn_, -1);
    for (int i = 0; i < nn_; ++i) {
      if (nodes_[i].kind == AK_SCALAR) continue;
      int &r = rep[find(i)];
      if (r < 0 || wide(i) > wide(r)) r = i;
    }
    int anchor_out = -1;
    for (int i = 0; i < nn_; ++i)
      if (nodes_[i].kind == AK_OUT && (anchor_out < 0 || wide(rep[find(i)]) > wide(rep[find(anchor_out)]))) anchor_out = i;
    const int anchor = anchor_out < 0 ? -1 : rep[find(anchor_out)];
    for (int c = 0; c < nn_ && anchor >= 0; ++c) {
      if (find(c) != c || rep[c] < 0 || c == find(anchor)) continue;
      const int i = rep[c];
      const ANode &o = nodes_[i], &f = nodes_[anchor];
      // the k-th dim of extent > 1 of the one is the k-th of the other when they list the same extents ...
      int od[kMaxRank], fdm[kMaxRank], no = 0, nf = 0;
      for (int d = 0; d < o.rank; ++d)
        if (o.dims[d] != 1) od[no++] = d;
      for (int d = 0; d < f.rank; ++d)
        if (f.dims[d] != 1) fdm[nf++] = d;
      bool same = no == nf;
      for (int q = 0; q < no && same; ++q) same = o.dims[od[q]] == f.dims[fdm[q]];
      if (same) {
        for (int q = 0; q < no; ++q) Union(Var(i, od[q]), Var(anchor, fdm[q]));
      } else {  // ... else dim by dim from the right, where the extents agree
        for (int d = 0; d < o.rank; ++d) {
          const int fd = d + f.rank - o.rank;
          if (fd >= 0 && o.dims[d] != 1 && o.dims[d] == f.dims[fd]) Union(Var(i, d), Var(anchor, fd));
        }
      }
    }
  }
  // classes with extent > 1 become domain axes
  n_axes_ = 0;
  std::vector<int> axis_of(uf_.size(), -1);
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    for (int d = 0; d < n.rank; ++d) {
      if (n.dims[d] == 1) continue;
      const int root = Find(Var(i, d));
      if (axis_of[root] < 0) {
        if (n_axes_ >= kMaxAxes) Fail("too many axes");
        axis_of[root] = n_axes_;
        axes_[n_axes_].extent = n.dims[d];
        axes_[n_axes_].reduced = false;
        axes_[n_axes_].before = 0;
        ++n_axes_;
      }
      if (axes_[axis_of[root]].extent != n.dims[d]) Fail("inconsistent axis extents");
      n.axis[d] = axis_of[root];
    }
  }
  for (size_t v = 0; v < uf_.size(); ++v) {
    if (!reduced_var[v]) continue;
    const int ax = axis_of[Find(static_cast<int>(v))];
    if (ax >= 0) axes_[ax].reduced = true;
  }
  // every reduce must reduce exactly the reduced axes present in its input
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.kind != AK_REDUCE) continue;
    const ANode &x = nodes_[n.in[0]];
    uint32_t in_axes = 0, out_axes = 0;
    for (int d = 0; d < x.rank; ++d)
      if (x.axis[d] >= 0) in_axes |= 1u << x.axis[d];
    for (int d = 0; d < n.rank; ++d)
      if (n.axis[d] >= 0) out_axes |= 1u << n.axis[d];
    for (int ax = 0; ax < n_axes_; ++ax) {
      const bool in_has = (in_axes >> ax) & 1u, out_has = (out_axes >> ax) & 1u;
      if (in_has && axes_[ax].reduced == out_has) Fail("reduces over different axes in one sub-kernel");
    }
  }
  // no value may have the same axis twice
  for (int i = 0; i < nn_; ++i) {
    uint32_t seen = 0;
    for (int d = 0; d < nodes_[i].rank; ++d) {
      const int ax = nodes_[i].axis[d];
      if (ax < 0) continue;
      if ((seen >> ax) & 1u) Fail("axis used twice by one value");
      seen |= 1u << ax;
    }
  }
}

void Compiler::OrderAndMerge() {
  // order constraints: within a value, an earlier dim is outside a later dim
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    uint32_t outer = 0;
    for (int d = 0; d < n.rank; ++d) {
      if (n.axis[d] < 0) continue;
      axes_[n.axis[d]].before |= outer;
      outer |= 1u << n.axis[d];
    }
  }
  uint32_t placed = 0;
  for (int k = 0; k < n_axes_; ++k) {
    int pick = -1;
    for (int ax = 0; ax < n_axes_; ++ax) {
      if ((placed >> ax) & 1u) continue;
      if ((axes_[ax].before & ~placed) == 0) {
        pick = ax;
        break;
      }
    }
    if (pick < 0) Fail("values disagree on the order of axes");
    order_[k] = pick;
    pos_[pick] = k;
    placed |= 1u << pick;
  }
  // merge neighbours that every memory operand either holds contiguously or lacks
  n_dims_ = 0;
  for (int k = 0; k < n_axes_; ++k) {
    bool merge = false;
    if (k > 0) {
      const int a0 = order_[k - 1], a1 = order_[k];
      merge = axes_[a0].reduced == axes_[a1].reduced;
      for (int i = 0; i < nn_ && merge; ++i) {
        const ANode &n = nodes_[i];
        if (n.kind != AK_MEM && n.kind != AK_OUT) continue;
        int d0 = -1, d1 = -1;
        for (int d = 0; d < n.rank; ++d) {
          if (n.axis[d] == a0) d0 = d;
          if (n.axis[d] == a1) d1 = d;
        }
        if ((d0 < 0) != (d1 < 0)) merge = false;
        if (d0 >= 0 && d1 >= 0) {
          // contiguous only if nothing of extent > 1 lies between them
          for (int d = d0 + 1; d < d1; ++d)
            if (n.dims[d] != 1) merge = false;
          // and, for a strided view, if the outer stride is what a dense walk would have
          if (n.view != nullptr && n.view->vstride_[d0] != n.view->vstride_[d1] * n.dims[d1]) merge = false;
        }
      }
    }
    // device coordinates are 32 bits wide: a tensor of 2^32 elements or more keeps its outer dims apart
    if (merge && dims_[n_dims_ - 1].extent * axes_[order_[k]].extent >= (1ll << 32)) merge = false;
    if (merge) {
      dims_[n_dims_ - 1].extent *= axes_[order_[k]].extent;
      dims_[n_dims_ - 1].last_axis = k;
    } else {
      dims_[n_dims_].extent = axes_[order_[k]].extent;
      dims_[n_dims_].reduced = axes_[order_[k]].reduced;
      dims_[n_dims_].first_axis = dims_[n_dims_].last_axis = k;
      ++n_dims_;
    }
    dim_of_axis_[k] = n_dims_ - 1;
  }
  if (n_dims_ == 0) {  // every extent is 1
    dims_[0].extent = 1;
    dims_[0].reduced = false;
    dims_[0].first_axis = dims_[0].last_axis = -1;
    n_dims_ = 1;
  }
  nk_ = nr_ = n_peel_ = 0;
  for (int d = n_dims_ - 1; d >= 0; --d) {
    if (dims_[d].reduced) {
      if (nr_ >= DVM_VEC_MAXR) Fail("too many reduced dims");
      rlist_[nr_++] = d;
    } else if (nk_ < DVM_VEC_MAXR) {
      klist_[nk_++] = d;
    } else {
      if (n_peel_ >= kMaxPeel) Fail("too many kept dims");
      peel_dim_[n_peel_++] = d;
    }
  }
}

// ---------- schedule and geometry ----------

namespace {
uint32_t Pow2Ceil(uint64_t v) {
  uint32_t p = 1;
  while (p < v) p <<= 1;
  return p;
}
uint32_t Log2(uint32_t v) {
  uint32_t l = 0;
  while ((1u << l) < v) ++l;
  return l;
}
}  // namespace

void Compiler::ChooseSchedule() {
  std::memset(&hdr_, 0, sizeof(hdr_));
  hdr_.entry = VE_VECTOR;
  const int inner = n_dims_ - 1;
  const bool inner_red = dims_[inner].reduced;
  hdr_.inner_extent = static_cast<uint32_t>(dims_[inner].extent);
  hdr_.inner_reduced = inner_red ? 1 : 0;
  const uint64_t inner_groups = (static_cast<uint64_t>(dims_[inner].extent) + E - 1) / E;
  uint64_t n_k = 1, n_r = 1;
  for (int i = 0; i < nk_; ++i) {
    const uint64_t ext = klist_[i] == inner ? inner_groups : static_cast<uint64_t>(dims_[klist_[i]].extent);
    hdr_.kdims[i] = MakeVDim(static_cast<uint32_t>(ext));
    n_k *= ext;
  }
  for (int i = 0; i < nr_; ++i) {
    const uint64_t ext = rlist_[i] == inner ? inner_groups : static_cast<uint64_t>(dims_[rlist_[i]].extent);
    hdr_.rdims[i] = MakeVDim(static_cast<uint32_t>(ext));
    n_r *= ext;
  }
  for (int i = nk_; i < DVM_VEC_MAXR; ++i) hdr_.kdims[i] = MakeVDim(1);
  for (int i = nr_; i < DVM_VEC_MAXR; ++i) hdr_.rdims[i] = MakeVDim(1);
  if (n_k >= (1ull << 31) || n_r >= (1ull << 31)) Fail("index space above 2^31 groups");
  for (int d = 0; d < n_dims_; ++d)
    if (dims_[d].extent >= (1ll << 32)) Fail("axis extent above 2^32");
  hdr_.n_kdim = nk_;
  hdr_.n_rdim = nr_;
  hdr_.n_kidx = static_cast<uint32_t>(n_k);
  hdr_.n_ridx = static_cast<uint32_t>(n_r);
  uint32_t threads = 256;
  single_round_ = true;
  // Slabs per lane per instruction: the wide build of the VM halves the dispatches per element at the price
  // of registers (at most 512 lanes per workgroup, two waves per SIMD). It pays where the instruction stream,
  // not memory, sets the pace: reduces along the innermost axis with long rows.
  // Measured on MI355X it does not pay (batch-norm 98 us against 76, RMSNorm 118 us against 104): two waves per
  // SIMD hide too little latency. Kept as a tuning switch, off by default.
  bool wide = false;
  if (const char *e = std::getenv("DVM_VEC_WIDE")) wide = e[0] == '1' && !(nr_ > 0 && !inner_red);
  u_ = wide ? DVM_VEC_U_WIDE : 2;
  const uint32_t U = static_cast<uint32_t>(u_);
  const uint32_t max_threads = wide ? 512u : 1024u;
  split_inner_ = false;
  if (nr_ == 0) {
    // A gathered operand (innermost stride neither 0 nor 1: a transposing view) is read element by element. In
    // the plain order a workgroup's slabs run along the innermost axis, so of every cache line it fetches it
    // uses 4 bytes, and the workgroups that use the rest run elsewhere, most of them behind another L2. With the
    // innermost axis walked in tiles of 64 elements (8 slabs) and the next axis inside that, a workgroup covers
    // 64 x 64 elements and uses every line it fetches in full:
    // kept dims [8 slabs][the other dims ...][innermost extent / 64].
    static const bool tile_gather = !(std::getenv("DVM_VEC_GATHER_TILE") != nullptr && std::getenv("DVM_VEC_GATHER_TILE")[0] == '0');
    if (tile_gather && nk_ >= 2 && nk_ < DVM_VEC_MAXR && klist_[0] == inner && dims_[inner].extent % (8 * E) == 0) {
      for (int i = 0; i < nn_ && !split_inner_; ++i) {
        const ANode &n = nodes_[i];
        if ((n.kind != AK_MEM && n.kind != AK_OUT) || n.view == nullptr) continue;
        for (int d = 0; d < n.rank; ++d) {
          if (n.axis[d] < 0 || pos_[n.axis[d]] != dims_[inner].last_axis) continue;
          const int64_t st = n.view->vstride_[d];
          if (st != 0 && st != 1) split_inner_ = true;
        }
      }
    }
    if (split_inner_) {
      hdr_.kdims[0] = MakeVDim(8);  // the other dims keep their places, the tiles go behind them
      hdr_.kdims[nk_] = MakeVDim(static_cast<uint32_t>(inner_groups / 8));
      hdr_.n_kdim = nk_ + 1;
    }
    hdr_.sched = VS_POINTWISE;
    if (n_k <= 64 * U) threads = 64;
    else if (n_k <= 128 * U) threads = 128;
    hdr_.n_items = static_cast<uint32_t>((n_k + static_cast<uint64_t>(threads) * U - 1) / (threads * U));
    n_sec_ = 1;
  } else if (inner_red) {
    hdr_.sched = VS_REDX;
    // lanes that share one output: enough to cover the reduce space in one round if possible
    uint32_t team = Pow2Ceil((n_r + U - 1) / U);
    if (team > max_threads) team = max_threads;
    // With many outputs a smaller team per output wins although every output then takes several rounds: the
    // scalar work between the sweeps runs on every wave instead of one wave per workgroup, and no workgroup
    // barrier separates the sweeps. Measured on MI355X, rows of 4096 bf16 (residual add + RMSNorm): 8192 rows
    // 98 us with 256 lanes per row, 83 us with 64; 2048 rows 30 / 28 (128 lanes) / 35 us; 1024 rows 18 / 22 / 30 us.
    // So: about 2^18 lanes in flight, at least one wave per output. DVM_VEC_TEAM caps the team by hand.
    {
      uint32_t cap = std::max<uint32_t>(64, Pow2Ceil((1ull << 18) / std::max<uint64_t>(n_k, 1)));
      if (const char *e = std::getenv("DVM_VEC_TEAM")) {
        const uint32_t c = static_cast<uint32_t>(std::atoi(e));
        if (c >= 1 && (c & (c - 1)) == 0) cap = c;
      }
      if (team > cap) team = cap;
    }
    if (team > 64) {
      hdr_.team_is_block = 1;
      threads = team;
      hdr_.team_log2 = Log2(team);
      hdr_.n_items = static_cast<uint32_t>(n_k);
    } else {
      hdr_.team_is_block = 0;
      hdr_.team_log2 = Log2(team);
      threads = n_k * team >= 256 ? 256 : std::max<uint32_t>(64, Pow2Ceil(n_k * team));
      const uint32_t per_wg = threads / team;
      hdr_.n_items = static_cast<uint32_t>((n_k + per_wg - 1) / per_wg);
    }
    single_round_ = n_r <= static_cast<uint64_t>(team) * U;
  } else {
    hdr_.sched = VS_REDY;
    uint32_t tx = n_k >= 64 ? 64 : Pow2Ceil(n_k);
    uint32_t ty = 256 / tx;
    const uint64_t items = (n_k + tx - 1) / tx;
    if (items < 128 && n_r > 256) ty = max_threads / tx;  // few outputs: give each more lanes along the reduce space
    while (ty > 1 && static_cast<uint64_t>(ty) * U > 2 * n_r) ty >>= 1;
    threads = std::max<uint32_t>(64, tx * ty);
    ty = threads / tx;
    hdr_.team_log2 = Log2(tx);
    hdr_.n_items = static_cast<uint32_t>(items);
    single_round_ = n_r <= static_cast<uint64_t>(ty) * U;
  }
  if (wide) hdr_.sched |= VS_WIDE;

  prog_->threads = threads;
}

// ---------- emission ----------

int Compiler::MemIndex(int v) {
  ANode &n = nodes_[v];
  if (n.mem_idx >= 0) return n.mem_idx;
  if (cube_mode_) return CubeMemIndex(v);
  if (n_mem_ >= DVM_VEC_MAXMEM) Fail("too many memory operands");
  VMemDesc &m = mems_[n_mem_];
  std::memset(&m, 0, sizeof(m));
  m.dtype = MemDType(n.dtype);
  // element stride of every axis the operand has (row-major over its own shape)
  int64_t stride = 1;
  int64_t dim_stride[kMaxAxes];
  bool dim_has[kMaxAxes] = {false};
  for (int d = n.rank - 1; d >= 0; --d) {
    if (n.axis[d] >= 0) {
      const int p = pos_[n.axis[d]];
      const int md = dim_of_axis_[p];
      dim_has[md] = true;
      // the innermost axis of a merged dim carries its stride; a strided view brings its own
      if (p == dims_[md].last_axis) dim_stride[md] = n.view != nullptr ? n.view->vstride_[d] : stride;
    }
    stride *= n.dims[d];
  }
  const int inner = n_dims_ - 1;
  bool aligned = true;
  const int64_t isz = static_cast<int64_t>(DTypeSize(n.dtype));
  const int64_t need = isz * E >= 16 ? 16 : isz * E;
  for (int i = 0; i < nk_; ++i) {
    const int md = klist_[i];
    if (!dim_has[md]) continue;
    if (dim_stride[md] >= (1ll << 32)) Fail("stride above 2^32");
    m.kstride[i] = static_cast<uint32_t>(dim_stride[md]);
    if (md != inner && (dim_stride[md] * isz) % need != 0) aligned = false;
  }
  if (split_inner_ && dim_has[inner]) {  // the tiles of 64 along the innermost axis are the outermost kept dim
    if (dim_stride[inner] * 64 >= (1ll << 32)) Fail("stride above 2^32");
    m.kstride[nk_] = static_cast<uint32_t>(dim_stride[inner] * 64);
  }
  for (int i = 0; i < nr_; ++i) {
    const int md = rlist_[i];
    if (!dim_has[md]) continue;
    if (dim_stride[md] >= (1ll << 32)) Fail("stride above 2^32");
    m.rstride[i] = static_cast<uint32_t>(dim_stride[md]);
    if (md != inner && (dim_stride[md] * isz) % need != 0) aligned = false;
  }
  for (int i = 0; i < n_peel_; ++i) {
    const int md = peel_dim_[i];
    peel_stride_[n_mem_][i] = dim_has[md] ? dim_stride[md] * isz : 0;  // in bytes
    if (peel_stride_[n_mem_][i] % need != 0) aligned = false;
  }
  if (dim_has[inner] && dims_[inner].first_axis >= 0) {
    if (dim_stride[inner] == 1) {
      m.flags |= VMF_VEC;
      if (aligned) m.flags |= VMF_ALIGNED;
    } else if (n.view != nullptr && dim_stride[inner] != 0) {
      // a transposing or element-skipping view: element by element (correct, not fast)
      if (dim_stride[inner] >= (1ll << 24) || dim_stride[inner] < 0) Fail("innermost stride above 2^24");
      m.flags |= VMF_GATHER | (static_cast<uint32_t>(dim_stride[inner]) << 8);
    } else if (dim_stride[inner] != 0) {
      Fail("innermost axis is not contiguous");
    }
  }
  Program::Patch p;
  p.word = static_cast<uint32_t>(sizeof(VVecHeader) / 8 + n_mem_ * (sizeof(VMemDesc) / 8));
  p.op_id = n.addr_op;
  p.ws_slot = n.ws_slot;
  p.byte_offset = n.view != nullptr ? n.view->view_base_ * isz : 0;
  mem_is_view_[n_mem_] = n.view != nullptr;
  p.role = Program::kPatchVecMem;
  prog_->patches.push_back(p);
  n.mem_idx = n_mem_++;
  return n.mem_idx;
}

int Compiler::AllocSReg() {
  for (int i = 0; i < DVM_VEC_NSREG; ++i) {
    if (!((sreg_used_ >> i) & 1u)) {
      sreg_used_ |= 1u << i;
      return i;
    }
  }
  Fail("out of S registers");
  return -1;
}

int Compiler::AllocVSlot(int n) {
  for (int i = 0; i + n <= vslot_limit_; ++i) {
    const uint32_t msk = ((1u << n) - 1u) << i;
    if ((vslot_used_ & msk) == 0) {
      vslot_used_ |= msk;
      max_vslot_ = std::max(max_vslot_, i + n);
      return i;
    }
  }
  Fail("out of V register slots");
  return -1;
}

void Compiler::ReleaseReg(int v) {
  ANode &n = nodes_[v];
  if (n.reg < 0) return;
  if (!n.has_inner) {
    sreg_used_ &= ~(1u << n.reg);
  } else {
    const int cnt = (n.reg_fmt == VF_F32 && !cube_mode_) ? 2 : 1;
    vslot_used_ &= ~(((1u << cnt) - 1u) << n.reg);
  }
  n.reg = -1;
}

void Compiler::SaveAcc(int v) {
  ANode &n = nodes_[v];
  if (n.reg >= 0) return;
  if (!n.has_inner) {
    n.reg = AllocSReg();
    Emit(VOP_STS, 0, 0, 0, n.reg, 0);
  } else if (cube_mode_) {
    // fragment temporaries hold the fp32 container as it is
    n.reg_fmt = VF_F32;
    n.reg = AllocVSlot(1);
    Emit(VOP_STR, 0, 0, 0, n.reg, 0);
  } else {
    n.reg_fmt = n.dtype == kFloat16 ? VF_F16 : (n.dtype == kBFloat16 ? VF_BF16 : VF_F32);
    if (n.dtype == kBool) n.reg_fmt = VF_F16;
    n.reg = AllocVSlot(n.reg_fmt == VF_F32 ? 2 : 1);
    Emit(VOP_STR, n.reg_fmt, 0, 0, n.reg, 0);
  }
}

// Called before an instruction replaces the accumulator by an unrelated value.
void Compiler::BeforeOverwrite() {
  if (acc_node_ < 0) return;
  ANode &n = nodes_[acc_node_];
  if (n.kind == AK_MEM || n.kind == AK_SCALAR) return;  // cheaper to fetch again than to park
  const bool needed_later = n.last_sec > cur_sec_ && (!n.fd || single_round_);
  if ((n.uses > 0 || needed_later) && n.reg < 0) SaveAcc(acc_node_);
}

void Compiler::ConsumeUse(int v) {
  ANode &n = nodes_[v];
  if (n.uses > 0) --n.uses;
  const bool needed_later = n.last_sec > cur_sec_ && (!n.fd || single_round_);
  if (n.uses != 0 || needed_later || n.reg < 0) return;
  // A sweep of several rounds runs its instructions again: a value from an earlier section keeps its
  // register until the sweep ends, or a temporary of round one would replace it before round two reads it.
  if ((cur_sec_ & 1) && !single_round_ && n.sec < cur_sec_) {
    bool listed = false;
    for (int i = 0; i < n_held_; ++i) listed |= held_[i] == v;
    if (!listed) held_[n_held_++] = v;
    return;
  }
  ReleaseReg(v);
}

bool Compiler::SimpleOperand(int v) {
  const ANode &n = nodes_[v];
  if (n.reg >= 0) return true;
  if (acc_node_ == v) return false;
  return n.kind == AK_MEM || n.kind == AK_SCALAR;
}

// acc = acc (op) value-of-v, v being a simple operand.
void Compiler::EmitOperandInsn(uint32_t op, uint32_t sub, uint32_t rnd, int v) {
  ANode &n = nodes_[v];
  if (n.reg >= 0) {
    if (!n.has_inner) {
      Emit(op, sub, VK_SREG, rnd, n.reg, 0);
    } else {
      Emit(op, sub | (static_cast<uint32_t>(n.reg_fmt) << 6), VK_REG, rnd, n.reg, 0);
    }
  } else if (n.kind == AK_MEM) {
    Emit(op, sub, VK_MEM, rnd, MemIndex(v), 0);
  } else if (n.kind == AK_SCALAR) {
    Emit(op, sub, VK_IMM, rnd, 0, ScalarToContainer(n.op->scalar.Get(), n.dtype));
  } else {
    Fail("operand is not addressable");
  }
  ConsumeUse(v);
}

// Puts value v into the accumulator.
void Compiler::EmitValue(int v) {
  v = Resolve(v);
  if (acc_node_ == v) return;
  ANode &n = nodes_[v];
  if (n.reg >= 0) {
    BeforeOverwrite();
    if (!n.has_inner) {
      Emit(VOP_LDS, 0, 0, 0, n.reg, 0);
    } else {
      Emit(VOP_LDR, n.reg_fmt, 0, 0, n.reg, 0);
    }
    acc_node_ = v;
    return;
  }
  ComputeInto(v);
  acc_node_ = v;
}

namespace {
uint32_t BinSubF(int op, bool reversed) {
  switch (op) {
    case kAdd: return VB_ADD;
    case kSub: return reversed ? VB_RSUB : VB_SUB;
    case kMul: return VB_MUL;
    case kDiv: return reversed ? VB_RDIV : VB_DIV;
    case kPow: return reversed ? VB_RPOW : VB_POW;
    case kMaximum: return VB_MAX;
    case kMinimum: return VB_MIN;
    case kLogicalAnd: return VB_AND;
    case kLogicalOr: return VB_OR;
    default: Throw("binary operator without a device form");
  }
}
uint32_t BinSubI(int op, bool reversed) {
  switch (op) {
    case kAdd: return VBI_ADD;
    case kSub: return reversed ? VBI_RSUB : VBI_SUB;
    case kMul: return VBI_MUL;
    case kMaximum: return VBI_MAX;
    case kMinimum: return VBI_MIN;
    default: Throw("binary operator without an int32 form");
  }
}
uint32_t CmpSub(int op, bool reversed, bool is_int) {
  static const uint32_t rev[6] = {VCMP_EQ, VCMP_NE, VCMP_LT, VCMP_LE, VCMP_GT, VCMP_GE};
  uint32_t t = static_cast<uint32_t>(op);  // kEqual..kLessEqual == VCMP_EQ..VCMP_LE
  if (reversed) t = rev[t];
  return t + (is_int ? VCMP_INT : 0);
}
bool NeedsRounding(int op) { return op == kAdd || op == kSub || op == kMul || op == kDiv || op == kPow; }
}  // namespace

// Emits the code that computes v (not in a register, not in the accumulator).
void Compiler::ComputeInto(int v) {
  ANode &n = nodes_[v];
  NDObject *o = n.op;
  // outside the sweeps of a reduce kernel, a value without the innermost axis is one number per lane
  struct UniformScope {
    bool &flag, saved;
    UniformScope(bool &f, bool v) : flag(f), saved(f) { flag = v; }
    ~UniformScope() { flag = saved; }
  } scope(uniform_emit_, !cube_mode_ && nr_ > 0 && (cur_sec_ & 1) == 0 && !n.has_inner && n.kind == AK_OP);
  switch (n.kind) {
    case AK_MEM:
      BeforeOverwrite();
      Emit(VOP_LD, 0, VK_MEM, 0, MemIndex(v), 0);
      return;
    case AK_SCALAR:
      BeforeOverwrite();
      Emit(VOP_LDI, 0, 0, 0, 0, ScalarToContainer(o->scalar.Get(), n.dtype));
      return;
    case AK_REDUCE:
      Fail("reduce result used before it is complete");
      return;
    default:
      break;
  }
  const bool is_int = (o->kind == kObjCompare || o->kind == kObjCompareS || o->kind == kObjBinary ||
                       o->kind == kObjBinaryS || o->kind == kObjUnary)
                          ? o->in[0]->type_id_ == kInt32
                          : false;
  switch (o->kind) {
    case kObjUnary: {
      const int x = Resolve(n.in[0]);
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      uint32_t sub;
      bool rnd = false;
      switch (o->op) {
        case kSqrt: sub = VU_SQRT; rnd = true; break;
        case kAbs: sub = is_int ? VU_IABS : VU_ABS; break;
        case kLog: sub = VU_LOG; rnd = true; break;
        case kExp: sub = VU_EXP; rnd = true; break;
        case kIsFinite: sub = VU_ISFINITE; break;
        case kRound: sub = VU_ROUND; break;
        case kFloor: sub = VU_FLOOR; break;
        case kCeil: sub = VU_CEIL; break;
        case kTrunc: sub = VU_TRUNC; break;
        default: Throw("unary operator without a device form");
      }
      Emit(VOP_UN, sub, 0, rnd ? RndOf(n.dtype) : 0, 0, 0);
      return;
    }
    case kObjCast: {
      const int x = Resolve(n.in[0]);
      const DataType s = o->in[0]->type_id_, d = n.dtype;
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      if (d == kInt32) {
        Emit(VOP_CAST, VC_F2I, 0, 0, 0, 0);
      } else if (s == kInt32) {
        Emit(VOP_CAST, VC_I2F, 0, RndOf(d), 0, 0);
      } else if (d == kBool) {
        Emit(VOP_CAST, VC_F2B, 0, 0, 0, 0);
      } else {
        Emit(VOP_CAST, VC_RND, 0, RndOf(d), 0, 0);
      }
      return;
    }
    case kObjBinaryS:
    case kObjCompareS: {
      const int x = Resolve(n.in[0]);
      EmitValue(x);
      ConsumeUse(x);
      BeforeOverwrite();
      const uint32_t imm = ScalarToContainer(o->scalar.Get(), o->in[0]->type_id_);
      if (o->kind == kObjCompareS) {
        Emit(VOP_CMP, CmpSub(o->op, o->scalar_left, is_int), VK_IMM, 0, 0, imm);
      } else if (is_int) {
        Emit(VOP_BINI, BinSubI(o->op, o->scalar_left), VK_IMM, 0, 0, imm);
      } else {
        Emit(VOP_BINF, BinSubF(o->op, o->scalar_left), VK_IMM, NeedsRounding(o->op) ? RndOf(n.dtype) : 0, 0, imm);
      }
      return;
    }
    case kObjBinary:
    case kObjCompare: {
      int a = Resolve(n.in[0]), b = Resolve(n.in[1]);
      bool reversed = false;
      uint32_t opc, sub, rnd = 0;
      auto pick = [&](bool rev) {
        if (o->kind == kObjCompare) {
          opc = VOP_CMP;
          sub = CmpSub(o->op, rev, is_int);
        } else if (is_int) {
          opc = VOP_BINI;
          sub = BinSubI(o->op, rev);
        } else {
          opc = VOP_BINF;
          sub = BinSubF(o->op, rev);
          rnd = NeedsRounding(o->op) ? RndOf(n.dtype) : 0;
        }
      };
      if (a == b) {
        EmitValue(a);
        ConsumeUse(a);
        ConsumeUse(a);
        BeforeOverwrite();
        pick(false);
        Emit(opc, sub, VK_ACC, rnd, 0, 0);
        return;
      }
      if (acc_node_ == b) {
        std::swap(a, b);
        reversed = true;
      }
      if (acc_node_ == a) {
        if (!SimpleOperand(b)) {
          // computing b would clobber a: park a, compute b, then use a as the operand
          SaveAcc(a);
          EmitValue(b);
          std::swap(a, b);
          reversed = !reversed;
        }
      } else if (SimpleOperand(b)) {
        EmitValue(a);
      } else if (SimpleOperand(a)) {
        EmitValue(b);
        std::swap(a, b);
        reversed = true;
      } else {
        EmitValue(b);
        if (SimpleOperand(a)) {
          // a was computed and parked on the way to b (b is a function of a, as in x / (exp(-x) + 1))
          std::swap(a, b);
          reversed = true;
        } else {
          SaveAcc(b);
          EmitValue(a);
        }
      }
      ConsumeUse(a);
      BeforeOverwrite();
      pick(reversed);
      EmitOperandInsn(opc, sub, rnd, b);
      return;
    }
    case kObjSelect: {
      const int c = Resolve(n.in[0]), x = Resolve(n.in[1]), y = Resolve(n.in[2]);
      if (!SimpleOperand(c)) {
        EmitValue(c);
        SaveAcc(c);
      }
      if (!SimpleOperand(x)) {
        EmitValue(x);
        SaveAcc(x);
      }
      EmitValue(y);
      ConsumeUse(y);
      BeforeOverwrite();
      EmitOperandInsn(VOP_MSK, 0, 0, c);
      EmitOperandInsn(VOP_MOVM, 0, 0, x);
      return;
    }
    default:
      Fail("operator without a vector form");
  }
}

// Counts, for the section being emitted, how often each value of the cone is read.
void Compiler::CountCone(int v) {
  v = Resolve(v);
  ANode &n = nodes_[v];
  ++n.uses;
  if (n.in_cone) return;
  n.in_cone = true;
  if (n.reg >= 0 || n.kind == AK_MEM || n.kind == AK_SCALAR || n.kind == AK_REDUCE) return;
  for (int j = 0; j < n.nin; ++j)
    if (n.in[j] >= 0) CountCone(n.in[j]);
}

void Compiler::EmitSection(int sec) {
  cur_sec_ = sec;
  last_mem_ = -1;
  const bool sweep = (sec & 1) != 0;
  for (int i = 0; i < nn_; ++i) {
    nodes_[i].uses = 0;
    nodes_[i].in_cone = false;
  }
  if (!sweep && sec > 0) {
    // results of the previous sweep's reduces become register values
    for (int i = 0; i < nn_; ++i) {
      ANode &n = nodes_[i];
      if (n.kind != AK_REDUCE || n.sec != sec - 1) continue;
      BeforeOverwrite();
      Emit(VOP_FIN, n.dtype == kInt32 ? VRF_INT : 0, 0, 0, n.reg_fmt, 0);
      acc_node_ = i;
      SaveAcc(i);
    }
  }
  // sinks of this section, in node order
  int sinks[kMaxNodes];
  int ns = 0;
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if ((n.kind == AK_REDUCE || n.kind == AK_OUT) && n.sec == sec) sinks[ns++] = i;
  }
  // values computed here that a later section reads from a register
  int keep[kMaxNodes];
  int nkp = 0;
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.sec != sec || n.last_sec <= sec) continue;
    if (n.kind == AK_MEM) {
      // an operand that does not vary inside the sweeps is loaded once per output into an S register
      if (sweep || n.has_inner || n_sec_ == 1) continue;
      if (__builtin_popcount(sreg_used_) >= DVM_VEC_NSREG - 3) continue;
      keep[nkp++] = i;
      continue;
    }
    if (n.kind != AK_OP) continue;
    if (n.fd && !single_round_) continue;  // recomputed by the later sweep
    keep[nkp++] = i;
  }
  if (sweep) {
    uint32_t kinds = 0xff;
    int slot = 0;
    for (int i = 0; i < ns; ++i) {
      ANode &n = nodes_[sinks[i]];
      if (n.kind != AK_REDUCE) continue;
      if (slot >= DVM_VEC_NSLOT) Fail("more than two reduces in one sweep");
      const uint32_t rk = n.op->op == kSum ? VR_SUM : (n.op->op == kMax ? VR_MAX : VR_MIN);
      kinds = (kinds & ~(0xfu << (4 * slot))) | (rk << (4 * slot));
      n.reg_fmt = static_cast<uint8_t>(slot);  // slot number until the result is fetched
      ++slot;
    }
    BeforeOverwrite();
    Emit(VOP_SWEEP, 0, 0, 0, 0, kinds);
    if (!single_round_) acc_node_ = -1;
  }
  for (int i = 0; i < ns; ++i) CountCone(nodes_[sinks[i]].in[0]);
  for (int i = 0; i < nkp; ++i) CountCone(keep[i]);
  for (int i = 0; i < ns; ++i) {
    ANode &n = nodes_[sinks[i]];
    const int x = Resolve(n.in[0]);
    EmitValue(x);
    if (n.kind == AK_REDUCE) {
      const uint32_t rk = n.op->op == kSum ? VR_SUM : (n.op->op == kMax ? VR_MAX : VR_MIN);
      Emit(VOP_RED, rk | (n.dtype == kInt32 ? VRF_INT : 0), 0, 0, n.reg_fmt, 0);
    } else {
      Emit(VOP_ST, 0, 0, 0, MemIndex(sinks[i]), 0);
    }
    ConsumeUse(x);
  }
  for (int i = 0; i < nkp; ++i) {
    const int v = keep[i];
    if (nodes_[v].reg < 0) {
      EmitValue(v);
      SaveAcc(v);
    }
    ConsumeUse(v);
  }
  if (sweep) {
    if (!single_round_) BeforeOverwrite();
    Emit(VOP_ENDSWEEP, 0, 0, 0, 0, 0);
    if (!single_round_) acc_node_ = -1;
  }
  for (int i = 0; i < n_held_; ++i)
    if (nodes_[held_[i]].uses == 0) ReleaseReg(held_[i]);
  n_held_ = 0;
}

void Compiler::EmitProgram() {
  const int inner = n_dims_ - 1;
  const int inner_first = dims_[inner].first_axis, inner_last = dims_[inner].last_axis;
  // classify values
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    n.has_inner = false;
    n.fd = false;
    for (int d = 0; d < n.rank; ++d) {
      if (n.axis[d] < 0) continue;
      const int p = pos_[n.axis[d]];
      if (inner_first >= 0 && p >= inner_first && p <= inner_last) n.has_inner = true;
      if (axes_[n.axis[d]].reduced) n.fd = true;
    }
    // Only a value that is the same for every slab of a lane fits an S register: slabs differ in
    // the kept position (pointwise) or in the reduce position (sweeps).
    if (n.fd || nr_ == 0) n.has_inner = true;
  }
  int max_level = 0;
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    n.level = 0;
    for (int j = 0; j < n.nin; ++j) {
      if (n.in[j] < 0) continue;
      const ANode &x = nodes_[n.in[j]];
      n.level = std::max(n.level, x.level + (x.kind == AK_REDUCE ? 1 : 0));
    }
    if (n.kind == AK_REDUCE) {
      // the reduce runs in the sweep of its input's level
      n.sec = 2 * n.level + 1;
    } else if (nr_ == 0) {
      n.sec = 0;
    } else {
      n.sec = 2 * n.level + (n.fd ? 1 : 0);
    }
    max_level = std::max(max_level, n.level);
  }
  // aliases inherit the class of what they resolve to
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    if (n.kind == AK_ALIAS) {
      const ANode &r = nodes_[Resolve(i)];
      n.sec = r.sec;
    }
  }
  // an output's section is that of the value it stores
  n_sec_ = nr_ == 0 ? 1 : 2 * (max_level + 1);
  for (int i = 0; i < nn_; ++i) nodes_[i].last_sec = -1;
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    if (n.kind == AK_ALIAS) continue;
    const int my_sec = n.sec;
    for (int j = 0; j < n.nin; ++j) {
      if (n.in[j] < 0) continue;
      ANode &x = nodes_[Resolve(n.in[j])];
      x.last_sec = std::max(x.last_sec, my_sec);
    }
  }
  // values recomputed by a later sweep pull their own inputs forward
  if (!single_round_) {
    for (int pass = 0; pass < nn_; ++pass) {
      bool changed = false;
      for (int i = nn_ - 1; i >= 0; --i) {
        ANode &n = nodes_[i];
        if (n.kind != AK_OP || !n.fd) continue;
        for (int j = 0; j < n.nin; ++j) {
          if (n.in[j] < 0) continue;
          ANode &x = nodes_[Resolve(n.in[j])];
          if (x.last_sec < n.last_sec) {
            x.last_sec = n.last_sec;
            changed = true;
          }
        }
      }
      if (!changed) break;
    }
  }
  // local memory budget for V registers
  const uint32_t per_slot = static_cast<uint32_t>(u_) * 16u * prog_->threads;
  const uint32_t budget = g_system.lds_per_wg > 80 * 1024 ? 72 * 1024 : g_system.lds_per_wg - 8 * 1024;
  vslot_limit_ = std::min<int>(DVM_VEC_NREG, static_cast<int>(budget / per_slot));
  sreg_used_ = vslot_used_ = 0;
  max_vslot_ = 0;
  acc_node_ = -1;
  code_.clear();
  n_mem_ = 0;
  for (int s = 0; s < n_sec_; ++s) EmitSection(s);
  Emit(VOP_END, 0, 0, 0, 0, 0);
}


// A rounding cast to fp16 / bf16 whose only reader is the store right behind it does nothing the store's own
// conversion does not do (same round to nearest even): the cast instruction is dropped. `mem_dtypes[i]` is the
// element type of memory operand i.
void Compiler::DropCastBeforeStore(const uint32_t *mem_dtypes) {
  std::vector<uint64_t> out;
  out.reserve(code_.size());
  for (size_t i = 0; i < code_.size(); ++i) {
    const uint64_t w = code_[i];
    if (VI_OP(w) == VOP_CAST && VI_SUB(w) == VC_RND && !(static_cast<uint32_t>(w) & VI_UNIFORM) && i + 2 < code_.size() + 1 && i + 1 < code_.size()) {
      const uint64_t st = code_[i + 1];
      const uint32_t next = i + 2 < code_.size() ? VI_OP(code_[i + 2]) : static_cast<uint32_t>(VOP_END);
      const bool acc_dead = next == VOP_END || next == VOP_ENDSWEEP || next == VOP_SWEEP || next == VOP_LD || next == VOP_LDR ||
                            next == VOP_LDS || next == VOP_LDI || next == VOP_FIN;
      if (VI_OP(st) == VOP_ST && acc_dead) {
        const uint32_t dt = mem_dtypes[VI_A(st)];
        if ((VI_RND(w) == VRND_F16 && dt == VDT_F16) || (VI_RND(w) == VRND_BF16 && dt == VDT_BF16)) continue;
      }
    }
    out.push_back(w);
  }
  code_.swap(out);
}

// The interpreter pays a fixed price per instruction, so the short bodies of sweeps are tightened:
//  * sum(x) and sum(x * x) of one value (mean and variance in one pass): the multiply joins the second reduce;
//  * two float binaries in a row with S-register operands (x * scale + shift) become one chained instruction;
//  * the VOP_ENDSWEEP behind a store or a reduce becomes a flag of that instruction.
// Every fused form computes what the separate instructions compute, rounding by rounding.
void Compiler::FuseSweepInstructions() {
  auto defines_acc = [](uint32_t op) {
    return op == VOP_LD || op == VOP_LDR || op == VOP_LDS || op == VOP_LDI || op == VOP_FIN || op == VOP_END;
  };
  std::vector<uint64_t> out;
  out.reserve(code_.size());
  size_t sweep_first = 0;  // index in code_ of the first instruction of the sweep being copied
  for (size_t i = 0; i < code_.size(); ++i) {
    const uint64_t w = code_[i];
    const uint32_t lo = static_cast<uint32_t>(w);
    if (VI_OP(w) == VOP_SWEEP) sweep_first = i + 1;
    // Mul acc, acc ; reduce_sum rB, acc ; endsweep   (acc dead afterwards)  ->  reduce_sum.square rB, acc
    if (VI_OP(w) == VOP_BINF && (VI_SUB(w) & 0x3fu) == VB_MUL && VI_KIND(w) == VK_ACC && VI_RND(w) == VRND_NONE &&
        !(lo & VI_UNIFORM) && i + 2 < code_.size() && VI_OP(code_[i + 1]) == VOP_RED && VI_SUB(code_[i + 1]) == VR_SUM &&
        VI_OP(code_[i + 2]) == VOP_ENDSWEEP && i + 3 < code_.size() && defines_acc(VI_OP(code_[i + 3])) &&
        sweep_first < code_.size() && defines_acc(VI_OP(code_[sweep_first])) && sweep_first <= i) {
      out.push_back(code_[i + 1] | (static_cast<uint64_t>(VRF_SQUARE) << 8));
      ++i;
      continue;
    }
    // two S-register float binaries in a row
    if (VI_OP(w) == VOP_BINF && VI_KIND(w) == VK_SREG && !(lo & VI_UNIFORM) && i + 1 < code_.size()) {
      const uint64_t n = code_[i + 1];
      if (VI_OP(n) == VOP_BINF && VI_KIND(n) == VK_SREG && !(static_cast<uint32_t>(n) & VI_UNIFORM)) {
        const uint32_t second = (VI_SUB(n) & 0x3fu) | (VI_A(n) << 8) | (VI_RND(n) << 16);
        out.push_back(VI_MAKE(VOP_BINF, VI_SUB(w), VK_SREG2, VI_RND(w), VI_A(w), second));
        ++i;
        continue;
      }
    }
    out.push_back(w);
  }
  // store / reduce ; endsweep  ->  one instruction that also closes the round; a sweep with nothing in it goes
  code_.clear();
  for (size_t i = 0; i < out.size(); ++i) {
    uint64_t w = out[i];
    if (VI_OP(w) == VOP_SWEEP && (VI_IMM(w) & 0xffu) == (VR_NONE | (VR_NONE << 4)) && i + 1 < out.size() &&
        VI_OP(out[i + 1]) == VOP_ENDSWEEP) {
      ++i;
      continue;
    }
    if (i + 1 < out.size() && VI_OP(out[i + 1]) == VOP_ENDSWEEP) {
      if (VI_OP(w) == VOP_ST) {
        code_.push_back(w | VI_ENDS);
        ++i;
        continue;
      }
      if (VI_OP(w) == VOP_RED) {
        code_.push_back(w | VI_ENDS);
        ++i;
        continue;
      }
    }
    code_.push_back(w);
  }
}

// Between sweeps a program computes per-output values (a mean, a scale): the same in every lane of the team
// that owns the output. When the team is the whole workgroup, such a run is executed by one wave, which hands
// the S registers and the accumulator to the others (VOP_UNI_BEGIN / VOP_UNI_END); sixteen waves interpreting
// the same twenty scalar instructions cost more than the two barriers.
void Compiler::MarkUniformRuns() {
  if ((hdr_.sched & VS_KIND_MASK) != VS_REDX || !hdr_.team_is_block) return;
  auto bcast_load = [&](uint64_t w) {
    return VI_OP(w) == VOP_LD && VI_KIND(w) == VK_MEM && !(mems_[VI_A(w)].flags & (VMF_VEC | VMF_GATHER)) && !mem_is_view_[VI_A(w)];
  };
  auto starts = [&](uint64_t w) {
    const uint32_t op = VI_OP(w);
    return op == VOP_FIN || op == VOP_LDS || op == VOP_LDI || bcast_load(w);
  };
  auto inside = [&](uint64_t w) {
    const uint32_t op = VI_OP(w);
    if (starts(w) || op == VOP_STS) return true;
    const bool arith = op == VOP_UN || op == VOP_CAST || op == VOP_BINF || op == VOP_BINI || op == VOP_CMP;
    return arith && (static_cast<uint32_t>(w) & VI_UNIFORM) != 0;
  };
  std::vector<uint64_t> out;
  out.reserve(code_.size() + 8);
  bool in_sweep = false;
  for (size_t i = 0; i < code_.size();) {
    const uint64_t w = code_[i];
    const uint32_t op = VI_OP(w);
    if (op == VOP_SWEEP) in_sweep = true;
    if (static_cast<uint32_t>(w) & VI_ENDS) {
      in_sweep = false;
    }
    if (!in_sweep && starts(w)) {
      size_t j = i;
      while (j < code_.size() && inside(code_[j])) ++j;
      if (j - i >= 4) {
        out.push_back(VI_MAKE(VOP_UNI_BEGIN, 0, 0, 0, 0, static_cast<uint32_t>(j - i + 1)));
        out.insert(out.end(), code_.begin() + i, code_.begin() + j);
        out.push_back(VI_MAKE(VOP_UNI_END, 0, 0, 0, 0, 0));
        i = j;
        continue;
      }
    }
    out.push_back(w);
    ++i;
  }
  code_.swap(out);
}

// A reduce with consumers reads its input twice: once for the statistics, once to apply them. What the
// second sweep does not have to fetch again from HBM:
//  * the first rounds of the first sweep stay in the workgroup's spare local memory (VI_LD_KEEP_WR/RD);
//  * a later sweep without reduces of its own runs last round first (VSW_REVERSE), starting with the data the
//    L2 cache still holds from the end of the sweep before, and ending with the parked rounds.
// Called with the blob filled in and lds_bytes set; edits the instruction words in the blob.
void Compiler::PlanRereads() {
  // tuning switch DVM_VEC_REREAD: 0 off, 2 parked rounds only, 3 reversed sweeps only (default: both)
  static const char mode = std::getenv("DVM_VEC_REREAD") != nullptr ? std::getenv("DVM_VEC_REREAD")[0] : '1';
  const bool on = mode != '0', park = mode != '3', reverse = mode != '2';
  if (!on || (hdr_.sched & VS_KIND_MASK) != VS_REDX || (hdr_.sched & VS_WIDE)) return;
  uint64_t *cw = prog_->blob.w + hdr_.code_off;
  const size_t n = code_.size();
  const uint32_t team = hdr_.team_is_block ? prog_->threads : (1u << hdr_.team_log2);
  const uint32_t per_round = team * u_;
  const uint32_t n_rounds = (hdr_.n_ridx + per_round - 1) / per_round;
  if (n_rounds < 2) return;
  // sweeps: position of the VOP_SWEEP word and of the load that opens it (or -1)
  struct Sw { size_t at; int ld; bool reduces; };
  std::vector<Sw> sweeps;
  for (size_t i = 0; i < n; ++i) {
    if (VI_OP(cw[i]) != VOP_SWEEP) continue;
    Sw sw{i, -1, (VI_IMM(cw[i]) & 0xffu) != (VR_NONE | (VR_NONE << 4))};
    if (i + 1 < n && VI_OP(cw[i + 1]) == VOP_LD && VI_KIND(cw[i + 1]) == VK_MEM && (mems_[VI_A(cw[i + 1])].flags & VMF_VEC)) {
      sw.ld = static_cast<int>(i + 1);
    }
    sweeps.push_back(sw);
  }
  for (size_t k = 1; k < sweeps.size(); ++k) {
    if (reverse && !sweeps[k].reduces) cw[sweeps[k].at] |= static_cast<uint64_t>(VSW_REVERSE) << 8;
  }
  // park rounds of the first pair of sweeps that open with a load of the same operand
  if (!park) return;
  for (size_t a = 0; a + 1 < sweeps.size(); ++a) {
    if (sweeps[a].ld < 0) continue;
    for (size_t b = a + 1; b < sweeps.size(); ++b) {
      if (sweeps[b].ld < 0 || VI_A(cw[sweeps[b].ld]) != VI_A(cw[sweeps[a].ld])) continue;
      // local memory left to this workgroup when as many workgroups as the registers allow share the CU
      const uint32_t per_cu = 1024 / std::max<uint32_t>(prog_->threads, 64);
      const uint32_t budget = std::min<uint32_t>(160 * 1024, g_system.lds_per_wg) / per_cu;
      const uint32_t fixed = prog_->lds_bytes + DVM_PARAM_BYTES + 1024;
      const uint32_t per_keep = prog_->threads * u_ * 32;
      if (budget <= fixed + per_keep) return;
      const uint32_t rounds = std::min<uint32_t>(n_rounds, (budget - fixed) / per_keep);
      cw[sweeps[a].ld] |= VI_LD_KEEP_WR | (static_cast<uint64_t>(rounds) << 32);
      cw[sweeps[b].ld] |= VI_LD_KEEP_RD | (static_cast<uint64_t>(rounds) << 32);
      prog_->lds_bytes += rounds * per_keep;
      return;
    }
  }
}

void Compiler::FinishProgram() {
  {
    uint32_t dts[DVM_VEC_MAXMEM];
    for (int i = 0; i < n_mem_; ++i) dts[i] = mems_[i].dtype;
    DropCastBeforeStore(dts);
  }
  // tuning switches: DVM_VEC_FUSE=0 keeps the instruction stream as emitted, DVM_VEC_UNIRUN=0 lets every wave
  // execute the per-team runs
  static const bool fuse = !(std::getenv("DVM_VEC_FUSE") != nullptr && std::getenv("DVM_VEC_FUSE")[0] == '0');
  static const bool unirun = !(std::getenv("DVM_VEC_UNIRUN") != nullptr && std::getenv("DVM_VEC_UNIRUN")[0] == '0');
  if (fuse && (hdr_.sched & VS_KIND_MASK) != VS_POINTWISE) FuseSweepInstructions();
  if (unirun) MarkUniformRuns();
  hdr_.n_mem = n_mem_;
  hdr_.n_code = static_cast<uint32_t>(code_.size());
  hdr_.mem_off = sizeof(VVecHeader) / 8;
  hdr_.code_off = hdr_.mem_off + n_mem_ * (sizeof(VMemDesc) / 8);
  hdr_.n_vslot = max_vslot_;
  if (hdr_.code_off + code_.size() > DVM_PARAM_WORDS) Fail("program larger than 4 KB");
  std::memset(&prog_->blob, 0, sizeof(VmParam));
  std::memcpy(prog_->blob.w, &hdr_, sizeof(hdr_));
  std::memcpy(prog_->blob.w + hdr_.mem_off, mems_, sizeof(VMemDesc) * n_mem_);
  std::memcpy(prog_->blob.w + hdr_.code_off, code_.data(), 8 * code_.size());
  prog_->lds_bytes = prog_->threads * 8 + static_cast<uint32_t>(max_vslot_) * u_ * 16 * prog_->threads;
  PlanRereads();
  uint64_t gt = (static_cast<uint64_t>(std::min<uint32_t>(hdr_.n_items, g_system.core_num * 4)) << 32) | prog_->threads;
  if (g_system.HasDevice()) {
    gt = g_system.Api().select_block_thread(hdr_.sched, hdr_.n_items, prog_->threads, prog_->lds_bytes);
  }
  prog_->grid = static_cast<uint32_t>(gt >> 32);
  if (prog_->grid == 0) prog_->grid = 1;
}

void Compiler::CompileArea(int a) {
  cur_area_ = a;
  k_->programs_.emplace_back();
  prog_ = &k_->programs_.back();
  cube_mode_ = false;
  if (areas_[a].attn >= 0) {
    CompileAttn(areas_[a].attn);
    return;
  }
  if (areas_[a].cube) {
    CompileCube(a);
    return;
  }
  BuildNodes(a);
  if (nn_ == 0) {  // only stores that other launches have already served
    prog_->skip = true;
    return;
  }
  // an empty domain: nothing to run, outputs that still have elements are zero-filled
  bool empty = false;
  for (int i = 0; i < nn_; ++i) {
    int64_t n = 1;
    for (int d = 0; d < nodes_[i].rank; ++d) n *= nodes_[i].dims[d];
    if (n == 0) empty = true;
  }
  if (empty) {
    prog_->skip = true;
    for (int i = 0; i < nn_; ++i) {
      const ANode &n = nodes_[i];
      if (n.kind != AK_OUT) continue;
      int64_t cnt = 1;
      for (int d = 0; d < n.rank; ++d) cnt *= n.dims[d];
      if (cnt == 0) continue;
      Program::Fill f;
      f.op_id = n.addr_op;
      f.ws_slot = n.ws_slot;
      f.value = 0;
      f.bytes = (static_cast<size_t>(cnt) * DTypeSize(n.dtype) + 3) & ~static_cast<size_t>(3);
      prog_->fills.push_back(f);
    }
    return;
  }
  UnifyAxes();
  OrderAndMerge();
  ChooseSchedule();
  // a stored value must span the index space it is stored from, or it would be written several times
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.kind != AK_OUT) continue;
    uint32_t have = 0;
    bool fd = false;
    for (int d = 0; d < n.rank; ++d) {
      if (n.axis[d] < 0) continue;
      have |= 1u << n.axis[d];
      if (axes_[n.axis[d]].reduced) fd = true;
    }
    for (int ax = 0; ax < n_axes_; ++ax) {
      if ((have >> ax) & 1u) continue;
      if (!axes_[ax].reduced || fd) Fail("output smaller than the kernel domain");
    }
  }
  EmitProgram();
  FinishProgram();
  if (n_peel_ > 0) ReplicatePeeled();
}

// One copy of the finished program per index of the peeled dims; patches are in operand order, one per VMemDesc.
void Compiler::ReplicatePeeled() {
  int64_t count = 1;
  for (int i = 0; i < n_peel_; ++i) count *= dims_[peel_dim_[i]].extent;
  if (count > 4096) Fail("too many kept dims");
  const Program base = *prog_;
  k_->programs_.pop_back();
  for (int64_t c = 0; c < count; ++c) {
    k_->programs_.push_back(base);
    Program &p = k_->programs_.back();
    if (c > 0) p.fills.clear();
    int64_t rest = c;
    for (int i = 0; i < n_peel_; ++i) {
      const int64_t ext = dims_[peel_dim_[i]].extent;
      const int64_t idx = rest % ext;
      rest /= ext;
      for (size_t m = 0; m < p.patches.size(); ++m) {
        p.patches[m].byte_offset += idx * peel_stride_[m][i];
      }
    }
  }
  prog_ = &k_->programs_.back();
}


// ---------- matmul sub-kernels ----------
//
// The matmul's operands are read from memory by the MFMA tile loop; every other operator of the
// sub-kernel has the matmul's output shape and becomes the epilogue program, emitted with the same
// accumulator-machine rules as a pointwise kernel whose accumulator starts out holding the product.

int Compiler::CubeMemIndex(int v) {
  ANode &n = nodes_[v];
  if (n_mem_ >= DVM_CUBE_MAXMEM) Fail("too many memory operands in a matmul epilogue");
  VCubeMem &m = cmems_[n_mem_];
  std::memset(&m, 0, sizeof(m));
  m.dtype = MemDType(n.dtype);
  const int R = cube_out_->rank();
  int64_t stride = 1;
  for (int d = n.rank - 1; d >= 0; --d) {
    const int od = d + R - n.rank;
    if (n.dims[d] != 1) {
      if (od < 0 || n.dims[d] != cube_out_->dim(od)) Fail("epilogue operand does not broadcast to the matmul result");
      const int64_t walk = n.view != nullptr ? n.view->vstride_[d] : stride;
      if (walk >= (1ll << 32) || walk < 0) Fail("stride above 2^32");
      const uint32_t st = static_cast<uint32_t>(walk);
      if (od == R - 1 && st != 1) Throw("DVM EXCEPTION. reason: a strided view whose innermost stride is not 1 is not supported by the gfx950 backend");
      if (od == R - 1) m.stride_n = st;
      else if (od == R - 2) m.stride_m = st;
      else if (od == R - 3) m.stride_b1 = st;
      else m.stride_b0 = st;
    }
    stride *= n.dims[d];
  }
  Program::Patch p;
  p.word = static_cast<uint32_t>(sizeof(VCubeHeader) / 8 + n_mem_ * (sizeof(VCubeMem) / 8));
  p.op_id = n.addr_op;
  p.ws_slot = n.ws_slot;
  p.byte_offset = n.view != nullptr ? n.view->view_base_ * static_cast<int64_t>(DTypeSize(n.dtype)) : 0;
  p.role = Program::kPatchPlain;
  prog_->patches.push_back(p);
  n.mem_idx = n_mem_++;
  return n.mem_idx;
}

void Compiler::CompileCube(int a) {
  cube_mode_ = true;
  BuildNodes(a);
  int c = -1;
  for (int i = 0; i < nn_; ++i)
    if (nodes_[i].kind == AK_OP && nodes_[i].op->kind == kObjMatMul) c = i;
  if (c < 0) Fail("matmul sub-kernel without a matmul");
  NDObject *mm = nodes_[c].op;
  cube_out_ = mm;
  const ANode &an = nodes_[nodes_[c].in[0]], &bn = nodes_[nodes_[c].in[1]];
  if (an.kind != AK_MEM || bn.kind != AK_MEM) Fail("matmul operands must come from memory");
  if (an.dtype != bn.dtype || (an.dtype != kFloat16 && an.dtype != kBFloat16)) Fail("matmul operands must both be fp16 or both bf16");
  const int R = mm->rank();
  const int br = R - 2;
  if (br > 2) Fail("matmul with more than two batch dimensions");
  VCubeHeader h;
  std::memset(&h, 0, sizeof(h));
  h.entry = VE_CUBE;
  h.dtype = MemDType(an.dtype);
  const int64_t M = mm->dim(R - 2), N = mm->dim(R - 1);
  const int64_t K = mm->trans_a ? an.dims[an.rank - 2] : an.dims[an.rank - 1];
  if (M >= (1ll << 31) || N >= (1ll << 31) || K >= (1ll << 31)) Fail("matmul extent above 2^31");
  h.m = static_cast<uint32_t>(M);
  h.n = static_cast<uint32_t>(N);
  h.k = static_cast<uint32_t>(K);
  h.trans_a = mm->trans_a ? 1 : 0;
  h.trans_b = mm->trans_b ? 1 : 0;
  h.lda = static_cast<uint32_t>(an.dims[an.rank - 1]);
  h.ldb = static_cast<uint32_t>(bn.dims[bn.rank - 1]);
  h.nb0 = br == 2 ? static_cast<uint32_t>(mm->dim(0)) : 1;
  h.nb1 = br >= 1 ? static_cast<uint32_t>(mm->dim(br - 1)) : 1;
  auto batch_strides = [&](const ANode &x, uint32_t *s0, uint32_t *s1) {
    *s0 = *s1 = 0;
    int64_t stride = x.dims[x.rank - 1] * x.dims[x.rank - 2];
    for (int d = x.rank - 3; d >= 0; --d) {
      const int od = d + R - x.rank;
      if (x.dims[d] != 1) {
        if (stride >= (1ll << 32)) Fail("stride above 2^32");
        if (od == R - 3) *s1 = static_cast<uint32_t>(stride);
        else *s0 = static_cast<uint32_t>(stride);
      }
      stride *= x.dims[d];
    }
  };
  batch_strides(an, &h.a_sb0, &h.a_sb1);
  batch_strides(bn, &h.b_sb0, &h.b_sb1);
  if (M == 0 || N == 0 || h.nb0 == 0 || h.nb1 == 0) {
    prog_->skip = true;
    return;
  }
  // block tile: the largest that still gives most compute units a tile
  const uint64_t batch = static_cast<uint64_t>(h.nb0) * h.nb1;
  auto tiles = [&](int64_t t) { return static_cast<uint64_t>((M + t - 1) / t) * static_cast<uint64_t>((N + t - 1) / t) * batch; };
  const uint64_t cus = g_system.core_num;
  int64_t bt;
  if (tiles(256) * 4 >= cus * 3) {
    h.tile = 0;
    bt = 256;
  } else if (tiles(128) * 2 >= cus) {
    h.tile = 1;
    bt = 128;
  } else {
    h.tile = 2;
    bt = 64;
  }
  if (const char *e = std::getenv("DVM_CUBE_TILE")) {  // tuning override: 256, 128 or 64
    const int v = std::atoi(e);
    if (v == 256 || v == 128 || v == 64) {
      bt = v;
      h.tile = v == 256 ? 0 : (v == 128 ? 1 : 2);
    }
  }
  // The 256x256 tile also exists on eight waves (two per SIMD, 64x128 accumulators each): the second wave hides
  // most of the epilogue and of the fragment-read latency, at 1.5 times the local-memory traffic per flop.
  // Measured on MI355X, 8192x4096x4096 bf16: both operands k-contiguous 289 -> 283 us (with bias + SiLU
  // 369 -> 354 us, k = 512: 81 -> 70 us); with a k-strided operand, whose tiles pass through registers, the four
  // waves stay ahead (286 us against 324 us). DVM_CUBE_WAVES=4 / 8 forces either.
  if (h.tile == 0) {
    bool eight = !h.trans_a && h.trans_b;
    if (const char *e = std::getenv("DVM_CUBE_WAVES")) {
      if (std::atoi(e) == 8) eight = true;
      if (std::atoi(e) == 4) eight = false;
    }
    if (eight) h.tile = 3;
  }
  h.tiles_m = static_cast<uint32_t>((M + bt - 1) / bt);
  h.tiles_n = static_cast<uint32_t>((N + bt - 1) / bt);
  if (tiles(bt) >= (1ull << 31)) Fail("too many matmul tiles");
  h.fast = (K % 64 == 0 && K > 0 && h.lda < (1u << 22) && h.ldb < (1u << 22) && h.lda % 8 == 0 && h.ldb % 8 == 0 && h.a_sb0 % 8 == 0 &&
            h.a_sb1 % 8 == 0 && h.b_sb0 % 8 == 0 && h.b_sb1 % 8 == 0)
               ? 1
               : 0;
  // operand addresses
  for (int which = 0; which < 2; ++which) {
    const ANode &x = which == 0 ? an : bn;
    if (x.view != nullptr) Throw("DVM EXCEPTION. reason: a strided view as a matmul operand is not supported by the gfx950 backend");
    Program::Patch p;
    p.word = static_cast<uint32_t>((which == 0 ? offsetof(VCubeHeader, a_addr) : offsetof(VCubeHeader, b_addr)) / 8);
    p.op_id = x.addr_op;
    p.ws_slot = x.ws_slot;
    p.role = Program::kPatchCubeOperand;
    prog_->patches.push_back(p);
  }
  // the epilogue: one section over values that all live in fragments
  for (int i = 0; i < nn_; ++i) {
    ANode &n = nodes_[i];
    n.has_inner = true;
    n.fd = false;
    n.sec = 0;
    n.last_sec = 0;
    n.level = 0;
    n.uses = 0;
    n.in_cone = false;
  }
  // the tile loop reads A and B itself: they are no values of the epilogue
  const int bias = nodes_[c].nin > 2 ? nodes_[c].in[2] : -1;
  if (bias >= 0 && nodes_[bias].kind != AK_MEM) Fail("matmul bias must come from memory");
  nodes_[c].nin = 0;
  nr_ = 0;
  n_sec_ = 1;
  cur_sec_ = 0;
  single_round_ = true;
  vslot_limit_ = DVM_CUBE_NTEMP;
  sreg_used_ = vslot_used_ = 0;
  max_vslot_ = 0;
  code_.clear();
  n_mem_ = 0;
  // the bias row joins the fp32 accumulators, which are then rounded once to the operand type: that
  // is the matmul's value (src/vm_aic.cce:34-470)
  if (bias >= 0) Emit(VOP_BINF, VB_ADD, VK_MEM, 0, MemIndex(bias), 0);
  Emit(VOP_CAST, VC_RND, 0, RndOf(mm->type_id_), 0, 0);
  acc_node_ = c;
  int sinks[kMaxNodes];
  int ns = 0;
  for (int i = 0; i < nn_; ++i)
    if (nodes_[i].kind == AK_OUT) sinks[ns++] = i;
  for (int i = 0; i < ns; ++i) CountCone(nodes_[sinks[i]].in[0]);
  for (int i = 0; i < ns; ++i) {
    const int x = Resolve(nodes_[sinks[i]].in[0]);
    EmitValue(x);
    Emit(VOP_ST, 0, 0, 0, MemIndex(sinks[i]), 0);
    ConsumeUse(x);
  }
  Emit(VOP_END, 0, 0, 0, 0, 0);
  {
    uint32_t dts[DVM_CUBE_MAXMEM];
    for (int i = 0; i < n_mem_; ++i) dts[i] = cmems_[i].dtype;
    DropCastBeforeStore(dts);
  }
  h.n_mem = n_mem_;
  h.n_code = static_cast<uint32_t>(code_.size());
  h.mem_off = sizeof(VCubeHeader) / 8;
  h.code_off = h.mem_off + n_mem_ * (sizeof(VCubeMem) / 8);
  if (h.code_off + code_.size() > DVM_PARAM_WORDS) Fail("program larger than 4 KB");
  std::memset(&prog_->blob, 0, sizeof(VmParam));
  std::memcpy(prog_->blob.w, &h, sizeof(h));
  std::memcpy(prog_->blob.w + h.mem_off, cmems_, sizeof(VCubeMem) * n_mem_);
  std::memcpy(prog_->blob.w + h.code_off, code_.data(), 8 * code_.size());
  prog_->threads = h.tile == 3 ? 512 : 256;
  prog_->lds_bytes = DVM_CUBE_LDS_BYTES(static_cast<uint32_t>(bt));
  prog_->grid = static_cast<uint32_t>(tiles(bt));
}


// ---------- fused attention ----------

void Compiler::DetectAttention() {
  std::vector<int> uses(n_, 0);
  for (int i = 0; i < n_; ++i) {
    if (!live_[i]) continue;
    const NDObject *o = k_->ops_[i];
    for (int j = 0; j < o->nin; ++j)
      if (o->in[j] != nullptr) ++uses[o->in[j]->id];
  }
  auto last_axis_keep = [](const NDObject *r) {
    if (!r->keepdims || r->aux_ref == nullptr || r->aux_ref->size != 1) return false;
    const int64_t ax = r->aux_ref->data[0];
    return ax == -1 || ax == r->in[0]->rank() - 1;
  };
  for (int i = 0; i < n_; ++i) {
    if (!live_[i]) continue;
    NDObject *m2 = k_->ops_[i];
    if (m2->kind != kObjMatMul || m2->trans_a || m2->trans_b || m2->in[2] != nullptr) continue;
    if (m2->type_id_ != kFloat16 && m2->type_id_ != kBFloat16) continue;
    NDObject *p = m2->in[0], *v = m2->in[1];
    if (p->kind != kObjCast || p->in[0]->type_id_ != kFloat32 || uses[p->id] != 1) continue;
    NDObject *dv = p->in[0];
    if (dv->kind != kObjBinary || dv->op != kDiv || uses[dv->id] != 1) continue;
    NDObject *e = dv->in[0], *sm = dv->in[1];
    if (sm->kind != kObjReduce || sm->op != kSum || sm->in[0] != e || uses[sm->id] != 1 || !last_axis_keep(sm)) continue;
    if (e->kind != kObjUnary || e->op != kExp || uses[e->id] != 2) continue;
    NDObject *sb = e->in[0];
    if (sb->kind != kObjBinary || sb->op != kSub || uses[sb->id] != 1) continue;
    NDObject *x = sb->in[0], *mx = sb->in[1];
    if (mx->kind != kObjReduce || mx->op != kMax || mx->in[0] != x || uses[mx->id] != 1 || !last_axis_keep(mx)) continue;
    if (x->kind != kObjCast || x->type_id_ != kFloat32 || uses[x->id] != 2) continue;
    NDObject *sc = x->in[0];
    NDObject *m1 = sc;
    float scale = 1.0f;
    NDObject *mul = nullptr;
    if (sc->kind == kObjBinaryS && sc->op == kMul && uses[sc->id] == 1) {
      mul = sc;
      m1 = sc->in[0];
      const uint32_t bits = ScalarToContainer(sc->scalar.Get(), sc->in[0]->type_id_);
      std::memcpy(&scale, &bits, 4);
    }
    if (m1->kind != kObjMatMul || m1->trans_a || !m1->trans_b || m1->in[2] != nullptr || uses[m1->id] != 1) continue;
    if (m1->type_id_ != m2->type_id_) continue;
    NDObject *q = m1->in[0], *kk = m1->in[1];
    if (q->kind != kObjLoad || kk->kind != kObjLoad || v->kind != kObjLoad || q->strided || kk->strided || v->strided) continue;
    const int r = q->rank();
    if (kk->rank() != r || v->rank() != r || r < 2) continue;
    bool ok = q->dim(r - 1) == DVM_ATTN_D && kk->dim(r - 1) == DVM_ATTN_D && v->dim(r - 1) == DVM_ATTN_D && kk->dim(r - 2) == v->dim(r - 2) &&
              kk->dim(r - 2) % DVM_ATTN_BKV == 0 && kk->dim(r - 2) > 0 && q->dim(r - 2) > 0;
    for (int d = 0; d < r - 2 && ok; ++d) ok = q->dim(d) == kk->dim(d) && q->dim(d) == v->dim(d) && q->dim(d) > 0;
    if (!ok || q->numel() >= (1ll << 31) || kk->numel() >= (1ll << 31)) continue;
    AttnGroup g = {m1, m2, q, kk, v, scale, -1};
    const int gi = static_cast<int>(attn_groups_.size());
    attn_groups_.push_back(g);
    NDObject *members[] = {m1, mul, x, mx, sb, e, sm, dv, p, m2};
    for (NDObject *mbr : members)
      if (mbr != nullptr) attn_of_[mbr->id] = gi;
  }
}

void Compiler::CompileAttn(int gi) {
  const AttnGroup &g = attn_groups_[gi];
  const int r = g.q->rank();
  VAttnHeader h;
  std::memset(&h, 0, sizeof(h));
  h.entry = VE_ATTN;
  h.dtype = MemDType(g.m2->type_id_);
  int64_t nb = 1;
  for (int d = 0; d < r - 2; ++d) nb *= g.q->dim(d);
  h.nb = static_cast<uint32_t>(nb);
  h.sq = static_cast<uint32_t>(g.q->dim(r - 2));
  h.skv = static_cast<uint32_t>(g.k->dim(r - 2));
  h.d = DVM_ATTN_D;
  h.scale = g.scale;
  h.q_blocks = (h.sq + DVM_ATTN_BQ - 1) / DVM_ATTN_BQ;
  if (static_cast<uint64_t>(h.nb) * h.q_blocks >= (1ull << 31)) Fail("too many attention blocks");
  std::memset(&prog_->blob, 0, sizeof(VmParam));
  std::memcpy(prog_->blob.w, &h, sizeof(h));
  auto patch = [&](size_t byte_off, int op_id, int ws_slot) {
    Program::Patch p;
    p.word = static_cast<uint32_t>(byte_off / 8);
    p.op_id = op_id;
    p.ws_slot = ws_slot;
    p.role = Program::kPatchAligned16;
    prog_->patches.push_back(p);
  };
  patch(offsetof(VAttnHeader, q_addr), g.q->id, -1);
  patch(offsetof(VAttnHeader, k_addr), g.k->id, -1);
  patch(offsetof(VAttnHeader, v_addr), g.v->id, -1);
  // the result goes to the user's store when there is one in this sub-kernel, else to workspace
  const int m2 = g.m2->id;
  if (store_of_[m2] >= 0 && area_[store_of_[m2]] == area_[m2]) {
    patch(offsetof(VAttnHeader, o_addr), store_of_[m2], -1);
  } else if (ws_slot_[m2] >= 0) {
    patch(offsetof(VAttnHeader, o_addr), -1, ws_slot_[m2]);
  } else {
    Fail("attention result has no destination");
  }
  // eight waves of 32 queries (two per SIMD: one wave's softmax runs under the other's MFMAs) measured 767-788 us
  // on fp16 [8,32,2048,128] against 920-940 us for four waves of 64 queries; DVM_ATTN_WAVES=4 selects the latter
  prog_->threads = 512;
  if (const char *e = std::getenv("DVM_ATTN_WAVES")) {
    if (std::atoi(e) == 4) prog_->threads = 256;
  }
  prog_->lds_bytes = DVM_ATTN_LDS_BYTES;
  prog_->grid = h.nb * h.q_blocks;
}

size_t VKernel::CodeGen(bool /*pre*/) {
  if (!normalized_) Normalize();
  Compiler c(this);
  const size_t ws = c.Run();
  compiled_ = true;
  return ws;
}

void VKernel::BindAddresses(const RelocEntry *relocs, size_t n, WsAllocator *alloc, void *workspace) {
  for (size_t i = 0; i < n; ++i) {
    if (relocs[i].io != nullptr) relocs[i].io->addr = relocs[i].addr;
  }
  if (ws_bytes_ > 0) {
    if (workspace != nullptr) {
      ws_base_ = workspace;
    } else if (alloc != nullptr) {
      ws_base_ = alloc->Alloc(ws_bytes_);
    }
    if (ws_base_ == nullptr) Throw("kernel needs workspace but none was provided");
  }
  for (Program &p : programs_) {
    if (p.skip) continue;
    for (const Program::Patch &pt : p.patches) {
      uint64_t addr = 0;
      if (pt.op_id >= 0) {
        addr = reinterpret_cast<uint64_t>(ops_[pt.op_id]->addr);
        if (addr != 0) addr += static_cast<uint64_t>(pt.byte_offset);
      } else if (pt.ws_slot >= 0) {
        addr = reinterpret_cast<uint64_t>(ws_base_) + ws_offsets_[pt.ws_slot] + static_cast<uint64_t>(pt.byte_offset);
      }
      if (addr == 0) Throw("a tensor address is missing at launch");
      p.blob.w[pt.word] = addr;
      if ((addr & 15u) != 0) {
        if (pt.role == Program::kPatchVecMem) {
          reinterpret_cast<VMemDesc *>(p.blob.w + pt.word)->flags &= ~static_cast<uint32_t>(VMF_ALIGNED);
        } else if (pt.role == Program::kPatchCubeOperand) {
          reinterpret_cast<VCubeHeader *>(p.blob.w)->fast = 0;
        } else if (pt.role == Program::kPatchAligned16) {
          Throw("fused attention needs 16-byte aligned tensors");
        }
      }
    }
  }
}

int VKernel::Launch(void *stream) {
  if (!compiled_) Throw("Launch before CodeGen");
  if (!g_system.HasDevice()) {
    Throw(std::string("no MI355X device layer: ") + g_system.LoadError());
  }
  const DeviceApi &api = g_system.Api();
  for (Program &p : programs_) {
    for (const Program::Fill &f : p.fills) {
      void *dst = f.op_id >= 0 ? ops_[f.op_id]->addr
                               : static_cast<void *>(static_cast<char *>(ws_base_) + ws_offsets_[f.ws_slot]);
      int rc = api.fill_u32(dst, f.value, f.bytes, stream);
      if (rc != 0) return rc;
    }
    if (p.skip) continue;
    int rc = api.launch_vm(&p.blob, p.grid, p.threads, p.lds_bytes, stream);
    if (rc != 0) return rc;
  }
  return 0;
}

}  // namespace dvm
