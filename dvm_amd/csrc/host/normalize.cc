// Operator list of a kernel and shape inference (the Normalize family of the reference, src/ops.cc:1117-1123,
// 2398-2464, 2683-2695, 3080-3123): every operator's shape from its inputs' shapes, strides and offsets of views.
#include <algorithm>
#include <cstring>

#include "ir.h"
#include "system.h"

namespace dvm {

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
        if (o->type_id_ == kInt64) {
          // the low words go to every second 32-bit word of the buffer, the high words (hi_view) to the ones between
          const size_t r = o->in[0]->shape_ref_->size;
          if (o->stride_ref != nullptr && o->stride_ref->size != r) Throw("stride list does not match the tensor rank");
          int64_t dense = 1;
          for (size_t i = r; i-- > 0;) {
            o->vstride_[i] = 2 * (o->stride_ref != nullptr ? o->stride_ref->data[i] : dense);
            dense *= o->shape_[i];
          }
          o->view_base_ = 2 * o->view_offset;
          NDObject *hv = o->hi_view;
          hv->SetShape(o->shape_, r);
          for (size_t i = 0; i < r; ++i) hv->vstride_[i] = o->vstride_[i];
          hv->view_base_ = o->view_base_ + 1;
          break;
        }
        if (o->pad_size >= 0) {
          // PadStore (src/ops.cc:1399-1412): the buffer's rows are pad_size elements longer than the value's
          const size_t r = o->in[0]->shape_ref_->size;
          if (r == 0) Throw("PadStore of a value without dims");
          int64_t dense = 1;
          for (size_t i = r; i-- > 0;) {
            o->vstride_[i] = dense;
            dense *= o->shape_[i] + (i + 1 == r ? o->pad_size : 0);
          }
          o->view_base_ = o->view_offset;
          break;
        }
        if (o->strided) {
          if (o->stride_ref->size != o->in[0]->shape_ref_->size) Throw("stride list does not match the tensor rank");
          for (size_t i = 0; i < o->stride_ref->size; ++i) o->vstride_[i] = o->stride_ref->data[i];
          o->view_base_ = o->view_offset;
        }
        break;
      case kObjPack64:
        o->SetShape(o->in[0]->shape_ref_->data, o->in[0]->shape_ref_->size);
        break;
      case kObjOneHot: {
        const NDObject *x = o->in[0];
        const size_t r = x->shape_ref_->size;
        if (r + 1 > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
        if (o->aux_ref == nullptr || o->aux_ref->size != 1 || o->aux_ref->data[0] < 0) Throw("OneHot needs one depth");
        int64_t axis = o->slice_dim;
        if (axis < 0) axis += static_cast<int64_t>(r) + 1;
        if (axis < 0 || axis > static_cast<int64_t>(r)) Throw("OneHot axis out of range");
        for (size_t i = 0, j = 0; i <= r; ++i) {
          o->shape_[i] = static_cast<int64_t>(i) == axis ? o->aux_ref->data[0] : x->shape_ref_->data[j++];
          o->vstride_[i] = static_cast<int64_t>(i) == axis ? 1 : 0;
        }
        o->own_ref_.size = r + 1;
        o->view_base_ = 0;  // (vstride_ describes the operator's own operand; the value itself is dense: strided stays false)
        break;
      }
      case kObjGather: {
        const NDObject *ix = o->in[0];
        const IntArrayRef *src = o->full_shape_ref;
        const size_t rs = src->size, ri = ix->shape_ref_->size;
        int64_t axis = o->slice_dim;
        if (axis < 0) axis += static_cast<int64_t>(rs);
        if (rs == 0 || axis < 0 || axis >= static_cast<int64_t>(rs)) Throw("gather axis out of range");
        int64_t dense[kMaxRank], acc = 1;
        for (size_t i = rs; i-- > 0;) {
          dense[i] = acc;
          acc *= src->data[i];
        }
        o->gather_extent = src->data[axis];
        o->gather_stride = dense[axis];
        if (acc >= (1ll << 31)) Throw("GatherLoad from a tensor of 2^31 elements or more");  // (offsets are int32 arithmetic)
        if (o->gather_extent == 0 && ix->numel() > 0) Throw("GatherLoad along an empty dim");
        if (o->op == 0) {  // the index has the source's rank; the result takes its shape
          if (ri != rs) Throw("the index of an element gather needs the rank of the source");
          for (size_t i = 0; i < rs; ++i) {
            if (static_cast<int64_t>(i) != axis && ix->shape_ref_->data[i] > src->data[i]) Throw("the index of an element gather reaches outside the source");
            o->shape_[i] = ix->shape_ref_->data[i];
            o->vstride_[i] = static_cast<int64_t>(i) == axis ? 0 : dense[i];
          }
          o->own_ref_.size = rs;
        } else {  // the index's dims stand where the gathered dim was
          const size_t r = rs - 1 + ri;
          if (r > static_cast<size_t>(kMaxRank)) Throw("tensor rank above 10");
          size_t n = 0;
          for (size_t i = 0; i < static_cast<size_t>(axis); ++i, ++n) {
            o->shape_[n] = src->data[i];
            o->vstride_[n] = dense[i];
          }
          for (size_t i = 0; i < ri; ++i, ++n) {
            o->shape_[n] = ix->shape_ref_->data[i];
            o->vstride_[n] = 0;
          }
          for (size_t i = static_cast<size_t>(axis) + 1; i < rs; ++i, ++n) {
            o->shape_[n] = src->data[i];
            o->vstride_[n] = dense[i];
          }
          o->own_ref_.size = r;
        }
        o->view_base_ = 0;  // (vstride_ describes the operator's own operand; the value itself is dense: strided stays false)
        break;
      }
      case kObjHalf64: {
        // the 32-bit words of an int64 Load: its strides (its own when it is a strided load, else those of a dense
        // tensor) doubled, its offset doubled, plus one for the high words
        const NDObject *x = o->in[0];
        const size_t r = x->shape_ref_->size;
        o->SetShape(x->shape_ref_->data, r);
        int64_t dense = 1;
        for (size_t i = r; i-- > 0;) {
          o->vstride_[i] = 2 * (x->strided ? x->vstride_[i] : dense);
          dense *= x->shape_ref_->data[i];
        }
        o->view_base_ = 2 * (x->strided ? x->view_base_ : 0) + o->op;
        o->strided = true;
        break;
      }
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
        if (n == 0 && o->elem_any) o->shape_[n++] = 1;  // (ElemAny's result has shape [1])
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
        if (o->gmm_type != 0) {  // src/ops_m.cc:721-762 of the reference
          const NDObject *gl = o->group_list;
          if (gl->rank() != 1) Throw("GroupedMatMul needs a list of one dim");
          const int64_t groups = gl->dim(0);
          if (o->gmm_type == 1) {
            if (ra != 2 || rb != 3 || b->dim(0) != groups) Throw("GroupedMatMul over rows needs lhs [m, k] and rhs [groups, k, n]");
            o->shape_[0] = m;
            o->shape_[1] = n;
            o->own_ref_.size = 2;
          } else {
            if (ra != 2 || rb != 2) Throw("GroupedMatMul over the k axis needs lhs [m, k] and rhs [k, n]");
            o->shape_[0] = groups;
            o->shape_[1] = m;
            o->shape_[2] = n;
            o->own_ref_.size = 3;
          }
          const NDObject *bias = o->nin > 2 ? o->in[2] : nullptr;
          if (bias != nullptr && (bias->rank() != 2 || bias->dim(0) != groups || bias->dim(1) != n)) Throw("GroupedMatMul needs a bias of [groups, n]");
          break;
        }
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
}  // namespace dvm
