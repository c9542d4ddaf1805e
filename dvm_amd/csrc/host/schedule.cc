// Nodes of one sub-kernel, domain axes, their order and merging, and the schedule with its launch geometry.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "compiler.h"

namespace dvm {

int Compiler::AddNode(AKind kind, NDObject *op, DataType t, const int64_t *dims, int rank) {
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
int Compiler::LeafFor(NDObject *v) {
  if (node_of_[v->id] >= 0) return node_of_[v->id];
  int idx;
  if (v->kind == kObjBroadcastS) {
    idx = AddNode(AK_SCALAR, v, v->type_id_, v->shape_ref_->data, v->rank());
  } else {
    idx = AddNode(AK_MEM, v, v->type_id_, v->shape_ref_->data, v->rank());
    const NDObject *root = ViewRoot(v);
    // a permuted or sliced value carries the strides of the whole chain down to the root's memory
    if (v->kind == kObjPermute || v->kind == kObjSlice || v->kind == kObjHalf64) nodes_[idx].view = v;
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

void Compiler::Fail(const char *why) {
  std::string msg = "cannot compile sub-kernel " + std::to_string(cur_area_) + " (partition mode " +
                    std::to_string(mode_) + "): " + why;
  if (k_->tuning_.debug) {
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
    if (o->kind == kObjStore && o->type_id_ == kInt64) {
      // an int64 value is two int32 values: each is stored through strides into its own words of the buffer
      for (int part = 0; part < 2; ++part) {
        const int out = AddNode(AK_OUT, o, kInt32, o->shape_ref_->data, o->rank());
        nodes_[out].nin = 1;
        nodes_[out].in[0] = in_idx[part];
        nodes_[out].addr_op = i;
        nodes_[out].view = part == 0 ? o : o->hi_view;
        if (part == 0) node_of_[i] = out;
      }
      continue;
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
    if (o->kind == kObjOneHot || o->kind == kObjGather) {
      n.view = o;  // the operator's own operand: positions along the new dim / the source tensor
      if (o->kind == kObjGather) n.addr_op = i;
    }
    node_of_[i] = idx;
    // a value later sub-kernels read and that the user does not store: write it to workspace
    if (mat_[i] && ws_slot_[i] >= 0) {
      const int out = AddNode(AK_OUT, o, o->type_id_, o->shape_ref_->data, o->rank());
      nodes_[out].nin = 1;
      nodes_[out].in[0] = idx;
      nodes_[out].ws_slot = ws_slot_[i];
      nodes_[out].view = PartsLayout(o);
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
  std::vector<char> &reduced_var = scratch_c_;
  reduced_var.assign(uf_.size(), 0);
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
        int od = n.op->part_split != 0 ? 1 : 0;  // (a reduce shared between workgroups: dim 0 numbers the parts)
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
        if (n.op->kind == kObjOneHot || (n.op->kind == kObjGather && n.op->op == 1)) {
          // the input's dims stand in the result's in order, apart from the dim a OneHot adds / with the dims of a
          // slice gather's index where the gathered dim was
          const ANode &x = nodes_[n.in[0]];
          int64_t at = n.op->slice_dim;
          if (n.op->kind == kObjOneHot) {
            if (at < 0) at += n.rank;
            for (int d = 0; d < x.rank; ++d) {
              const int od = d < at ? d : d + 1;
              if (x.dims[d] != 1 && x.dims[d] == n.dims[od]) Union(Var(i, od), Var(n.in[0], d));
            }
          } else {
            if (at < 0) at += n.rank - x.rank + 1;
            for (int d = 0; d < x.rank; ++d)
              if (x.dims[d] != 1 && x.dims[d] == n.dims[at + d]) Union(Var(i, static_cast<int>(at) + d), Var(n.in[0], d));
          }
          break;
        }
        for (int j = 0; j < n.nin; ++j)
          if (n.in[j] >= 0) UnifyAligned(i, n.in[j]);
        break;
    }
  }
  // Reduces that share a sub-kernel have the same input shape and axes: their inputs walk the
  // same index space even when no operator relates them, so their dims are unified by position.
  {
    int first = -1, first_red = -1;
    for (int i = 0; i < nn_; ++i) {
      if (nodes_[i].kind != AK_REDUCE) continue;
      if (first < 0) {
        first = nodes_[i].in[0];
        first_red = i;
        continue;
      }
      const ANode &x = nodes_[nodes_[i].in[0]], &f = nodes_[first];
      if (x.rank != f.rank) Fail("reduces of different rank in one sub-kernel");
      if (nodes_[i].op->part_split != 0 && first_red >= 0 && nodes_[first_red].op->part_split != 0) Union(Var(i, 0), Var(first_red, 0));
      for (int d = 0; d < x.rank; ++d)
        if (x.dims[d] != 1 && x.dims[d] == f.dims[d]) Union(Var(nodes_[i].in[0], d), Var(first, d));
    }
  }
  // Parts of the sub-kernel that no operator relates to each other (consumers of two different views of one
  // buffer, each with its own store; a copy beside a reduce) walk the same index space too.
  {
    std::vector<int> &comp = scratch_a_;
    comp.resize(nn_);
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
    std::vector<int> &rep = scratch_b_;
    rep.assign(nn_, -1);
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
  std::vector<int> &axis_of = scratch_a_;
  axis_of.assign(uf_.size(), -1);
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
  // the axis that numbers the parts of a shared reduce lies outside every other axis
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.kind != AK_REDUCE || n.op->part_split == 0 || n.axis[0] < 0) continue;
    for (int ax = 0; ax < n_axes_; ++ax)
      if (ax != n.axis[0]) axes_[ax].before |= 1u << n.axis[0];
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
        if (n.kind != AK_MEM && n.kind != AK_OUT && !(n.kind == AK_OP && n.view != nullptr)) continue;
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
  // A reduce shared between workgroups: the axis that numbers its parts must be the outermost kept dim, by itself;
  // the schedule is laid out for one part of the reduced index space.
  uint32_t parts = 0;
  for (int i = 0; i < nn_; ++i) {
    const ANode &n = nodes_[i];
    if (n.kind != AK_REDUCE || n.op->part_split == 0) continue;
    parts = static_cast<uint32_t>(n.op->part_split);
    const int ax = n.axis[0];
    if (ax < 0 || nk_ == 0) Fail("no axis for the parts of a shared reduce");
    const Dim &outer = dims_[klist_[nk_ - 1]];
    if (outer.first_axis != pos_[ax] || outer.last_axis != pos_[ax] || n_peel_ > 0) Fail("the parts of a shared reduce are not the outermost kept dim");
  }
  const uint64_t n_r_whole = n_r;
  if (parts != 0) n_r = (n_r + parts - 1) / parts;
  uint32_t threads = 256;
  single_round_ = true;
  // Slabs per lane per instruction: the wide build of the VM halves the dispatches per element at the price
  // of registers (at most 512 lanes per workgroup, two waves per SIMD). It pays where the instruction stream,
  // not memory, sets the pace: reduces along the innermost axis with long rows.
  // Measured on MI355X it does not pay (batch-norm 98 us against 76, RMSNorm 118 us against 104): two waves per
  // SIMD hide too little latency. Kept as a tuning switch, off by default.
  bool wide = false;
  if (k_->tuning_.vec_wide == 1) wide = !(nr_ > 0 && !inner_red) && parts == 0;
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
    const bool tile_gather = k_->tuning_.vec_gather_tile != 0;
    if (tile_gather && nk_ >= 2 && nk_ < DVM_VEC_MAXR && klist_[0] == inner && dims_[inner].extent % (8 * E) == 0) {
      for (int i = 0; i < nn_ && !split_inner_; ++i) {
        const ANode &n = nodes_[i];
        if ((n.kind != AK_MEM && n.kind != AK_OUT && n.kind != AK_OP) || n.view == nullptr) continue;
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
    if (threads > pw_threads_cap_) threads = pw_threads_cap_;  // (fewer lanes: more V register slots for each)
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
    // (Rounded down to a power of two since the sweep build exists: rows of one wave or two then run as native loops.
    // The same graph: 1536 rows 22.5 us with 256 lanes per row, 20.0 with 128; 3072 rows 28.5 with 128, 25.7 with 64.)
    {
      const uint64_t lanes_per_output = (1ull << 18) / std::max<uint64_t>(n_k, 1);
      uint32_t cap = Pow2Ceil(lanes_per_output);
      if (cap > lanes_per_output) cap >>= 1;
      cap = std::max<uint32_t>(64, cap);
      if (k_->tuning_.vec_team >= 1) {
        const uint32_t c = static_cast<uint32_t>(k_->tuning_.vec_team);
        if ((c & (c - 1)) == 0) cap = c;
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
    // (a shared reduce: the lanes along the kept space stay inside one part where its outputs are few, so that the
    // parts spread over workgroups)
    const uint64_t n_k_part = parts != 0 ? std::max<uint64_t>(n_k / parts, 1) : n_k;
    uint32_t tx = n_k_part >= 64 ? 64 : Pow2Ceil(n_k_part);
    uint32_t ty = 256 / tx;
    const uint64_t items = (n_k + tx - 1) / tx;
    if (items < 128 && n_r > 256) ty = 512 / tx;  // few outputs: give each more lanes along the reduce space (the kernel's limit is 512)
    else if (items < 128 && n_r >= 64) ty = 512 / tx;     // (the launch that reduces over the parts of a shared reduce, mostly)
    // (the parts of a shared reduce: with fewer than two workgroups per compute unit, 512 lanes each put twice the
    // loads in flight. Measured on MI355X, fp32 sums over axis 0: [8192,1024] 57 -> 47 us, [65536,768] 136 -> 97 us,
    // [32,3136,256] over its first two axes 86 -> 70 us; 1024 lanes are slower again, 54 / 120 / 79 us)
    if (parts != 0 && items < 2ull * g_system.core_num && n_r >= 32) ty = 512 / tx;
    while (ty > 1 && static_cast<uint64_t>(ty) * U > 2 * n_r) ty >>= 1;
    threads = std::max<uint32_t>(64, tx * ty);
    ty = threads / tx;
    hdr_.team_log2 = Log2(tx);
    hdr_.n_items = static_cast<uint32_t>(items);
    single_round_ = n_r <= static_cast<uint64_t>(ty) * U;
  }
  if (wide) hdr_.sched |= VS_WIDE;
  if (parts != 0) {
    if (nr_ == 0) Fail("a shared reduce without a reduced dim");
    // indices of the reduced space one round of a team covers; a part is whole rounds
    const uint32_t team_lanes = inner_red ? (hdr_.team_is_block ? threads : (1u << hdr_.team_log2)) : threads >> hdr_.team_log2;
    const uint64_t round = static_cast<uint64_t>(team_lanes) * U;
    const uint64_t chunk = (n_r + round - 1) / round * round;
    if (chunk >= (1ull << 31)) Fail("index space above 2^31 groups");
    hdr_.r_chunk = static_cast<uint32_t>(chunk);
    hdr_.k_per_chunk = static_cast<uint32_t>(n_k / parts);
    if (hdr_.k_per_chunk == 0 || n_k % parts != 0) Fail("the parts of a shared reduce do not divide the kept index space");
    single_round_ = chunk <= round;
    (void)n_r_whole;
  }

  prog_->threads = threads;
}
}  // namespace dvm
