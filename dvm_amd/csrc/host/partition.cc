// Which operators share a launch (sub-kernel), and which values cross launches through memory.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "compiler.h"

namespace dvm {

// ---------- liveness ----------
void Compiler::MarkLive() {
  for (int i = n_ - 1; i >= 0; --i) {
    NDObject *o = k_->ops_[i];
    if (o->kind == kObjStore && !o->temp) live_[i] = 1;
    if (!live_[i]) continue;
    for (int j = 0; j < o->nin; ++j)
      if (o->in[j] != nullptr) live_[o->in[j]->id] = 1;
    for (NDObject *p : o->parts) live_[p->id] = 1;
  }
}

bool Compiler::DomCompatible(const AreaInfo &ai, const int64_t *dims, int rank) const {
  const int r = std::max(ai.rank, rank);
  for (int i = 0; i < r; ++i) {
    const int64_t da = i + ai.rank >= r ? ai.dom[i + ai.rank - r] : 1;
    const int64_t db = i + rank >= r ? dims[i + rank - r] : 1;
    if (da != db && da != 1 && db != 1) return false;
  }
  return true;
}

void Compiler::DomMerge(AreaInfo &ai, const int64_t *dims, int rank) {
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

bool Compiler::SameReduce(const NDObject *a, const NDObject *b) {
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
int Compiler::LevelIn(int a, const NDObject *o) const {
  int lvl = 0;
  for (int j = 0; j < o->nin; ++j) {
    const NDObject *v = o->in[j];
    if (v == nullptr || area_[v->id] != a) continue;
    lvl = std::max(lvl, level_[v->id] + (v->kind == kObjReduce ? 1 : 0));
  }
  return lvl;
}

bool Compiler::CanJoin(int a, const NDObject *o) {
  if (a >= static_cast<int>(areas_.size())) return true;  // a fresh sub-kernel
  const AreaInfo &ai = areas_[a];
  if (ai.stage != o->stage) return false;
  // a store goes where the value it stores is computed (an operator's own output is never a reason to cut)
  if (IsStoreLike(o) && ai.attn < 0 && !ai.cube && area_[o->in[0]->id] == a) return true;
  if (ai.has_part || (o->kind == kObjReduce && o->part_split != 0 && ai.has_reduce)) {
    // beside a reduce shared between workgroups only its like and operators on its input's index space
    if (o->kind == kObjReduce) {
      if (!ai.has_part || o->part_split != ai.reduce->part_split) return false;
    } else if (o->numel() != ai.reduce->in[0]->numel()) {
      return false;
    }
  }
  // The launch that reduces over the parts of a shared reduce holds what works on the reduce's output (the mean, the
  // variance, their stores). An operator on a larger index space (x - mean) would make that launch walk the larger
  // space and reduce the parts again for every one of its elements: it reads the result from memory in a launch of its own.
  if (ai.over_parts != 0 && o->numel() > ai.over_parts) return false;
  if (o->kind == kObjReduce && LevelIn(a, o) < 8 && ai.red_at_level[LevelIn(a, o)] >= 2) return false;
  if (o->kind == kObjMatMul) return false;
  if (ai.n_ops >= area_ops_limit_ && !IsStoreLike(o)) return false;  // long graphs are cut into several launches
  if (ai.attn >= 0) return o->kind == kObjStore && (o->in[0] == attn_groups_[ai.attn].m2 || o == attn_groups_[ai.attn].out_store);
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

void Compiler::Join(int a, const NDObject *o) {
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
      ai.has_part = o->part_split != 0;
    }
    if (o->in[0] != nullptr) {
      const NDObject *src = ViewRoot(o->in[0]);
      if (src->kind == kObjReduce && src->part_split != 0) ai.over_parts = std::max<int64_t>(ai.over_parts, o->numel());
    }
    DomMerge(ai, o->in[0]->shape_ref_->data, o->in[0]->rank());
  }
  DomMerge(ai, o->shape_ref_->data, o->rank());
}

void Compiler::Partition() {
  areas_.clear();
  const bool fuse = !conservative_;
  // Operators that share no tensor (directly or through other operators) never share a
  // sub-kernel: connected components are numbered first, each gets its own range of areas.
  std::vector<int> &comp = scratch_a_;
  comp.resize(n_);
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
  std::vector<int> &comp_base = scratch_b_;
  comp_base.assign(n_, -1);
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
      if (v->kind == kObjReduce && v->part_split != 0) cut = true;  // the reduce over the parts is a launch of its own
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

// ---------- reduces shared between workgroups ----------
bool Compiler::SplitLongReduces() {
  const int forced = k_->tuning_.red_split;
  if (forced == 0 || forced == 1) return false;
  std::vector<NDObject *> &ops = k_->ops_;
  const uint64_t cus = std::max<uint64_t>(g_system.core_num, 1);
  struct Cand {
    NDObject *r;
    int split;
  };
  std::vector<Cand> cands;
  for (NDObject *r : ops) {
    if (r->kind != kObjReduce || r->in[0] == nullptr || r->aux_ref == nullptr) continue;
    const NDObject *x = r->in[0];
    const int xr = x->rank();
    if (xr == 0 || r->rank() + 1 > kMaxRank) continue;
    bool red[kMaxRank] = {false};
    for (size_t j = 0; j < r->aux_ref->size; ++j) {
      int64_t d = r->aux_ref->data[j];
      if (d < 0) d += xr;
      if (d >= 0 && d < xr) red[d] = true;
    }
    uint64_t n_red = 1, n_out = 1;
    int kept_dims = 0, last = -1;
    bool empty = false;
    for (int d = 0; d < xr; ++d) {
      const int64_t e = x->dim(d);
      if (e <= 0) empty = true;
      if (e == 1) continue;
      last = d;
      if (red[d]) {
        n_red *= static_cast<uint64_t>(e);
      } else {
        n_out *= static_cast<uint64_t>(e);
        ++kept_dims;
      }
    }
    if (empty || last < 0 || n_red < 2 || kept_dims > DVM_VEC_MAXR - 1) continue;
    int split = 0;
    if (forced >= 2) {
      split = forced;
    } else {
      // workgroups the schedules would give it: one per output when the innermost axis is reduced, else one per
      // 64 lanes of 8 outputs along the innermost axis
      const uint64_t wgs = red[last] ? n_out : (n_out + 511) / 512;
      if (wgs >= cus) continue;
      // worth a second launch only when a workgroup would have a quarter of a million elements to itself (measured:
      // [32, 65536] summed along its rows takes 18 us in one launch and 24-29 us in two)
      const uint64_t outs_per_wg = red[last] ? 1 : std::min<uint64_t>(n_out, 512);
      if (n_red * outs_per_wg < (1u << 18)) continue;
      uint64_t want = 2 * cus / wgs;
      split = 1;
      while (static_cast<uint64_t>(split) * 2 <= want && split < 256) split *= 2;
      // a part is worth a workgroup's while: 32k elements
      while (split > 1 && n_red / static_cast<uint64_t>(split) * outs_per_wg < 32768) split /= 2;
    }
    if (split < 2 || n_red < 2ull * static_cast<uint64_t>(split)) continue;
    // every consumer works on the reduce's own output, or on a larger index space (x - max of a softmax: it then
    // reads the result from memory in a launch of its own, see CanJoin)
    bool ok = false;
    for (const NDObject *c : ops) {
      for (int j = 0; j < c->nin; ++j) {
        if (c->in[j] != r) continue;
        ok = true;
        if (c->numel() < r->numel() || c->kind == kObjReduce || c->kind == kObjMatMul || c->kind == kObjConcatPart) split = 0;
      }
      for (const NDObject *part : c->parts)
        if (part == r) split = 0;
    }
    if (ok && split >= 2) cands.push_back({r, split});
  }
  // reduces that would share a launch are shared alike or not at all
  for (size_t i = 0; i < cands.size(); ++i) {
    for (const NDObject *q : ops) {
      if (q->kind != kObjReduce || q == cands[i].r || q->in[0] == nullptr || q->aux_ref == nullptr) continue;
      if (!SameReduce(cands[i].r, q)) continue;
      bool also = false;
      for (const Cand &c : cands)
        if (c.r == q && c.split == cands[i].split) also = true;
      if (!also) cands[i].split = 0;
    }
  }
  bool any = false;
  for (const Cand &c : cands) any = any || c.split >= 2;
  if (!any) return false;
  saved_ops_ = ops;
  std::vector<NDObject *> next;
  next.reserve(ops.size() + cands.size());
  for (NDObject *o : saved_ops_) {
    next.push_back(o);
    for (const Cand &c : cands) {
      if (c.r != o || c.split < 2) continue;
      SplitRecord *rec = new SplitRecord();
      rec->reduce = o;
      rec->rank = static_cast<size_t>(o->rank());
      for (size_t d = 0; d < rec->rank; ++d) rec->shape[d] = o->dim(static_cast<int>(d));
      rec->axis0.data = &rec->zero;
      rec->axis0.size = 1;
      NDObject *second = new NDObject(kObjReduce, o->type_id_);
      second->op = o->op;
      second->in[0] = o;
      second->nin = 1;
      second->aux_ref = &rec->axis0;
      second->keepdims = false;
      second->stage = o->stage;
      second->SetShape(rec->shape, rec->rank);
      rec->second = second;
      int64_t longer[kMaxRank];
      longer[0] = c.split;
      for (size_t d = 0; d < rec->rank; ++d) longer[d + 1] = rec->shape[d];
      o->SetShape(longer, rec->rank + 1);
      o->part_split = c.split;
      splits_.push_back(rec);
      if (k_->tuning_.red_split_turn != 0) {
        // The partial results are written with the parts innermost ([outputs][parts]: a scattered store of a few
        // values per workgroup), and the second reduce reads them through a view of that shape: it reduces the
        // innermost axis of a dense operand, a row per output, rows spread over workgroups, every element of a row
        // fetched at once. Over the outermost axis the same reduce had one workgroup per 512 outputs and a round
        // trip to memory per two parts.
        NDObject *layout = new NDObject(kObjStore, o->type_id_);
        layout->strided = true;
        layout->view_base_ = 0;
        layout->vstride_[0] = 1;
        NDObject *turned = new NDObject(kObjPermute, o->type_id_);
        turned->in[0] = o;
        turned->nin = 1;
        turned->stage = o->stage;
        turned->strided = true;
        turned->view_base_ = 0;
        int64_t shape_t[kMaxRank], dense = c.split;
        for (size_t d = rec->rank; d-- > 0;) {
          shape_t[d] = rec->shape[d];
          turned->vstride_[d] = dense;
          layout->vstride_[d + 1] = dense;
          dense *= rec->shape[d];
          rec->turn_dims[d] = static_cast<int64_t>(d) + 1;
        }
        shape_t[rec->rank] = c.split;
        turned->vstride_[rec->rank] = 1;
        rec->turn_dims[rec->rank] = 0;
        rec->turn_order.data = rec->turn_dims;
        rec->turn_order.size = rec->rank + 1;
        turned->aux_ref = &rec->turn_order;
        turned->SetShape(shape_t, rec->rank + 1);
        rec->layout = layout;
        rec->turned = turned;
        rec->zero = static_cast<int64_t>(rec->rank);
        second->in[0] = turned;
        next.push_back(turned);
      }
      next.push_back(second);
    }
  }
  for (NDObject *c : saved_ops_) {
    for (int j = 0; j < c->nin; ++j) {
      for (SplitRecord *rec : splits_) {
        if (c->in[j] != rec->reduce) continue;
        repoints_.push_back({c, j, c->in[j]});
        c->in[j] = rec->second;
      }
    }
  }
  ops.swap(next);
  for (size_t i = 0; i < ops.size(); ++i) ops[i]->id = static_cast<int>(i);
  return true;
}

void Compiler::UndoSplitReduces(bool keep_programs) {
  std::vector<NDObject *> during = k_->ops_;  // operator numbers the programs refer to
  for (const Repoint &rp : repoints_) rp.consumer->in[rp.slot] = rp.was;
  repoints_.clear();
  for (SplitRecord *rec : splits_) {
    rec->reduce->part_split = 0;
    rec->reduce->SetShape(rec->shape, rec->rank);
  }
  k_->ops_ = saved_ops_;
  saved_ops_.clear();
  for (size_t i = 0; i < k_->ops_.size(); ++i) k_->ops_[i]->id = static_cast<int>(i);
  // (the records go whatever happens below: a later code generation must not find them again)
  struct DropRecords {
    std::vector<SplitRecord *> &v;
    ~DropRecords() {
      for (SplitRecord *rec : v) {
        delete rec->second;
        delete rec->turned;
        delete rec->layout;
        delete rec;
      }
      v.clear();
    }
  } drop{splits_};
  if (keep_programs) {
    auto renumber = [&](int &op_id) {
      if (op_id < 0) return;
      NDObject *o = during[static_cast<size_t>(op_id)];
      for (SplitRecord *rec : splits_)
        if (rec->second == o) Throw("a program addresses memory through a reduce over parts");
      op_id = o->id;
    };
    for (Program &p : k_->programs_) {
      for (Program::Patch &pt : p.patches) renumber(pt.op_id);
      for (Program::Fill &f : p.fills) renumber(f.op_id);
    }
  }
}

// ---------- which values cross sub-kernels ----------
void Compiler::PlanMaterialisation() {
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
      if (attn_of_[i] >= 0 && attn_groups_[attn_of_[i]].out_store == o) continue;  // (the attention kernel writes it through strides)
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

// ---------- fused attention ----------

Compiler::AttnLayout Compiler::AttnOperandLayout(const NDObject *x) const {
  AttnLayout l;
  const NDObject *root = ViewRoot(x);
  if (root->kind != kObjLoad) return l;
  const bool is_view = x != root ? (x->kind == kObjPermute || x->kind == kObjSlice) : root->strided;
  if (x != root && !is_view) return l;      // (a reshape in the chain)
  if (x != root && root->strided) return l; // (a view of a strided load: its strides are not composed)
  const int r = x->rank();
  if (r < 2) return l;
  l.root = root;
  const int64_t rows = x->dim(r - 2), d = x->dim(r - 1);
  if (!is_view) {  // dense: any number of batch axes, they collapse into one
    l.ok = true;
    l.row = static_cast<uint32_t>(d);
    l.outer = static_cast<uint32_t>(rows * d);
    l.inner = 0;
    l.nb_inner = 1;
    return l;
  }
  if (r > 4) return l;
  const int64_t *st = x->vstride_;
  if (d != 1 && st[r - 1] != 1) return l;
  auto fits = [](int64_t v) { return v >= 0 && v < (1ll << 24) * 64 && v % 8 == 0; };
  const int64_t row = rows == 1 ? d : st[r - 2];
  if (row < d || row >= (1ll << 22) || row % 8 != 0 || x->view_base_ % 8 != 0 || x->view_base_ < 0) return l;
  int64_t outer = 0, inner = 0, nb_inner = 1;
  if (r == 3) {
    outer = x->dim(0) == 1 ? 0 : st[0];
  } else if (r == 4) {
    outer = x->dim(0) == 1 ? 0 : st[0];
    inner = x->dim(1) == 1 ? 0 : st[1];
    nb_inner = x->dim(1);
  }
  if (!fits(outer) || !fits(inner) || outer >= (1ll << 32) || inner >= (1ll << 32)) return l;
  l.ok = true;
  l.base = x->view_base_;
  l.row = static_cast<uint32_t>(row);
  l.outer = static_cast<uint32_t>(outer);
  l.inner = static_cast<uint32_t>(inner);
  l.nb_inner = static_cast<uint32_t>(nb_inner);
  return l;
}

void Compiler::DetectAttention() {
  std::vector<int> &uses = scratch_a_;
  uses.assign(n_, 0);
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
    if (m2->kind != kObjMatMul || m2->gmm_type != 0 || m2->trans_a || m2->trans_b || m2->in[2] != nullptr) continue;
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
    // the scale: on the 16-bit product in front of the cast (the example's order), or on the fp32 scores behind it
    float scale = 1.0f;
    NDObject *mul = nullptr, *mul32 = nullptr;
    if (x->kind == kObjBinaryS && x->op == kMul && x->type_id_ == kFloat32 && uses[x->id] == 2 && x->in[0]->kind == kObjCast &&
        uses[x->in[0]->id] == 1) {
      mul32 = x;
      const uint32_t bits = ScalarToContainer(x->scalar.Get(), kFloat32);
      std::memcpy(&scale, &bits, 4);
      x = x->in[0];
    } else if (uses[x->id] != 2) {
      continue;
    }
    if (x->kind != kObjCast || x->type_id_ != kFloat32) continue;
    NDObject *sc = x->in[0];
    NDObject *m1 = sc;
    if (mul32 == nullptr && sc->kind == kObjBinaryS && sc->op == kMul && uses[sc->id] == 1) {
      mul = sc;
      m1 = sc->in[0];
      const uint32_t bits = ScalarToContainer(sc->scalar.Get(), sc->in[0]->type_id_);
      std::memcpy(&scale, &bits, 4);
    }
    if (m1->kind != kObjMatMul || m1->gmm_type != 0 || m1->trans_a || !m1->trans_b || m1->in[2] != nullptr || uses[m1->id] != 1) continue;
    if (m1->type_id_ != m2->type_id_) continue;
    NDObject *q = m1->in[0], *kk = m1->in[1];
    // q, k, v: loads, or views of loads the kernel can walk in place (a heads-first view of a [batch, seq, heads, d]
    // tensor, a slice of a longer cache); the three agree on how the batch axes split
    const AttnLayout lq = AttnOperandLayout(q), lk = AttnOperandLayout(kk), lv = AttnOperandLayout(v);
    if (!lq.ok || !lk.ok || !lv.ok) continue;
    {
      uint32_t nbi = 1;
      bool same = true;
      for (const AttnLayout *l : {&lq, &lk, &lv}) {
        if (l->nb_inner == 1) continue;
        if (nbi != 1 && nbi != l->nb_inner) same = false;
        nbi = l->nb_inner;
      }
      // (a dense operand beside a view with two batch axes: its collapsed batch stride must split the same way,
      // which holds when its own rank gives the same inner extent)
      for (const AttnLayout *l : {&lq, &lk, &lv})
        if (nbi != 1 && l->nb_inner == 1 && l->inner == 0 && l->root != nullptr) {
          const NDObject *t = l == &lq ? q : (l == &lk ? kk : v);
          if (t->rank() != 4 || static_cast<uint32_t>(t->dim(1)) != nbi) same = false;
        }
      if (!same) continue;
    }
    const int r = q->rank();
    if (kk->rank() != r || v->rank() != r || r < 2) continue;
    bool ok = DVM_ATTN_D_OK(q->dim(r - 1)) && kk->dim(r - 1) == q->dim(r - 1) && v->dim(r - 1) == q->dim(r - 1) && kk->dim(r - 2) == v->dim(r - 2) &&
              kk->dim(r - 2) > 0 && q->dim(r - 2) > 0 && scale > 0.0f;  // (the kernel takes maxima before it scales)
    for (int d = 0; d < r - 2 && ok; ++d) ok = q->dim(d) == kk->dim(d) && q->dim(d) == v->dim(d) && q->dim(d) > 0;
    if (!ok || q->numel() >= (1ll << 31) || kk->numel() >= (1ll << 31)) continue;
    AttnGroup g = {m1, m2, q, kk, v, scale, -1};
    // Where the result goes when its one consumer is a Store through strides, or a Permute (head dimension still
    // innermost) whose one consumer is a dense Store: the kernel writes rows of d elements through a row stride and
    // two batch strides, so the [batch, seq, heads, d] layout of a [batch, heads, seq, d] result costs no copy.
    NDObject *out_store = nullptr;
    if (uses[m2->id] == 1 && r >= 2 && r <= 4) {
      NDObject *c1 = nullptr;
      for (int j = i + 1; j < n_ && c1 == nullptr; ++j) {
        NDObject *o = k_->ops_[j];
        if (!live_[j]) continue;
        for (int t = 0; t < o->nin; ++t)
          if (o->in[t] == m2) c1 = o;
      }
      int64_t st[kMaxRank];
      bool have = false;
      int64_t base = 0;
      if (c1 != nullptr && c1->kind == kObjStore && c1->strided && c1->pad_size < 0 && c1->type_id_ == m2->type_id_ && c1->stride_ref != nullptr) {
        for (int d = 0; d < r; ++d) st[d] = c1->vstride_[d];
        base = c1->view_base_;
        out_store = c1;
        have = true;
      } else if (c1 != nullptr && c1->kind == kObjPermute && uses[c1->id] == 1 && c1->aux_ref != nullptr && static_cast<int>(c1->aux_ref->size) == r) {
        NDObject *c2 = nullptr;
        for (int j = c1->id + 1; j < n_ && c2 == nullptr; ++j) {
          NDObject *o = k_->ops_[j];
          if (live_[j] && o->nin >= 1 && o->in[0] == c1) c2 = o;
        }
        if (c2 != nullptr && c2->kind == kObjStore && !c2->strided && !c2->temp && !c2->inplace && c2->type_id_ == m2->type_id_) {
          // result dim perm[i] lies at the dense stride of dim i of the permuted value
          int64_t dense = 1;
          for (int d = r - 1; d >= 0; --d) {
            int64_t src = c1->aux_ref->data[d];
            if (src < 0) src += r;
            st[src] = dense;
            dense *= c1->dim(d);
          }
          out_store = c2;
          have = true;
        }
      }
      if (have) {
        auto fits = [](int64_t v) { return v >= 0 && v < (1ll << 32) && v % 8 == 0; };
        const int64_t d = m2->dim(r - 1), rows = m2->dim(r - 2);
        const int64_t row = rows == 1 ? d : st[r - 2];
        bool ok_out = (d == 1 || st[r - 1] == 1) && row >= d && row < (1ll << 22) && row % 8 == 0 && base >= 0 && base % 8 == 0;
        int64_t outer = 0, inner = 0, nbi = 1;
        if (r == 3) {
          outer = m2->dim(0) == 1 ? 0 : st[0];
        } else if (r == 4) {
          outer = m2->dim(0) == 1 ? 0 : st[0];
          inner = m2->dim(1) == 1 ? 0 : st[1];
          nbi = m2->dim(1);
        }
        ok_out = ok_out && fits(outer) && fits(inner);
        // the operands must split their (batch, head) pairs the same way: views with two batch axes already do, or
        // they are dense rank-4 tensors whose second dim is the inner extent
        if (ok_out && nbi != 1) {
          for (const AttnLayout *l : {&lq, &lk, &lv}) {
            const NDObject *t = l == &lq ? q : (l == &lk ? kk : v);
            if (l->nb_inner != 1 ? l->nb_inner != static_cast<uint32_t>(nbi) : (t->rank() != 4 || t->dim(1) != nbi)) ok_out = false;
          }
        } else if (ok_out) {
          for (const AttnLayout *l : {&lq, &lk, &lv})
            if (l->nb_inner != 1) ok_out = false;  // (rank 4 with one head: the operands' split decides; keep it simple)
        }
        if (ok_out) {
          g.out_store = out_store;
          g.out_row = static_cast<uint32_t>(row);
          g.out_outer = static_cast<uint32_t>(outer);
          g.out_inner = static_cast<uint32_t>(inner);
          g.out_nb_inner = static_cast<uint32_t>(nbi);
          g.out_base = base;
        } else {
          out_store = nullptr;
        }
      }
    }
    const int gi = static_cast<int>(attn_groups_.size());
    attn_groups_.push_back(g);
    NDObject *members[] = {m1, mul, x, mul32, mx, sb, e, sm, dv, p, m2, g.out_store};
    for (NDObject *mbr : members)
      if (mbr != nullptr) attn_of_[mbr->id] = gi;
  }
}
}  // namespace dvm
