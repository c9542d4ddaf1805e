// The fused attention launch.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "compiler.h"

namespace dvm {

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
  h.d = static_cast<uint32_t>(g.q->dim(r - 1));
  h.scale = g.scale;
  h.q_blocks = (h.sq + DVM_ATTN_BQ - 1) / DVM_ATTN_BQ;
  // where the (batch, head) pairs of each operand lie (views are walked in place)
  AttnLayout lay[3] = {AttnOperandLayout(g.q), AttnOperandLayout(g.k), AttnOperandLayout(g.v)};
  uint32_t nb_inner = 1;
  for (const AttnLayout &l : lay) {
    if (!l.ok) Fail("attention operand layout");
    if (l.nb_inner != 1) nb_inner = l.nb_inner;
  }
  if (g.out_store != nullptr && g.out_nb_inner != 1) nb_inner = g.out_nb_inner;
  h.nb_inner = nb_inner;
  for (int i = 0; i < 3; ++i) {
    const NDObject *t = i == 0 ? g.q : (i == 1 ? g.k : g.v);
    h.row_stride[i] = lay[i].row;
    if (lay[i].nb_inner == 1 && nb_inner != 1) {  // dense beside a view with two batch axes: split its batch stride
      const int64_t per = t->dim(r - 2) * t->dim(r - 1);
      h.inner_stride[i] = static_cast<uint32_t>(per);
      h.outer_stride[i] = static_cast<uint32_t>(per * nb_inner);
    } else {
      h.outer_stride[i] = lay[i].outer;
      h.inner_stride[i] = lay[i].inner;
    }
  }
  // the result is dense, [nb][sq][d], unless it goes into a Store through strides
  h.row_stride[3] = h.d;
  h.inner_stride[3] = nb_inner != 1 ? h.sq * h.d : 0;
  h.outer_stride[3] = h.sq * h.d * nb_inner;
  if (g.out_store != nullptr) {
    h.row_stride[3] = g.out_row;
    if (g.out_nb_inner == 1 && nb_inner != 1) {  // one batch stride beside operands with two: split it
      h.inner_stride[3] = g.out_outer;
      h.outer_stride[3] = g.out_outer * nb_inner;
    } else {
      h.inner_stride[3] = g.out_inner;
      h.outer_stride[3] = g.out_outer;
    }
  }
  if (static_cast<uint64_t>(h.nb) * h.q_blocks >= (1ull << 31)) Fail("too many attention blocks");
  std::memset(&prog_->blob, 0, sizeof(VmParam));
  std::memcpy(prog_->blob.w, &h, sizeof(h));
  auto patch = [&](size_t byte_off, int op_id, int ws_slot, int64_t elem_offset = 0) {
    Program::Patch p;
    p.word = static_cast<uint32_t>(byte_off / 8);
    p.op_id = op_id;
    p.ws_slot = ws_slot;
    p.byte_offset = elem_offset * 2;
    p.role = Program::kPatchAligned16;
    prog_->patches.push_back(p);
  };
  patch(offsetof(VAttnHeader, q_addr), lay[0].root->id, -1, lay[0].base);
  patch(offsetof(VAttnHeader, k_addr), lay[1].root->id, -1, lay[1].base);
  patch(offsetof(VAttnHeader, v_addr), lay[2].root->id, -1, lay[2].base);
  // the result goes to the user's store when there is one in this sub-kernel, else to workspace
  const int m2 = g.m2->id;
  if (g.out_store != nullptr) {
    patch(offsetof(VAttnHeader, o_addr), g.out_store->id, -1, g.out_base);
  } else if (store_of_[m2] >= 0 && area_[store_of_[m2]] == area_[m2]) {
    patch(offsetof(VAttnHeader, o_addr), store_of_[m2], -1);
  } else if (ws_slot_[m2] >= 0) {
    patch(offsetof(VAttnHeader, o_addr), -1, ws_slot_[m2]);
  } else {
    Fail("attention result has no destination");
  }
  // eight waves of 32 queries (two per SIMD: one wave's softmax runs under the other's MFMAs) measured 767-788 us
  // on fp16 [8,32,2048,128] against 920-940 us for four waves of 64 queries; DVM_ATTN_WAVES=4 selects the latter
  prog_->threads = 512;
  if (k_->tuning_.attn_waves == 4) prog_->threads = 256;
  prog_->lds_bytes = DVM_ATTN_LDS_BYTES_D(h.d);
  prog_->grid = h.nb * h.q_blocks;
}
}  // namespace dvm
