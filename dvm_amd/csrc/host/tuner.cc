// Online tuner of the matmul launches: which block tile and how many parts of the k axis.
//
// The reference keeps a table of tuned tile parameters per product shape and fills it by running candidates on the
// device (CubeTuner::CacheTable, OnlineCubeTuner and LazyCubeTuner, src/ops_m.h:174-263; switched by
// Config::SetOnlineTuner / SetLazyTuner, include/dvm.h:735-738). Here the host normally picks tile and split from
// figures measured once on an MI355X (CompileCube); with either tuner switched on, the first code generation of a
// product shape on a machine with a device runs every candidate (the plain product on scratch operands, timed with
// events), remembers the fastest in a process-wide table, and that and every later code generation of the shape use it.
#include <array>
#include <map>
#include <mutex>
#include <stdexcept>
#include <tuple>
#include <vector>

#include "compiler.h"
#include "system.h"

namespace dvm {
namespace {

using Key = std::array<int64_t, 8>;

struct Table {
  std::mutex mu;
  std::map<Key, CubeChoice> best;
  uint64_t tuned = 0;  // shapes measured so far (tests read it through CubeTunerStats)
};

Table &TheTable() {
  static Table t;
  return t;
}

struct ScratchAlloc : public WsAllocator {
  std::vector<void *> blocks;
  void *Alloc(size_t size) override {
    void *p = nullptr;
    if (g_system.Api().malloc(&p, size == 0 ? 16 : size) != 0) throw std::runtime_error("tuner: no device memory for a workspace");
    blocks.push_back(p);
    return p;
  }
  ~ScratchAlloc() {
    for (void *p : blocks) g_system.Api().free(p);
  }
};

struct DeviceBuffer {
  void *p = nullptr;
  explicit DeviceBuffer(size_t bytes) {
    if (g_system.Api().malloc(&p, bytes == 0 ? 16 : bytes) != 0) p = nullptr;
  }
  ~DeviceBuffer() {
    if (p != nullptr) g_system.Api().free(p);
  }
};

// Microseconds of the fastest of three launches of the plain product with the given tile and split, or a negative
// number when that candidate cannot be compiled or launched.
double TimeCandidate(const CubeProblem &q, int tile, int split, void *a, void *b, void *c) {
  const DeviceApi &api = g_system.Api();
  try {
    Kernel k;
    k.Reset(kMix, 0);
    std::vector<int64_t> sa, sb;
    if (q.nb0 * q.nb1 > 1) {
      sa.push_back(q.nb0 * q.nb1);
      sb.push_back(q.nb0 * q.nb1);
    }
    sa.push_back(q.trans_a ? q.k : q.m);
    sa.push_back(q.trans_a ? q.m : q.k);
    sb.push_back(q.trans_b ? q.n : q.k);
    sb.push_back(q.trans_b ? q.k : q.n);
    IntArrayRef ra(sa), rb(sb);
    NDObject *la = k.Load(a, &ra, q.dtype), *lb = k.Load(b, &rb, q.dtype);
    k.Store(c, k.MatMul(la, lb, q.trans_a, q.trans_b, nullptr));
    k.GetImpl()->tuning_.cube_tile = tile;
    k.GetImpl()->tuning_.cube_splitk = split <= 1 ? 0 : split;
    k.GetImpl()->tuning_.in_tuner = true;
    k.Normalize();
    ScratchAlloc ws;
    k.CodeGen(nullptr, 0, &ws);
    void *e0 = nullptr, *e1 = nullptr;
    if (api.create_event(&e0) != 0 || api.create_event(&e1) != 0) return -1.0;
    double best = -1.0;
    for (int it = 0; it < 4; ++it) {  // the first launch warms up
      api.record_event(e0, nullptr);
      if (k.Launch(nullptr) != 0) {
        best = -1.0;
        break;
      }
      api.record_event(e1, nullptr);
      if (api.synchronize_event(e1) != 0) {
        best = -1.0;
        break;
      }
      float ms = 0.0f;
      api.event_elapsed_time(&ms, e0, e1);
      if (it > 0 && (best < 0.0 || ms * 1e3 < best)) best = ms * 1e3;
    }
    api.destroy_event(e0);
    api.destroy_event(e1);
    return best;
  } catch (const std::exception &) {
    return -1.0;
  }
}

}  // namespace

bool CubeTunerLookup(const CubeProblem &q, CubeChoice *out) {
  if (!(g_system.online_tuner_ || g_system.lazy_tuner_) || !g_system.HasDevice()) return false;
  const Key key = {q.m, q.n, q.k, q.nb0, q.nb1, static_cast<int64_t>(q.dtype), q.trans_a ? 1 : 0, q.trans_b ? 1 : 0};
  Table &t = TheTable();
  std::lock_guard<std::mutex> lock(t.mu);
  auto hit = t.best.find(key);
  if (hit != t.best.end()) {
    *out = hit->second;
    return out->tile != 0;
  }
  CubeChoice choice;  // tile 0: nothing measured (too large for scratch operands): the host's own rule stays
  const uint64_t batch = static_cast<uint64_t>(q.nb0) * static_cast<uint64_t>(q.nb1);
  const uint64_t bytes_a = batch * q.m * q.k * 2, bytes_b = batch * q.k * q.n * 2, bytes_c = batch * q.m * q.n * 2;
  if (q.m > 0 && q.n > 0 && q.k > 0 && bytes_a + bytes_b + bytes_c <= (3ull << 30)) {
    DeviceBuffer a(bytes_a), b(bytes_b), c(bytes_c);
    if (a.p != nullptr && b.p != nullptr && c.p != nullptr) {
      // operands of ones (fp16 0x3c00; as bf16 the same bits are a small positive number): defined values, no NaNs
      g_system.Api().fill_u32(a.p, 0x3c003c00u, bytes_a & ~static_cast<size_t>(3), nullptr);
      g_system.Api().fill_u32(b.p, 0x3c003c00u, bytes_b & ~static_cast<size_t>(3), nullptr);
      static const int kTiles[3] = {256, 128, 64};
      static const int kSplits[6] = {1, 2, 4, 8, 16, 32};
      for (int tile : kTiles) {
        if (tile > 64 && (q.m * 2 <= tile && q.n * 2 <= tile)) continue;  // (a tile four times the output)
        for (int split : kSplits) {
          if (split > 1 && q.k / split < 256) break;
          const double us = TimeCandidate(q, tile, split, a.p, b.p, c.p);
          if (us > 0.0 && (choice.tile == 0 || us < choice.us)) {
            choice.tile = tile;
            choice.split = split;
            choice.us = us;
          }
        }
      }
      ++t.tuned;
    }
  }
  t.best[key] = choice;
  *out = choice;
  return choice.tile != 0;
}

void CubeTunerStats(uint64_t *shapes_measured, uint64_t *table_size) {
  Table &t = TheTable();
  std::lock_guard<std::mutex> lock(t.mu);
  *shapes_measured = t.tuned;
  *table_size = t.best.size();
}

void CubeTunerClear() {
  Table &t = TheTable();
  std::lock_guard<std::mutex> lock(t.mu);
  t.best.clear();
}

}  // namespace dvm
