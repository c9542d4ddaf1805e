// VKernel::CodeGen / BindAddresses / Launch and the loop over partition modes.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstddef>
#include <cstring>
#include <stdexcept>
#include <string>

#include "compiler.h"

namespace dvm {

VKernel::~VKernel() {
  delete compiler_;
  for (NDObject *o : ops_) {
    delete o->hi_view;
    delete o;
  }
}

void Tuning::Read() {
  auto num = [](const char *name) {
    const char *e = std::getenv(name);
    return e != nullptr ? std::atoi(e) : -1;
  };
  vec_wide = num("DVM_VEC_WIDE");
  vec_team = num("DVM_VEC_TEAM");
  vec_runs = num("DVM_VEC_RUNS");
  vec_pair = num("DVM_VEC_PAIR");
  vec_fuse = num("DVM_VEC_FUSE");
  vec_unirun = num("DVM_VEC_UNIRUN");
  vec_reread = num("DVM_VEC_REREAD");
  vec_sweeps = num("DVM_VEC_SWEEPS");
  vec_gather_tile = num("DVM_VEC_GATHER_TILE");
  cube_tile = num("DVM_CUBE_TILE");
  cube_waves = num("DVM_CUBE_WAVES");
  cube_exact = num("DVM_CUBE_EXACT");
  cube_dump16 = num("DVM_CUBE_DUMP16");
  cube_splitk = num("DVM_CUBE_SPLITK");
  red_split = num("DVM_RED_SPLIT");
  red_split_turn = num("DVM_RED_SPLIT_TURN");
  attn_waves = num("DVM_ATTN_WAVES");
  cube_fuse_act = num("DVM_CUBE_FUSE_ACT");
  debug = std::getenv("DVM_DEBUG") != nullptr;
}

// Partition modes, tried in order until every sub-kernel compiles: 0 joins an operator to its
// producers' sub-kernel whenever the hard rules allow, 1 also requires broadcast-compatible
// shapes, 2 additionally ends a sub-kernel after every reduce (the reference's rule), 3 gives
// every operator its own sub-kernel.
size_t Compiler::Run() {
  // Reduces with few outputs and a long reduced extent are rewritten, for this code generation only, into a reduce
  // per part of the reduced index space and a reduce over the parts; should that graph not compile, the kernel
  // is compiled as it was built.
  if (SplitLongReduces()) {
    const int mode_before = k_->part_mode_;  // (the partition mode a kernel remembers is that of the graph as built)
    bool done = false;
    size_t ws = 0;
    try {
      ws = RunModes();
      done = true;
    } catch (...) {  // whatever it was: the operator list must be restored, and the kernel as built gets its chance
    }
    UndoSplitReduces(done);
    k_->part_mode_ = mode_before;
    if (done) return ws;
  }
  return RunModes();
}

size_t Compiler::RunModes() {
  n_ = static_cast<int>(k_->ops_.size());
  const int first_mode = k_->part_mode_;
  area_ops_limit_ = kMaxAreaOps;
  pw_threads_cap_ = 256;
  if (k_->ops_limit_ != 0) {  // what this kernel needed last time
    area_ops_limit_ = k_->ops_limit_;
    pw_threads_cap_ = k_->pw_cap_;
    try {
      const size_t ws = RunOnce(first_mode);
      area_ops_limit_ = kMaxAreaOps;
      pw_threads_cap_ = 256;
      return ws;
    } catch (const std::runtime_error &) {
      k_->ops_limit_ = 0;
      k_->pw_cap_ = 0;
      area_ops_limit_ = kMaxAreaOps;
      pw_threads_cap_ = 256;
    }
  }
  for (int mode = first_mode; mode < 3; ++mode) {
    try {
      const size_t ws = RunOnce(mode);
      k_->part_mode_ = mode;
      return ws;
    } catch (const std::runtime_error &e) {
      if (k_->tuning_.debug) std::fprintf(stderr, "dvm: partition mode %d does not compile: %s\n", mode, e.what());
      // A sub-kernel that holds more values at once than it has registers (a wide expression tree), more operands than
      // descriptors or more code than a blob: the same rules with fewer operators per sub-kernel, before the rules
      // themselves get stricter. (The cut values cross launches through the workspace.)
      const std::string why = e.what();
      const bool resources = why.find("out of V register slots") != std::string::npos || why.find("out of S registers") != std::string::npos ||
                             why.find("too many memory operands") != std::string::npos || why.find("program larger than 4 KB") != std::string::npos;
      if (resources && mode == first_mode) {
        // (first with pointwise workgroups of 128 lanes, which have twice the V register slots per lane)
        struct Restore {
          Compiler *c;
          ~Restore() {
            c->area_ops_limit_ = kMaxAreaOps;
            c->pw_threads_cap_ = 256;
          }
        } restore{this};
        pw_threads_cap_ = 128;
        for (int limit : {kMaxAreaOps, 40, 20, 10, 5}) {
          if (limit != kMaxAreaOps && limit >= n_) continue;
          area_ops_limit_ = limit;
          try {
            const size_t ws = RunOnce(mode);
            k_->part_mode_ = mode;
            k_->ops_limit_ = limit;
            k_->pw_cap_ = pw_threads_cap_;
            return ws;
          } catch (const std::runtime_error &e2) {
            if (k_->tuning_.debug) std::fprintf(stderr, "dvm: partition mode %d, %d operators a sub-kernel: %s\n", mode, limit, e2.what());
          }
        }
      }
    }
  }
  k_->part_mode_ = 3;
  try {
    return RunOnce(3);
  } catch (const std::runtime_error &) {
    k_->part_mode_ = first_mode;  // (what failed may be the rewritten graph: the next attempt starts where this one did)
    throw;
  }
}

size_t Compiler::RunOnce(int mode) {
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
  for (Program &p : k_->programs_)
    if (!p.skip) p.RememberBindDependent();
  size_t total = 0;
  for (size_t i = 0; i < k_->ws_sizes_.size(); ++i) {
    k_->ws_offsets_.push_back(total);
    total += (k_->ws_sizes_[i] + 255) & ~static_cast<size_t>(255);
  }
  k_->ws_bytes_ = total;
  return total;
}

size_t VKernel::CodeGen(bool /*pre*/) {
  if (!normalized_) Normalize();
  if (compiler_ == nullptr) compiler_ = new Compiler(this);
  const size_t ws = compiler_->Run();
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
    for (const auto &orig : p.bind_dependent) reinterpret_cast<uint32_t *>(p.blob.w)[orig.first] = orig.second;
    for (const Program::Patch &pt : p.patches) {
      uint64_t addr = 0;
      if (pt.role == Program::kPatchIota) {  // positions along an axis: no memory, the word is the first value
        p.blob.w[pt.word] = static_cast<uint64_t>(pt.byte_offset / 4);
        continue;
      }
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
          // (the sweep build accesses the operands of its interior rounds without guards: the generic kernel runs instead)
          uint32_t sched;
          char *sched_at = reinterpret_cast<char *>(p.blob.w) + offsetof(VVecHeader, sched);
          std::memcpy(&sched, sched_at, sizeof(sched));
          sched &= ~static_cast<uint32_t>(VS_SWEEPS);
          std::memcpy(sched_at, &sched, sizeof(sched));
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
