// A framework-side consumer of the C++ graph API: includes include/dvm.h only (plus the device layer's C header for
// device memory), links libdvm.so, builds kernels the way a framework adapter does and checks the results.
//
// What it covers of the reference's include/dvm.h contract:
//   1. fixed addresses: Load(addr) / Store(addr) / CodeGen() / Launch(nullptr, 0, nullptr, stream), the flow of the
//      reference's examples/cc/muladd.cc:57-75 (x * y + 0.5 over 1024 floats, expected 6.5);
//   2. late binding: Load(nullptr) / Store(nullptr), PreCodeGen() once, then Launch(relocs, n, workspace, stream)
//      with different buffers (include/dvm.h:201-206, :706-707);
//   3. dynamic shapes: one IntArrayRef re-read at every Normalize() + CodeGen(relocs, n, ws) (include/dvm.h:149-159),
//      with a row sum, so a second schedule of the device VM runs;
//   4. errors arrive as std::runtime_error("DVM EXCEPTION. reason: ...") (include/dvm.h:752).
// Exit status 0 and a last line "PASS" on success.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <vector>

#include "dvm.h"
#include "dvm_hip.h"

namespace {

int g_failures = 0;

void Expect(bool ok, const char *what) {
  if (!ok) {
    std::fprintf(stderr, "FAILED: %s\n", what);
    ++g_failures;
  }
}

void Must(int code, const char *what) {
  if (code != 0) {
    std::fprintf(stderr, "%s: %s\n", what, dvm_hip_error_string(code));
    std::exit(2);
  }
}

// Device buffer of floats with host mirror.
struct Buffer {
  explicit Buffer(size_t n, float fill = 0.0f) : host(n, fill) {
    Must(dvm_hip_malloc(&dev, n * sizeof(float)), "dvm_hip_malloc");
    Upload();
  }
  ~Buffer() { dvm_hip_free(dev); }
  void Upload() { Must(dvm_hip_mem_to_dev(dev, host.data(), host.size() * sizeof(float)), "copy to device"); }
  void Download() { Must(dvm_hip_mem_from_dev(host.data(), dev, host.size() * sizeof(float)), "copy from device"); }
  void *dev = nullptr;
  std::vector<float> host;
};

struct Workspace : dvm::WsAllocator {
  void *Alloc(size_t size) override {
    void *p = nullptr;
    Must(dvm_hip_malloc(&p, size == 0 ? 16 : size), "workspace");
    blocks.push_back(p);
    return p;
  }
  ~Workspace() {
    for (void *p : blocks) dvm_hip_free(p);
  }
  std::vector<void *> blocks;
};

void FixedAddresses(void *stream) {
  const size_t n = 1024;
  Buffer x(n, 2.0f), y(n, 3.0f), out(n, -1.0f);
  std::vector<int64_t> dims = {static_cast<int64_t>(n)};
  dvm::IntArrayRef shape(dims);
  dvm::Kernel k;
  k.Reset(dvm::kVector, 0);
  dvm::NDObject *product = k.Binary<dvm::kMul>(k.Load(x.dev, &shape, dvm::kFloat32), k.Load(y.dev, &shape, dvm::kFloat32));
  k.Store(out.dev, k.Binary<dvm::kAdd>(product, 0.5f));
  k.CodeGen();
  Expect(k.Launch(nullptr, 0, nullptr, stream) == 0, "launch with fixed addresses");
  Must(dvm_hip_synchronize_stream(stream), "synchronize");
  out.Download();
  bool ok = true;
  for (float v : out.host) ok = ok && std::fabs(v - 6.5f) <= 1e-5f;
  Expect(ok, "x * y + 0.5 == 6.5 everywhere");
  Expect(std::string(k.Das()).find("Mul.fp32") != std::string::npos, "Das() shows the multiply");
}

void LateBinding(void *stream) {
  const size_t n = 3000;  // not a multiple of the slab width: the guarded tail runs
  std::vector<int64_t> dims = {static_cast<int64_t>(n)};
  dvm::IntArrayRef shape(dims);
  dvm::Kernel k;
  k.Reset(dvm::kVector, 0);
  dvm::NDObject *a = k.Load(nullptr, &shape, dvm::kFloat32);
  dvm::NDObject *b = k.Load(nullptr, &shape, dvm::kFloat32);
  dvm::NDObject *st = k.Store(nullptr, k.Binary<dvm::kSub>(k.Unary<dvm::kAbs>(a), k.Binary<dvm::kMul>(b, 2.0f)));
  const size_t ws_bytes = k.PreCodeGen();
  void *ws = nullptr;
  if (ws_bytes != 0) Must(dvm_hip_malloc(&ws, ws_bytes), "workspace");
  for (int round = 0; round < 2; ++round) {
    Buffer x(n), y(n), out(n, 7.0f);
    for (size_t i = 0; i < n; ++i) {
      x.host[i] = (round == 0 ? -1.0f : 1.0f) * static_cast<float>(i % 17) - 3.0f;
      y.host[i] = 0.25f * static_cast<float>(i % 5) + round;
    }
    x.Upload();
    y.Upload();
    const dvm::RelocEntry relocs[] = {{a, x.dev}, {b, y.dev}, {st, out.dev}};
    Expect(k.Launch(relocs, 3, ws, stream) == 0, "launch with relocations");
    Must(dvm_hip_synchronize_stream(stream), "synchronize");
    out.Download();
    bool ok = true;
    for (size_t i = 0; i < n; ++i) ok = ok && out.host[i] == std::fabs(x.host[i]) - y.host[i] * 2.0f;
    Expect(ok, round == 0 ? "|x| - 2y, first buffers" : "|x| - 2y, second buffers");
  }
  if (ws != nullptr) dvm_hip_free(ws);
}

void DynamicShapes(void *stream) {
  const int64_t cols = 640;
  std::vector<int64_t> dims = {1, cols};
  dvm::IntArrayRef shape(dims);
  std::vector<int64_t> axes = {1};
  dvm::IntArrayRef axes_ref(axes);
  dvm::Kernel k;
  k.Reset(dvm::kSplit, 0);
  dvm::NDObject *in = k.Load(nullptr, &shape, dvm::kFloat32);
  dvm::NDObject *st = k.Store(nullptr, k.Reduce<dvm::kSum>(k.Binary<dvm::kMul>(in, in), &axes_ref, true));
  for (int64_t rows : {5, 300, 64, 5}) {
    dims[0] = rows;  // the kernel reads the shape again through the IntArrayRef it was given
    Buffer x(static_cast<size_t>(rows * cols)), out(static_cast<size_t>(rows), -1.0f);
    for (size_t i = 0; i < x.host.size(); ++i) x.host[i] = static_cast<float>((i * 7) % 13) * 0.125f - 0.5f;
    x.Upload();
    const dvm::RelocEntry relocs[] = {{in, x.dev}, {st, out.dev}};
    Workspace ws;
    k.Normalize();
    k.CodeGen(relocs, 2, &ws);
    Expect(k.Launch(stream) == 0, "launch after CodeGen(relocs)");
    Must(dvm_hip_synchronize_stream(stream), "synchronize");
    out.Download();
    dvm::IntArrayRef *oshape = dvm::Kernel::GetShape(st);
    Expect(oshape->size == 2 && oshape->data[0] == rows && oshape->data[1] == 1, "inferred output shape [rows, 1]");
    bool ok = true;
    for (int64_t r = 0; r < rows; ++r) {
      double want = 0.0;
      for (int64_t c = 0; c < cols; ++c) want += static_cast<double>(x.host[r * cols + c]) * x.host[r * cols + c];
      ok = ok && std::fabs(out.host[r] - want) <= 1e-5 * (1.0 + want);
    }
    Expect(ok, "row sums of squares at a new row count");
  }
}

void Errors() {
  std::vector<int64_t> d3 = {3}, d4 = {4};
  dvm::IntArrayRef s3(d3), s4(d4);
  dvm::Kernel k;
  k.Reset(dvm::kVector, 0);
  bool thrown = false;
  try {
    dvm::NDObject *a = k.Load(nullptr, &s3, dvm::kFloat32), *b = k.Load(nullptr, &s4, dvm::kFloat32);
    k.Store(nullptr, k.Binary<dvm::kAdd>(a, b));
    k.PreCodeGen();
  } catch (const std::runtime_error &e) {
    thrown = std::string(e.what()).rfind("DVM EXCEPTION. reason: ", 0) == 0;
  }
  Expect(thrown, "shapes [3] + [4] are refused with a DVM EXCEPTION");
}

}  // namespace

int main() {
  dvm_hip_sysconfig conf;
  Must(dvm_hip_init_vm(0, &conf), "dvm_hip_init_vm");
  void *stream = nullptr;
  Must(dvm_hip_create_stream(&stream), "dvm_hip_create_stream");
  try {
    FixedAddresses(stream);
    LateBinding(stream);
    DynamicShapes(stream);
    Errors();
  } catch (const std::exception &e) {
    std::fprintf(stderr, "unexpected exception: %s\n", e.what());
    return 3;
  }
  dvm_hip_destroy_stream(stream);
  if (g_failures != 0) return 1;
  std::puts("PASS");
  return 0;
}
