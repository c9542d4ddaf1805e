// Drives the device layer alone: libdvm_hip.so through include/dvm_hip.h, no host compiler, no Python. The program
// is a 4096-byte blob in the device VM's bytecode (dvm_amd/csrc/isa_gfx950.h is the format), read from a fixture
// that tests/golden/make_blob_fixture.py wrote; this file fills in the three tensor addresses, launches it through
// dvm_hip_launch_vm and again through dvm_hip_launch_vm_static_ws, and checks out = x * y + 0.5.
//
// usage: device_blob <blob file> <workgroups> <threads> <lds bytes> <elements>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "dvm_hip.h"
#include "isa_gfx950.h"

static void Must(int code, const char *what) {
  if (code != 0) {
    std::fprintf(stderr, "%s: %s\n", what, dvm_hip_error_string(code));
    std::exit(2);
  }
}

int main(int argc, char **argv) {
  if (argc != 6) {
    std::fprintf(stderr, "usage: %s <blob file> <workgroups> <threads> <lds bytes> <elements>\n", argv[0]);
    return 2;
  }
  const uint32_t blocks = std::atoi(argv[2]), threads = std::atoi(argv[3]), lds = std::atoi(argv[4]);
  const size_t n = std::atoi(argv[5]);
  alignas(16) unsigned char blob[DVM_PARAM_BYTES];
  FILE *f = std::fopen(argv[1], "rb");
  if (f == nullptr || std::fread(blob, 1, sizeof(blob), f) != sizeof(blob)) {
    std::fprintf(stderr, "cannot read %zu bytes from %s\n", sizeof(blob), argv[1]);
    return 2;
  }
  std::fclose(f);
  VVecHeader *h = reinterpret_cast<VVecHeader *>(blob);
  if (h->entry != VE_VECTOR || h->n_mem != 3) {
    std::fprintf(stderr, "the fixture is not the three-operand vector program this test expects\n");
    return 2;
  }
  dvm_hip_sysconfig conf;
  Must(dvm_hip_init_vm(0, &conf), "dvm_hip_init_vm");
  if (conf.wave_size != 64) {
    std::fprintf(stderr, "wave size %llu\n", static_cast<unsigned long long>(conf.wave_size));
    return 1;
  }
  std::vector<float> x(n), y(n), out(n);
  for (size_t i = 0; i < n; ++i) {
    x[i] = 0.5f * static_cast<float>(i % 11) - 2.0f;
    y[i] = 0.25f * static_cast<float>(i % 7) + 1.0f;
  }
  void *dx, *dy, *dout, *stream;
  Must(dvm_hip_malloc(&dx, n * 4), "malloc");
  Must(dvm_hip_malloc(&dy, n * 4), "malloc");
  Must(dvm_hip_malloc(&dout, n * 4), "malloc");
  Must(dvm_hip_create_stream(&stream), "stream");
  Must(dvm_hip_mem_to_dev(dx, x.data(), n * 4), "copy");
  Must(dvm_hip_mem_to_dev(dy, y.data(), n * 4), "copy");
  // the memory operand descriptors sit at word offset mem_off, in the order the graph named them: x, y, out
  VMemDesc *mems = reinterpret_cast<VMemDesc *>(blob + 8 * h->mem_off);
  mems[0].addr = reinterpret_cast<uint64_t>(dx);
  mems[1].addr = reinterpret_cast<uint64_t>(dy);
  mems[2].addr = reinterpret_cast<uint64_t>(dout);
  int failures = 0;
  for (int route = 0; route < 2; ++route) {
    Must(dvm_hip_fill_u32(dout, 0x7fc00000u, n * 4, stream), "fill");  // NaN everywhere: every element must be written
    if (route == 0) {
      Must(dvm_hip_launch_vm(blob, blocks, threads, lds, stream), "dvm_hip_launch_vm");
    } else {
      const uint32_t geometry[3] = {blocks, threads, lds};
      Must(dvm_hip_launch_vm_static_ws(blob, 1, geometry, nullptr, 0, 0, stream), "dvm_hip_launch_vm_static_ws");
    }
    Must(dvm_hip_synchronize_stream(stream), "synchronize");
    Must(dvm_hip_mem_from_dev(out.data(), dout, n * 4), "copy back");
    for (size_t i = 0; i < n; ++i) {
      if (out[i] != x[i] * y[i] + 0.5f) {
        if (failures < 5) std::fprintf(stderr, "route %d element %zu: %g, expected %g\n", route, i, out[i], x[i] * y[i] + 0.5f);
        ++failures;
      }
    }
  }
  dvm_hip_destroy_stream(stream);
  dvm_hip_free(dx);
  dvm_hip_free(dy);
  dvm_hip_free(dout);
  if (failures != 0) return 1;
  std::puts("PASS");
  return 0;
}
