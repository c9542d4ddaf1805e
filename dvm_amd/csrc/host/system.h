// Process-wide state of the host library: the bound device layer, the device
// limits used by the emitter, and the Config switches.
// Role in the reference: g_system (src/system.h:150-285, src/system.cc:314-359).
#ifndef DVM_AMD_HOST_SYSTEM_H_
#define DVM_AMD_HOST_SYSTEM_H_

#include <cstddef>
#include <cstdint>

#include "../../../include/dvm.h"
#include "../../../include/dvm_hip.h"

namespace dvm {

// Function table of libdvm_hip.so, resolved with dlopen so that the host
// library also loads (for code generation, dumps and disassembly) on a machine
// without a GPU runtime.
struct DeviceApi {
  decltype(&dvm_hip_init_vm) init_vm = nullptr;
  decltype(&dvm_hip_select_block_thread) select_block_thread = nullptr;
  decltype(&dvm_hip_launch_vm) launch_vm = nullptr;
  decltype(&dvm_hip_fill_u32) fill_u32 = nullptr;
  decltype(&dvm_hip_get_device_count) get_device_count = nullptr;
  decltype(&dvm_hip_set_device) set_device = nullptr;
  decltype(&dvm_hip_get_device) get_device = nullptr;
  decltype(&dvm_hip_create_stream) create_stream = nullptr;
  decltype(&dvm_hip_destroy_stream) destroy_stream = nullptr;
  decltype(&dvm_hip_synchronize_stream) synchronize_stream = nullptr;
  decltype(&dvm_hip_malloc) malloc = nullptr;
  decltype(&dvm_hip_free) free = nullptr;
  decltype(&dvm_hip_malloc_host) malloc_host = nullptr;
  decltype(&dvm_hip_free_host) free_host = nullptr;
  decltype(&dvm_hip_mem_to_dev) mem_to_dev = nullptr;
  decltype(&dvm_hip_mem_from_dev) mem_from_dev = nullptr;
  decltype(&dvm_hip_mem_to_dev_async) mem_to_dev_async = nullptr;
  decltype(&dvm_hip_memset) memset = nullptr;
  decltype(&dvm_hip_create_event) create_event = nullptr;
  decltype(&dvm_hip_destroy_event) destroy_event = nullptr;
  decltype(&dvm_hip_record_event) record_event = nullptr;
  decltype(&dvm_hip_synchronize_event) synchronize_event = nullptr;
  decltype(&dvm_hip_event_elapsed_time) event_elapsed_time = nullptr;
  decltype(&dvm_hip_error_string) error_string = nullptr;
};

class System : public Config {
 public:
  void Init();  // idempotent
  bool IsInit() const { return initialized_; }
  bool HasDevice() const { return has_device_; }
  const DeviceApi &Api() const { return api_; }
  const char *LoadError() const { return load_error_; }

  Config &SetDeterm() override { determ_ = true; return *this; }
  Config &UnsetDeterm() override { determ_ = false; return *this; }
  Config &SetOnlineTuner() override { online_tuner_ = true; return *this; }
  Config &UnsetOnlineTuner() override { online_tuner_ = false; return *this; }
  Config &SetLazyTuner() override { lazy_tuner_ = true; return *this; }
  Config &UnsetLazyTuner() override { lazy_tuner_ = false; return *this; }
  Config &SetVfFusion(int mode = 1) override { vf_fusion_ = mode; return *this; }
  Config &UnsetVfFusion() override { vf_fusion_ = 0; return *this; }

  // Device limits the emitter plans against. Without a device they hold the
  // MI355X figures, so that code generation and disassembly are the same on a
  // CPU-only machine as on the GPU box.
  int device_id = 0;  // the device the VM was initialised on
  uint32_t core_num = 256;
  uint32_t lds_per_wg = 160 * 1024;
  uint32_t lds_per_cu = 160 * 1024;
  bool determ_ = false;
  bool online_tuner_ = false;
  bool lazy_tuner_ = false;
  int vf_fusion_ = 0;

 private:
  bool initialized_ = false;
  bool has_device_ = false;
  DeviceApi api_;
  const char *load_error_ = "";
};

extern System g_system;

}  // namespace dvm
#endif  // DVM_AMD_HOST_SYSTEM_H_
