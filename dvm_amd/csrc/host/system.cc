#include "system.h"

#include <dlfcn.h>

#include <cstdlib>
#include <mutex>
#include <stdexcept>
#include <string>

#include "ir.h"

namespace dvm {

System g_system;

namespace {
std::mutex g_init_mutex;
std::string g_err_store;

// libdvm_hip.so sits next to this library.
std::string SiblingPath(const char *name) {
  Dl_info info;
  if (dladdr(reinterpret_cast<void *>(&SiblingPath), &info) != 0 && info.dli_fname != nullptr) {
    std::string p(info.dli_fname);
    auto pos = p.rfind('/');
    if (pos != std::string::npos) return p.substr(0, pos + 1) + name;
  }
  return name;
}
}  // namespace

void System::Init() {
  std::lock_guard<std::mutex> lock(g_init_mutex);
  if (initialized_) return;
  initialized_ = true;
  const char *env = std::getenv("DVM_HIP_LIBRARY");
  std::string path = env != nullptr ? std::string(env) : SiblingPath("libdvm_hip.so");
  void *handle = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (handle == nullptr) {
    const char *e = dlerror();
    g_err_store = std::string("cannot load ") + path + ": " + (e != nullptr ? e : "?");
    load_error_ = g_err_store.c_str();
    return;
  }
  bool ok = true;
#define DVM_BIND(field, sym)                                                        \
  api_.field = reinterpret_cast<decltype(api_.field)>(dlsym(handle, #sym));       \
  if (api_.field == nullptr) {                                                      \
    ok = false;                                                                     \
    g_err_store = std::string("missing symbol ") + #sym + " in " + path;           \
  }
  DVM_BIND(init_vm, dvm_hip_init_vm)
  DVM_BIND(select_block_thread, dvm_hip_select_block_thread)
  DVM_BIND(launch_vm, dvm_hip_launch_vm)
  DVM_BIND(fill_u32, dvm_hip_fill_u32)
  DVM_BIND(get_device_count, dvm_hip_get_device_count)
  DVM_BIND(set_device, dvm_hip_set_device)
  DVM_BIND(get_device, dvm_hip_get_device)
  DVM_BIND(create_stream, dvm_hip_create_stream)
  DVM_BIND(destroy_stream, dvm_hip_destroy_stream)
  DVM_BIND(synchronize_stream, dvm_hip_synchronize_stream)
  DVM_BIND(malloc, dvm_hip_malloc)
  DVM_BIND(free, dvm_hip_free)
  DVM_BIND(malloc_host, dvm_hip_malloc_host)
  DVM_BIND(free_host, dvm_hip_free_host)
  DVM_BIND(mem_to_dev, dvm_hip_mem_to_dev)
  DVM_BIND(mem_from_dev, dvm_hip_mem_from_dev)
  DVM_BIND(mem_to_dev_async, dvm_hip_mem_to_dev_async)
  DVM_BIND(memset, dvm_hip_memset)
  DVM_BIND(create_event, dvm_hip_create_event)
  DVM_BIND(destroy_event, dvm_hip_destroy_event)
  DVM_BIND(record_event, dvm_hip_record_event)
  DVM_BIND(synchronize_event, dvm_hip_synchronize_event)
  DVM_BIND(event_elapsed_time, dvm_hip_event_elapsed_time)
  DVM_BIND(error_string, dvm_hip_error_string)
#undef DVM_BIND
  if (!ok) {
    load_error_ = g_err_store.c_str();
    api_ = DeviceApi();
    return;
  }
  uint32_t count = 0;
  if (api_.get_device_count(&count) != 0 || count == 0) {
    load_error_ = "no HIP device visible";
    return;
  }
  int dev = 0;
  if (const char *id = std::getenv("DEVICE_ID")) dev = std::atoi(id);
  dvm_hip_sysconfig conf{};
  int rc = api_.init_vm(dev, &conf);
  if (rc != 0) {
    g_err_store = std::string("dvm_hip_init_vm failed: ") + api_.error_string(rc);
    load_error_ = g_err_store.c_str();
    return;
  }
  device_id = dev;
  core_num = static_cast<uint32_t>(conf.core_num);
  lds_per_wg = static_cast<uint32_t>(conf.local_mem_size);
  lds_per_cu = lds_per_wg;
  has_device_ = true;
}

Config &Config::Instance() { return g_system; }
bool Config::IsInitialized() const { return g_system.IsInit(); }

void Throw(const std::string &msg) { DvmException(msg.c_str()); }

void DvmException(const char *error_str) {
  static const char kPrefix[] = "DVM EXCEPTION. reason: ";
  const std::string msg(error_str);
  // (some callers spell the prefix out themselves: it appears once either way)
  throw std::runtime_error(msg.compare(0, sizeof(kPrefix) - 1, kPrefix) == 0 ? msg : kPrefix + msg);
}

}  // namespace dvm
