#include "hip_api.h"

#include <dlfcn.h>

#include <mutex>
#include <string>

#include "errors.h"

namespace mercury {

namespace {
HipApi g_api;
std::once_flag g_once;
std::string g_failure;

void* find(const char* name) {
  // The runtime already in the process (PyTorch loads its own with global visibility) ...
  if (void* symbol = dlsym(RTLD_DEFAULT, name)) return symbol;
  // ... or, in a process without one, the system's.
  static void* handle = dlopen("libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
  return handle ? dlsym(handle, name) : nullptr;
}

template <typename F>
void bind(F& slot, const char* name) {
  slot = reinterpret_cast<F>(find(name));
  if (!slot && g_failure.empty()) g_failure = std::string("the HIP runtime has no ") + name;
}

void load() {
  bind(g_api.host_malloc, "hipHostMalloc");
  bind(g_api.host_free, "hipHostFree");
  bind(g_api.memcpy_async, "hipMemcpyAsync");
  bind(g_api.event_create, "hipEventCreateWithFlags");
  bind(g_api.event_record, "hipEventRecord");
  bind(g_api.event_synchronize, "hipEventSynchronize");
  bind(g_api.event_destroy, "hipEventDestroy");
  bind(g_api.error_string, "hipGetErrorString");
}
}  // namespace

const HipApi& hip() {
  std::call_once(g_once, load);
  if (!g_failure.empty()) throw KernelError(g_failure);
  return g_api;
}

}  // namespace mercury
