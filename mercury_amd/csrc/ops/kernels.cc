#include "kernels.h"

#include <dlfcn.h>

namespace mercury {

namespace {
KernelTable g_table;

template <typename F>
void lookup(void* handle, const char* name, F& slot, const std::string& path) {
  void* symbol = dlsym(handle, name);
  if (!symbol) throw KernelError(path + " has no entry point " + name + "; rebuild the kernel libraries");
  slot = reinterpret_cast<F>(symbol);
}
}  // namespace

void load_kernel_library(const std::string& name, const std::string& path) {
  const bool core = name == "core";
  if (!core && name != "mfma") throw KernelError("unknown kernel library '" + name + "'");
  if (core ? g_table.has_core() : g_table.has_mfma()) return;
  void* handle = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!handle) throw KernelError("cannot load " + path + ": " + dlerror());
  int (*version)() = nullptr;
  lookup(handle, "mk_abi_version", version, path);
  if (version() != MK_ABI_VERSION) {
    throw KernelError(path + " has ABI " + std::to_string(version()) + ", the host core expects " +
                      std::to_string(MK_ABI_VERSION) + "; rebuild");
  }
  KernelTable next = g_table;
#define MK_LOOKUP(fn) lookup(handle, #fn, next.fn, path);
  if (core) {
    MK_CORE_FUNCTIONS(MK_LOOKUP)
    lookup(handle, "mk_last_error", next.core_error, path);
  } else {
    MK_MFMA_FUNCTIONS(MK_LOOKUP)
    lookup(handle, "mk_last_error", next.mfma_error, path);
  }
#undef MK_LOOKUP
  g_table = next;
}

const KernelTable& kernels() { return g_table; }

const KernelTable& need_core() {
  if (!g_table.has_core()) throw KernelError("the kernel library 'core' is not loaded");
  return g_table;
}

const KernelTable& need_mfma() {
  if (!g_table.has_mfma()) {
    throw KernelError("the kernel library 'mfma' (bfloat16 matrix-core kernels) is not loaded");
  }
  return g_table;
}

void check_core(int code, const char* what) {
  if (code != 0) throw KernelError(std::string(what) + ": " + g_table.core_error());
}

void check_mfma(int code, const char* what) {
  if (code != 0) throw KernelError(std::string(what) + ": " + g_table.mfma_error());
}

}  // namespace mercury
