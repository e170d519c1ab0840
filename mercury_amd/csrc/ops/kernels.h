// The kernel libraries as the host core sees them: shared objects opened at run time, their
// entry points looked up by name.  "core" holds the float32-arithmetic kernels every model
// and dtype uses, "mfma" the bfloat16 matrix-core kernels that only bfloat16 serving needs;
// the host core runs with "core" alone when "mfma" was never loaded.
#pragma once

#include <string>

#include "../host/errors.h"
#include "../mercury_kernels.h"
// MK_CORE_FUNCTIONS(X) and MK_MFMA_FUNCTIONS(X): the entry points of the two libraries by
// name, written by the build from the declarations in mercury_kernels.h.
#include "kernel_names.inc"

namespace mercury {

struct KernelTable {
#define MK_DECLARE(name) decltype(&::name) name = nullptr;
  MK_CORE_FUNCTIONS(MK_DECLARE)
  MK_MFMA_FUNCTIONS(MK_DECLARE)
#undef MK_DECLARE
  const char* (*core_error)() = nullptr;
  const char* (*mfma_error)() = nullptr;
  bool has_core() const { return core_error != nullptr; }
  bool has_mfma() const { return mfma_error != nullptr; }
};

// Open a kernel library ("core" or "mfma") from `path`; a second call for the same name is a
// no-op.  Throws KernelError when the file cannot be opened, an entry point is missing or its
// ABI version is not the one this core was compiled against.
void load_kernel_library(const std::string& name, const std::string& path);
const KernelTable& kernels();
// The table with the named library required: throws a clear error when it was never loaded.
const KernelTable& need_core();
const KernelTable& need_mfma();
// Throws KernelError(what + the library's message) when `code` is not 0.
void check_core(int code, const char* what);
void check_mfma(int code, const char* what);

}  // namespace mercury
