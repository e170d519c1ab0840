// The kernel libraries as the host core sees them: shared objects opened at run time, their
// entry points looked up by name.  "core" holds the float32-arithmetic kernels every model
// and dtype uses, "mfma" the bfloat16 matrix-core kernels that only bfloat16 serving needs;
// the host core runs with "core" alone when "mfma" was never loaded.
#pragma once

#include <stdexcept>
#include <string>

#include "../mercury_kernels.h"

namespace mercury {

class KernelError : public std::runtime_error {
 public:
  using std::runtime_error::runtime_error;
};

#define MK_CORE_FUNCTIONS(X)                                                                 \
  X(mk_embed) X(mk_rmsnorm) X(mk_silu_mul) X(mk_rope_kv_write) X(mk_linear_generic)          \
  X(mk_attention_generic) X(mk_qkv_finish) X(mk_argmax) X(mk_sample_scratch_bytes)           \
  X(mk_sample) X(mk_fill_normal)

#define MK_MFMA_FUNCTIONS(X)                                                                 \
  X(mk_linear_skinny_slices) X(mk_linear_skinny) X(mk_linear_skinny_unsplit)                 \
  X(mk_linear_skinny_acc) X(mk_gated_skinny) X(mk_qkv_skinny) X(mk_qkv_tiled)                \
  X(mk_gated_tiled) X(mk_linear_tiled_slices) X(mk_linear_tiled_partials) X(mk_linear_tiled) \
  X(mk_attention_mfma_supported) X(mk_attention_mfma_max_rows) X(mk_attention_mfma_staged)   \
  X(mk_attention_mfma_wide)                                                                  \
  X(mk_attention_mfma)

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
