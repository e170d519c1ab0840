// The host-side error channel and version query; compiled into every kernel library.
#include "common.h"
#include "mercury_kernels.h"

#include <stdarg.h>
#include <string>

static thread_local std::string g_last_error;

void mk_set_error(const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
}

extern "C" const char* mk_last_error() { return g_last_error.c_str(); }

extern "C" int mk_abi_version() { return MK_ABI_VERSION; }
