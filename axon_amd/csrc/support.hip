// What every kernel library has beside its kernels: the error channel of the C interface and the
// build's compute dtype.  Compiled into the engine's own library and into every library built
// from a part's own kernel sources (each has its own channel).
#include <stdarg.h>
#include <stdio.h>

#include "api.h"
#include "common.h"

static thread_local char g_error[512] = "";

void axk_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
}

extern "C" const char* axk_last_error(void) { return g_error; }
extern "C" int axk_is_bf16(void) { return AXON_BF16; }
extern "C" int axk_elem_size(void) { return (int)sizeof(elem_t); }
