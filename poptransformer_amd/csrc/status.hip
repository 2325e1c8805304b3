// Library status: version and the per-thread message of the last failure.
// The reference reports failures by throwing popart::error / poplar::poplar_error while the
// graph is being built (e.g. custom_ops/int4_to_half_custom_op.cpp:65-98); across a C ABI the
// same predicates become a negative return code plus this message.
#include "common.h"
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_last_error[512] = "";

void pta_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

extern "C" int pta_version(void) { return 100; }  // 0.1.0
extern "C" const char* pta_last_error(void) { return g_last_error; }
