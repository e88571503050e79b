// core.hip — what every tier of the library shares: the error text behind zg_last_error, the HIP status plumbing of the
// ZG_HIP / ZG_REQUIRE macros, and the note of the last kernel instantiation a launcher picked.  No device state lives here, so
// a library that holds only one tier (the layered-model tier without the GPT-2 tiers) links this file and nothing of the others.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include "zg_common.h"

namespace zg {

static thread_local char g_err[512] = "";

int decode_paths_off() {
    const char* e = getenv("ZGPT2_DECODE_PATHS_OFF");
    return e ? atoi(e) : 0;
}

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

static thread_local char g_kernel[160] = "";
void note_kernel(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_kernel, sizeof(g_kernel), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char* what, const char* file, int line) {
    set_error("HIP error %d (%s) at %s:%d: %s", (int)e, hipGetErrorString(e), file, line, what);
    (void)hipGetLastError();
    return ZG_ERR_HIP;
}

const char* last_kernel_note() { return g_kernel; }

}  // namespace zg

extern "C" {

const char* zg_last_error(void) { return zg::g_err; }

int zg_debug_last_kernel(char* out, size_t n) {
    if (!out || n == 0) return ZG_ERR_ARG;
    snprintf(out, n, "%s", zg::last_kernel_note());
    return ZG_OK;
}

}  // extern "C"
