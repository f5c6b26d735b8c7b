// Error channel and identification entry points of libxma_hip.so.
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace xma {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace xma

extern "C" {

const char* xma_last_error(void) { return xma::g_error; }
const char* xma_version(void) { return "0.1.0"; }
const char* xma_target_arch(void) { return "gfx950"; }
int xma_abi_version(void) { return XMA_ABI_VERSION; }

}  // extern "C"
