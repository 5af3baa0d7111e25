// Error reporting and version entry points of libvrwkv_hip.so.
#include "vrwkv_common.h"

namespace vrwkv {
namespace {
thread_local char g_err[512] = "";
}

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return VRWKV_OK;
    set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return VRWKV_LAUNCH_FAILED;
}
}  // namespace vrwkv

extern "C" int vrwkv_version(void) { return 100; }
extern "C" const char* vrwkv_last_error(void) { return vrwkv::g_err; }
