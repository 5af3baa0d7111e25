// Error reporting and version entry points of libvrwkv_hip.so.
#include "vrwkv_common.h"
#include <atomic>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <mutex>

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

// ---- tuning / testing switches: read from the environment once, changed afterwards only through the C ABI ----
namespace {
const char* const kOptionNames[N_OPTIONS] = {
    "biwkv_l", "biwkv_s", "biwkv_grid", "biwkv_no_stage", "biwkv_no_resident", "biwkv_bwd_serial",
    "wkv6_fwd_scalar", "wkv6_bwd_scalar", "wkv6_bwd_unfused",
};
std::atomic<int> g_options[N_OPTIONS];
std::once_flag g_options_once;

void load_options_from_env() {
    for (int i = 0; i < N_OPTIONS; ++i) {
        char env[64] = "VRWKV_";
        size_t n = strlen(env);
        for (const char* c = kOptionNames[i]; *c && n + 1 < sizeof(env); ++c) env[n++] = (char)toupper((unsigned char)*c);
        env[n] = 0;
        const char* v = getenv(env);
        g_options[i].store(v ? atoi(v) : 0, std::memory_order_relaxed);
    }
}
int find_option(const char* name) {
    if (!name) return -1;
    for (int i = 0; i < N_OPTIONS; ++i)
        if (!strcmp(name, kOptionNames[i])) return i;
    return -1;
}
}  // namespace

int option(Option o) {
    std::call_once(g_options_once, load_options_from_env);
    return g_options[o].load(std::memory_order_relaxed);
}

int device_cus() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
        n = 256;
    return n;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return VRWKV_OK;
    set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return VRWKV_LAUNCH_FAILED;
}
}  // namespace vrwkv

extern "C" int vrwkv_version(void) { return 200; }

extern "C" int vrwkv_set_option(const char* name, int value) {
    const int i = vrwkv::find_option(name);
    if (i < 0) {
        vrwkv::set_error("vrwkv_set_option: unknown option '%s'", name ? name : "(null)");
        return VRWKV_INVALID_ARG;
    }
    bool ok = value == 0 || value == 1;
    if (i == vrwkv::OPT_BIWKV_L) ok = value == 0 || value == 4 || value == 8 || value == 16 || value == 25 || value == 28;
    if (i == vrwkv::OPT_BIWKV_S) ok = value == 0 || (value >= 2 && value <= 8);
    if (i == vrwkv::OPT_BIWKV_GRID) ok = value >= 0;
    if (!ok) {
        vrwkv::set_error("vrwkv_set_option: %d is no value of '%s'", value, name);
        return VRWKV_INVALID_ARG;
    }
    (void)vrwkv::option((vrwkv::Option)i);          // the environment is read before the first change
    vrwkv::g_options[i].store(value, std::memory_order_relaxed);
    return VRWKV_OK;
}

extern "C" int vrwkv_get_option(const char* name, int* value) {
    const int i = vrwkv::find_option(name);
    if (i < 0 || !value) {
        vrwkv::set_error("vrwkv_get_option: unknown option '%s' or null result pointer", name ? name : "(null)");
        return VRWKV_INVALID_ARG;
    }
    *value = vrwkv::option((vrwkv::Option)i);
    return VRWKV_OK;
}
extern "C" const char* vrwkv_last_error(void) { return vrwkv::g_err; }
