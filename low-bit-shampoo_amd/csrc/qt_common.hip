// Host-side plumbing of libqtensor_hip.so: error slot, device queries, division constants.
#include "qt_common.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace qt {
namespace {
thread_local int t_error_code = 0;
thread_local char t_error_text[512] = "";
constexpr int kMaxDevices = 64;
int g_cu_count[kMaxDevices];  // 0 = not queried yet
}  // namespace

void clear_error() {
    t_error_code = 0;
    t_error_text[0] = '\0';
}

int error_code() { return t_error_code; }

void set_error(int code, const char *fmt, ...) {
    t_error_code = code;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_error_text, sizeof(t_error_text), fmt, ap);
    va_end(ap);
    fprintf(stderr, "libqtensor_hip: %s\n", t_error_text);
}

bool launch_ok(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return t_error_code == 0;
    set_error(kLaunchFailed, "%s: %s", what, hipGetErrorString(e));
    return false;
}

int compute_units() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    int n = __atomic_load_n(&g_cu_count[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        __atomic_store_n(&g_cu_count[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.divisor = d == 0 ? 1 : d;
    d = f.divisor;
    if ((d & (d - 1)) == 0) {   // power of two (d == 1 is short-circuited on the device)
        uint32_t lg = 0;
        while ((1u << lg) < d) ++lg;
        f.magic = 0x80000000u;
        f.shift = lg == 0 ? 0 : lg - 1;
        return f;
    }
    uint32_t s = 31;
    while (!(d >> s)) --s;      // s = floor(log2 d)
    f.magic = (uint32_t)(((uint64_t)1 << (32 + s)) / d + 1);
    f.shift = s;
    return f;
}

}  // namespace qt

extern "C" int qtensor_hip_version(void) { return 100; }
extern "C" int qtensor_hip_last_error(void) { return qt::t_error_code; }
extern "C" const char *qtensor_hip_last_error_string(void) { return qt::t_error_text; }
