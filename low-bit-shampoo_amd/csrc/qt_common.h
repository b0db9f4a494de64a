// Shared host/device helpers of libqtensor_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qt {

// ---- host side: per-thread error slot and launch helpers --------------------------
void clear_error();
void set_error(int code, const char *fmt, ...);
// Records a failed launch (hipGetLastError) under `what`; returns true when all is well.
bool launch_ok(const char *what);
// Compute units of the current device (cached per device ordinal).
int compute_units();

enum ErrorCode : int {
    kOk = 0,
    kBadBlocksize = 1,
    kBadOrder = 2,
    kNullPointer = 3,
    kLaunchFailed = 4,
    kBadArgument = 5,
};

inline bool is_aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Exact floor(k / d) for k < 2^29 and 1 <= d < 2^15 as (mulhi(k, magic) >> shift).
struct FastDiv {
    uint32_t magic;
    uint32_t shift;
    uint32_t divisor;
};
FastDiv make_fastdiv(uint32_t d);

#if defined(__HIPCC__)
// ---- device side -------------------------------------------------------------------
__device__ __forceinline__ uint32_t fastdiv(uint32_t k, FastDiv f) {
    return f.divisor == 1 ? k : (__umulhi(k, f.magic) >> f.shift);
}

// Total order on fp32 bit patterns: negative values reversed below the positives.
__device__ __forceinline__ uint32_t float_to_key(float f) {
    uint32_t b = __float_as_uint(f);
    return b ^ (uint32_t)(((int32_t)b >> 31) | 0x80000000);
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// Round to nearest even; every NaN becomes 0x7FC0 (what torch's CPU cast produces).
__device__ __forceinline__ uint16_t float_to_bf16_bits(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Maximum over each aligned row of 16 lanes, delivered to all 16 (DPP, no LDS).
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
__device__ __forceinline__ uint32_t row16_max_u32(uint32_t v) {
    v = max(v, dpp_u32<0xB1>(v));   // quad_perm [1,0,3,2]
    v = max(v, dpp_u32<0x4E>(v));   // quad_perm [2,3,0,1]
    v = max(v, dpp_u32<0x141>(v));  // row_half_mirror
    v = max(v, dpp_u32<0x140>(v));  // row_mirror
    return v;
}
// Maximum over aligned groups of G lanes (G = 16, 32 or 64), delivered to every lane.
template <int G>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
    v = row16_max_u32(v);
    if (G >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16, 64));
    if (G >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32, 64));
    return v;
}
#endif  // __HIPCC__

}  // namespace qt
