// Shared host/device helpers of libqtensor_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qt {

// ---- host side: per-thread error slot and launch helpers --------------------------
void clear_error();
void set_error(int code, const char *fmt, ...);
int error_code();          // this host thread's slot (0: the last call went through)
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

__device__ __forceinline__ bool is_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// Round to nearest even; every NaN becomes 0x7FC0 (what torch's CPU cast produces).
__device__ __forceinline__ uint16_t float_to_bf16_bits(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// 16-byte global accesses with an optional streaming (nontemporal) hint: data that is touched
// once should not displace what the caches hold.  On MI355X the hint lifts a pure read stream
// from about 6.4 to 7.2 TB/s.
typedef float qt_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t qt_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t qt_u32x2 __attribute__((ext_vector_type(2)));
template <bool STREAM>
__device__ __forceinline__ float4 load_f32x4(const float *p) {
    const qt_f32x4 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const qt_f32x4 *>(p))
                              : *reinterpret_cast<const qt_f32x4 *>(p);
    return make_float4(v.x, v.y, v.z, v.w);
}
template <bool STREAM>
__device__ __forceinline__ uint4 load_u32x4(const void *p) {
    const qt_u32x4 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const qt_u32x4 *>(p))
                              : *reinterpret_cast<const qt_u32x4 *>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
template <bool STREAM>
__device__ __forceinline__ uint2 load_u32x2(const void *p) {
    const qt_u32x2 v = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const qt_u32x2 *>(p))
                              : *reinterpret_cast<const qt_u32x2 *>(p);
    return make_uint2(v.x, v.y);
}
template <bool STREAM>
__device__ __forceinline__ void store_f32x4(float *p, float4 y) {
    const qt_f32x4 v = {y.x, y.y, y.z, y.w};
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<qt_f32x4 *>(p));
    else *reinterpret_cast<qt_f32x4 *>(p) = v;
}
template <bool STREAM>
__device__ __forceinline__ void store_u32x2(void *p, uint2 y) {
    const qt_u32x2 v = {y.x, y.y};
    if (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<qt_u32x2 *>(p));
    else *reinterpret_cast<qt_u32x2 *>(p) = v;
}

// Makes this wave's LDS writes visible to its own later LDS reads.  Enough when every wave only
// touches a private staging area: no block barrier is needed then.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Maximum over aligned groups of G lanes (G = 8, 16, 32 or 64), delivered to every lane of the
// group.  Up to 16 lanes it is a DPP butterfly inside one row (no LDS); wider groups finish
// with cross-row permutes.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
template <int G>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
    static_assert(G == 8 || G == 16 || G == 32 || G == 64, "unsupported group width");
    v = max(v, dpp_u32<0xB1>(v));                 // quad_perm [1,0,3,2]
    v = max(v, dpp_u32<0x4E>(v));                 // quad_perm [2,3,0,1]
    v = max(v, dpp_u32<0x141>(v));                // row_half_mirror
    if (G >= 16) v = max(v, dpp_u32<0x140>(v));   // row_mirror
    if (G >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16, 64));
    if (G >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32, 64));
    return v;
}
#endif  // __HIPCC__

}  // namespace qt
