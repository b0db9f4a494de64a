// Correctly rounded fp32 division by a per-segment constant without the full IEEE sequence.
#pragma once

#include "qt_common.h"

namespace qt {
#if defined(__HIPCC__)

// Divisors the fast route accepts: 2^-60 <= a <= 2^60 (as bit patterns).
constexpr uint32_t kFastDivLo = 0x21800000u;
constexpr uint32_t kFastDivHi = 0x5d800000u;

// fl(1/a) for a in [2^-60, 2^60]: hardware reciprocal plus one Newton step.  Equality with IEEE
// division for every fp32 in that range is checked exhaustively on the device by
// qtensor_hip_check_fast_division (qt_selfcheck.hip).
__device__ __forceinline__ float exact_reciprocal(float a) {
    const float r0 = __builtin_amdgcn_rcpf(a);
    const float e = __builtin_fmaf(-a, r0, 1.0f);
    return __builtin_fmaf(e, r0, r0);
}

// Correctly rounded x / a for a in [2^-60, 2^60] and |x/a| >= 2^-40 (or x == 0), given
// r = fl(1/a): q0 = fl(x*r) is within one ulp, the residual x - q0*a is exact in fp32, and one
// more fma lands on the correctly rounded quotient (Markstein's division theorem).
__device__ __forceinline__ float quotient(float x, float a, float r) {
    const float q0 = x * r;
    const float rem = __builtin_fmaf(-q0, a, x);
    return __builtin_fmaf(rem, r, q0);
}

#endif  // __HIPCC__
}  // namespace qt
