// Device-side self checks and a calibration copy.  None of this is on the quantization path;
// it lets a test prove, on the GPU at hand, the arithmetic shortcut the quantizer relies on, and
// gives profilers a kernel of exactly known traffic.
#include "qt_common.h"
#include "qt_divide.h"

namespace qt {
namespace {

// For every fp32 divisor a with bit pattern in [lo, hi] (stride `stride`):
//   counts[0] += 1 if exact_reciprocal(a) != 1.0f / a
//   for x_per_a pseudo-random x with |x| <= a spread over 40 binades below a:
//     counts[1] += 1 if |x/a| >= 2^-40 and quotient(x, a, r) != x / a;  counts[2] += pairs tried
__global__ __launch_bounds__(256) void check_division_kernel(uint32_t lo, uint32_t hi, uint32_t stride, int x_per_a,
                                                             unsigned long long *__restrict__ counts) {
    const unsigned long long step = (unsigned long long)gridDim.x * blockDim.x * stride;
    unsigned long long bad_r = 0, bad_q = 0, tried = 0;
    for (unsigned long long b = lo + ((unsigned long long)blockIdx.x * blockDim.x + threadIdx.x) * stride; b <= hi; b += step) {
        const float a = __uint_as_float((uint32_t)b);
        const float r = exact_reciprocal(a);
        bad_r += __float_as_uint(r) != __float_as_uint(1.0f / a);
        unsigned long long s = b * 0x9E3779B97F4A7C15ull + 12345ull;
        for (int i = 0; i < x_per_a; ++i) {
            s ^= s >> 30; s *= 0xBF58476D1CE4E5B9ull; s ^= s >> 27; s *= 0x94D049BB133111EBull; s ^= s >> 31;
            const int ex = (int)((b >> 23) & 0xff) - (int)((s >> 23) % 40);
            if (ex < 1) continue;
            float x = __uint_as_float(((uint32_t)ex << 23) | (uint32_t)(s & 0x7fffff));
            if (x > a) x = a;
            if ((s >> 40) & 1) x = -x;
            const float want = x / a;
            ++tried;
            if (fabsf(want) >= 9.094947e-13f && __float_as_uint(quotient(x, a, r)) != __float_as_uint(want)) ++bad_q;
        }
    }
    if (bad_r) atomicAdd(&counts[0], bad_r);
    if (bad_q) atomicAdd(&counts[1], bad_q);
    atomicAdd(&counts[2], tried);
}

__global__ __launch_bounds__(256) void copy_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst, size_t n4) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

}  // namespace
}  // namespace qt

extern "C" void qtensor_hip_check_fast_division(uint32_t lo_bits, uint32_t hi_bits, uint32_t stride, int x_per_a,
                                                unsigned long long *counts, void *stream) {
    qt::clear_error();
    if (!counts || stride == 0 || lo_bits > hi_bits || lo_bits < qt::kFastDivLo || hi_bits > qt::kFastDivHi) {
        qt::set_error(qt::kBadArgument, "check_fast_division: need counts != NULL, stride >= 1 and "
                                        "0x21800000 <= lo <= hi <= 0x5d800000");
        return;
    }
    hipLaunchKernelGGL(qt::check_division_kernel, dim3(qt::compute_units() * 8), dim3(256), 0, (hipStream_t)stream,
                       lo_bits, hi_bits, stride, x_per_a, counts);
    qt::launch_ok("check_fast_division");
}

extern "C" void qtensor_hip_copy_f32(const float *src, float *dst, unsigned long long n, void *stream) {
    qt::clear_error();
    if (!src || !dst || n % 4 != 0 || !qt::is_aligned(src, 16) || !qt::is_aligned(dst, 16)) {
        qt::set_error(qt::kBadArgument, "copy_f32: need 16-byte aligned pointers and n divisible by 4");
        return;
    }
    if (n == 0) return;
    const size_t n4 = n / 4;
    const size_t blocks = (n4 + 255) / 256;
    const size_t cap = (size_t)qt::compute_units() * 4;
    hipLaunchKernelGGL(qt::copy_kernel, dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst), n4);
    qt::launch_ok("copy_f32");
}
