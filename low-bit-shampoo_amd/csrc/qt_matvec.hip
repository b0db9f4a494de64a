// Matrix-vector products for a whole stack of square fp32 matrices in one launch: out[b] = A[b] v[b].
// The power iteration that scales the ridge term of the inverse roots (optimizers/matrix_functions.py:21-48 of
// the reference: torch.mv per matrix and round) needs ten of them per stack; the stack is read once per
// product, so the launch is bound by memory bandwidth.
// One wave per row: 64 lanes x 16-byte loads along the row, eight partial sums per lane, a butterfly over the
// wave -- a fixed summation order, so the result does not depend on the grid.
#include "qt_common.h"

namespace qt {
namespace {

#define QT_GLOBAL __attribute__((address_space(1)))

__global__ __launch_bounds__(256) void matvec_kernel(const float *A, const float *v, float *out, int n, long long rows) {
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);       // over all matrices of the stack
    if (row >= rows) return;
    const long long b = row / n;
    const float *a = A + row * n, *x = v + b * n;
    float part[4] = {0.f, 0.f, 0.f, 0.f};
    if ((n & 3) == 0 && is_aligned16(a) && is_aligned16(x)) {
        int c = lane * 4;
        for (; c + 768 < n; c += 1024) {                                      // four loads in flight per lane
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const qt_f32x4 p = *(const QT_GLOBAL qt_f32x4 *)(a + c + 256 * i);
                const qt_f32x4 q = *(const QT_GLOBAL qt_f32x4 *)(x + c + 256 * i);
                part[i] = __builtin_fmaf(p.x, q.x, __builtin_fmaf(p.y, q.y, __builtin_fmaf(p.z, q.z, __builtin_fmaf(p.w, q.w, part[i]))));
            }
        }
        for (; c < n; c += 256) {
            const qt_f32x4 p = *(const QT_GLOBAL qt_f32x4 *)(a + c);
            const qt_f32x4 q = *(const QT_GLOBAL qt_f32x4 *)(x + c);
            part[0] = __builtin_fmaf(p.x, q.x, __builtin_fmaf(p.y, q.y, __builtin_fmaf(p.z, q.z, __builtin_fmaf(p.w, q.w, part[0]))));
        }
    } else {
        for (int c = lane; c < n; c += 64) part[0] = __builtin_fmaf(a[c], x[c], part[0]);
    }
    float sum = (part[0] + part[1]) + (part[2] + part[3]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) out[row] = sum;
}

}  // namespace
}  // namespace qt

extern "C" void qtensor_hip_matvec_batched(const float *a, const float *v, float *out, int n, int batch, void *stream) {
    using namespace qt;
    clear_error();
    if (!a || !v || !out) { set_error(kNullPointer, "matvec_batched: null pointer"); return; }
    if (n < 1 || batch < 1) { set_error(kBadArgument, "matvec_batched: need n >= 1 and batch >= 1 (got %d, %d)", n, batch); return; }
    const long long rows = (long long)n * batch;
    const long long blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffffLL) { set_error(kBadArgument, "matvec_batched: too many rows (%lld)", rows); return; }
    hipLaunchKernelGGL(matvec_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a, v, out, n, rows);
    launch_ok("matvec_batched");
}
