// Batched Cholesky factorisation and triangular solve for stacks of square fp32 matrices whose
// order is a multiple of 64: the two steps of a Cholesky QR round (R = chol(Q^T Q), Q <- Q R^-1),
// which replaces the QR factorisation the reference calls once per statistic and update
// (torch.linalg.qr at qtensor/utils.py:157 of the reference).
//
// Both are blocked with 64-wide panels.  The only arithmetic done outside the matrix-core GEMM
// (qtensor_hip_gemm) is the 64 x 64 diagonal block: one wave per matrix factors it in LDS and also
// inverts the factor, so that every panel solve becomes a product with that small inverse.
//   factor:  for each block row j:  U_jj = chol(G_jj);  U_j,> = U_jj^-T G_j,>;  G_>,> -= U_j,>^T U_j,>
//   solve :  for each block col j:  X_j = (Q_j - X_<j U_<j,j) U_jj^-1
// All launches go to the caller's stream; nothing is allocated or synchronised here.
#include "qt_common.h"

#include "qtensor_hip.h"

#include <initializer_list>

namespace qt {
namespace {

constexpr int NB = 64;

// One wave per matrix: upper Cholesky factor U (G = U^T U) of a 64 x 64 block and U^-1.
// Reads the upper triangle of G only.  A non-positive (or NaN) pivot sets info[b] = 1 and is
// replaced by 1; the factor of that matrix is then meaningless.
//
// Lane i keeps row i of the (full, symmetric) trailing matrix in registers.  Because the matrix
// stays symmetric, column k of step k is row k, i.e. the registers of lane k: they are broadcast
// with v_readlane, so the whole factorisation and the inversion of the factor run without LDS
// traffic or barriers (LDS only stages the block on the way in).
__device__ __forceinline__ float lane_value(float x, int lane) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(x), lane));
}

__global__ __launch_bounds__(NB) void cholesky64_kernel(const float *gram, long long g_stride, int ldg, float *u,
                                                        long long u_stride, int ldu, float *inv, long long inv_stride,
                                                        int *info) {
    __shared__ float stage[NB][NB + 1];
    const int b = blockIdx.x, lane = threadIdx.x;
    const float *G = gram + (long long)b * g_stride;
    for (int r = 0; r < NB; ++r) stage[r][lane] = G[(long long)r * ldg + lane];
    __syncthreads();
    float row[NB];                               // row `lane` of the symmetric matrix; ends as row `lane` of L = U^T
#pragma unroll
    for (int j = 0; j < NB; ++j) row[j] = j >= lane ? stage[lane][j] : stage[j][lane];
    bool ok = true;
#pragma unroll
    for (int k = 0; k < NB; ++k) {
        float d = lane_value(row[k], k);
        if (!(d > 0.0f)) { ok = false; d = 1.0f; }
        // a[i][j] -= a[i][k] a[k][j] / d: one multiply per lane, then a broadcast and a multiply-add per column
        const float t = row[k] / d;
#pragma unroll
        for (int j = k + 1; j < NB; ++j) row[j] -= t * lane_value(row[j], k);
        row[k] = row[k] / sqrtf(d);              // L[lane][k] (lanes above k: unused values)
    }
    // column `lane` of L^-1 by forward substitution; L[i][k] sits in lane i
    float x[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        float s = i == lane ? 1.0f : 0.0f;
#pragma unroll
        for (int k = 0; k < i; ++k) s -= lane_value(row[k], i) * x[k];
        x[i] = i >= lane ? s / lane_value(row[i], i) : 0.0f;
    }
    float *U = u + (long long)b * u_stride;
    float *I = inv + (long long)b * inv_stride + lane * NB;
#pragma unroll
    for (int r = 0; r < NB; ++r) U[(long long)r * ldu + lane] = r <= lane ? row[r] : 0.0f;        // U[r][lane] = L[lane][r]
#pragma unroll
    for (int c = 0; c < NB; c += 4)              // U^-1[lane][c] = L^-1[c][lane] = x[c] of this lane
        *reinterpret_cast<float4 *>(I + c) = make_float4(x[c], x[c + 1], x[c + 2], x[c + 3]);
    if (!ok && lane == 0) info[b] = 1;
}

qtensor_batch_ptr strided(const float *base, long long stride) {
    qtensor_batch_ptr p;
    p.base = base;
    p.list = nullptr;
    p.stride = stride;
    return p;
}

bool run(qtensor_gemm_desc &d, hipStream_t stream) {
    qtensor_hip_gemm(&d, stream);
    return qtensor_hip_last_error() == 0;
}

bool stack_args_ok(const char *what, int n, int batch, std::initializer_list<const void *> ptrs) {
    for (const void *p : ptrs)
        if (!p) { set_error(kNullPointer, "%s: null pointer", what); return false; }
    if (n < NB || n % NB != 0 || batch < 1 || batch > 65535 || (long long)n * n * batch >= (1LL << 40)) {
        set_error(kBadArgument, "%s: order must be a positive multiple of %d and 1 <= batch <= 65535 (got %d, %d)", what, NB, n, batch);
        return false;
    }
    return true;
}

}  // namespace
}  // namespace qt

extern "C" void qtensor_hip_cholesky_upper_batched(float *gram, float *u, float *inv, int *info, int n, int batch, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("cholesky_upper_batched", n, batch, {gram, u, inv, info})) return;
    hipStream_t stream = (hipStream_t)stream_v;
    const long long mat = (long long)n * n;
    const int blocks = n / NB;
    const long long inv_mat = (long long)blocks * NB * NB;
    for (int j = 0; j < blocks; ++j) {
        const int j0 = j * NB, j1 = j0 + NB, rest = n - j1;
        const long long corner = (long long)j0 * n + j0;
        float *inv_j = inv + (long long)j * NB * NB;
        hipLaunchKernelGGL(cholesky64_kernel, dim3(batch), dim3(NB), 0, stream, gram + corner, mat, n, u + corner, mat, n, inv_j,
                           inv_mat, info);
        if (!launch_ok("cholesky_upper_batched (diagonal block)")) return;
        if (rest == 0) break;
        const long long row = (long long)j0 * n + j1;
        qtensor_gemm_desc d = {};
        // U_j,> = U_jj^-T G_j,>
        d.M = NB; d.N = rest; d.K = NB; d.batch = batch;
        d.kind_a = QTENSOR_DENSE_T; d.kind_b = QTENSOR_DENSE; d.epilogue = QTENSOR_EPI_STORE;
        d.args.A = strided(inv_j, inv_mat); d.args.lda = NB;
        d.args.B = strided(gram + row, mat); d.args.ldb = n;
        d.args.C = strided(u + row, mat); d.args.ldc = n;
        if (!run(d, stream)) return;
        // G_>,> -= U_j,>^T U_j,>   (symmetric: upper tiles, mirrored)
        qtensor_gemm_desc t = {};
        t.M = rest; t.N = rest; t.K = NB; t.batch = batch;
        t.kind_a = QTENSOR_DENSE_T; t.kind_b = QTENSOR_DENSE; t.epilogue = QTENSOR_EPI_AXPBY_DENSE;
        t.args.A = strided(u + row, mat); t.args.lda = n;
        t.args.B = strided(u + row, mat); t.args.ldb = n;
        const long long next = (long long)j1 * n + j1;
        t.args.C = strided(gram + next, mat); t.args.ldc = n;
        t.args.E = strided(gram + next, mat); t.args.lde = n;
        t.args.alpha = -1.0f; t.args.beta = 1.0f;
        t.args.symmetric = 1;
        if (!run(t, stream)) return;
    }
}

extern "C" void qtensor_hip_solve_upper_right_batched(const float *q, const float *u, const float *inv, float *panel, float *x,
                                                      int rows, int n, int batch, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("solve_upper_right_batched", n, batch, {q, u, inv, panel, x})) return;
    if (rows < 1) { set_error(kBadArgument, "solve_upper_right_batched: rows must be positive"); return; }
    hipStream_t stream = (hipStream_t)stream_v;
    const long long mat = (long long)n * n, tall = (long long)rows * n;
    const int blocks = n / NB;
    const long long inv_mat = (long long)blocks * NB * NB;
    for (int j = 0; j < blocks; ++j) {
        const int j0 = j * NB;
        const float *rhs = q + j0;
        long long rhs_stride = tall;
        int rhs_ld = n;
        if (j > 0) {
            // panel = Q_j - X_<j U_<j,j
            qtensor_gemm_desc d = {};
            d.M = rows; d.N = NB; d.K = j0; d.batch = batch;
            d.kind_a = QTENSOR_DENSE; d.kind_b = QTENSOR_DENSE; d.epilogue = QTENSOR_EPI_AXPBY_DENSE;
            d.args.A = strided(x, tall); d.args.lda = n;
            d.args.B = strided(u + j0, mat); d.args.ldb = n;
            d.args.E = strided(q + j0, tall); d.args.lde = n;
            d.args.C = strided(panel, (long long)rows * NB); d.args.ldc = NB;
            d.args.alpha = -1.0f; d.args.beta = 1.0f;
            if (!run(d, stream)) return;
            rhs = panel; rhs_stride = (long long)rows * NB; rhs_ld = NB;
        }
        // X_j = panel U_jj^-1
        qtensor_gemm_desc s = {};
        s.M = rows; s.N = NB; s.K = NB; s.batch = batch;
        s.kind_a = QTENSOR_DENSE; s.kind_b = QTENSOR_DENSE; s.epilogue = QTENSOR_EPI_STORE;
        s.args.A = strided(rhs, rhs_stride); s.args.lda = rhs_ld;
        s.args.B = strided(inv + (long long)j * NB * NB, inv_mat); s.args.ldb = NB;
        s.args.C = strided(x + j0, tall); s.args.ldc = n;
        if (!run(s, stream)) return;
    }
}
