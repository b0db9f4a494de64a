// Batched Cholesky factorisation and triangular solve for stacks of square fp32 matrices whose
// order is a multiple of 64: the two steps of a Cholesky QR round (R = chol(Q^T Q), Q <- Q R^-1),
// which replaces the QR factorisation the reference calls once per statistic and update
// (torch.linalg.qr at qtensor/utils.py:157 of the reference).
//
// The only arithmetic done outside the matrix-core GEMM (qtensor_hip_gemm) is the 64 x 64 diagonal
// block: four waves per matrix factor it in registers and also invert the factor.
//   factor:  for each block row j:  U_jj = chol(G_jj);  U_j,> = U_jj^-T G_j,>;  G_>,> -= U_j,>^T U_j,>
//            (the last step for the rows of the current 256-row panel at once, for the rest per panel)
//   solve :  the inverted diagonal blocks are doubled up to 256 x 256 -- with blocks A, C already
//            inverted and B the block of U between them, [A^-1 B; 0 C^-1] gets -A^-1 B C^-1; every level is
//            two launches for all pairs of all matrices -- then, for each 256-wide column panel j,
//            X_j = (Q_j - X_<j U_<j,j) U_jj^-1; products with a triangular factor skip its zero part.
// All launches go to the caller's stream; nothing is allocated or synchronised here.
#include "qt_common.h"

#include "qtensor_hip.h"

#include <cstdlib>
#include <initializer_list>

namespace qt {
void gemm_with_tile(const qtensor_gemm_desc *d, hipStream_t stream, int tile);     // qt_gemm.hip
namespace {

constexpr int NB = 64;
constexpr int kFactorPanel = 256;      // rows factored between two updates of the whole trailing matrix
constexpr int kSolvePanel = 256;       // diagonal blocks of the factor are inverted up to this size, then panels of that width are solved

// One workgroup of four waves per matrix: upper Cholesky factor U (G = U^T U) of a 64 x 64 block and U^-1.
// Reads the upper triangle of G only.  A pivot that is not above `pivot_floor` is a column that depends on
// the ones before it up to the rounding noise of the Gram matrix.  With pivot_floor > 0 such a column is
// taken out of the factorisation: its pivot becomes the floor and the rest of its row of U zero (bit 1 of
// info[b] is set), so nothing of its noise reaches the columns after it; Q U^-1 still takes the earlier
// columns out of it and lifts what is left by 1 / sqrt(floor), and the next round treats it like any other
// column.  (Raising the pivot alone lets the noise grow geometrically through the trailing updates.)
// `inv` receives U^-1; `panel_inv`, if not null, the same with the dropped columns' rows of U^-T zeroed: the
// factor that turns G_j,> into the block row U_j,> with zero rows for the dropped columns.
// With pivot_floor == 0, and for a NaN pivot always, bit 0 of info[b] is set, the pivot is replaced by 1 and
// the factor of that matrix is meaningless.
// `set_aside`, if not null: the columns taken out are reported there (bit k of set_aside[b * aside_stride]) instead of in info, and
// their columns of `inv` are zero, so that Q inv has zero columns in their place for the caller to fill.
//
// Lane i of every wave stands for row i of the (full, symmetric) trailing matrix; wave w keeps the columns 16 w ..
// 16 w + 15 of that row in registers, and the same columns of the right-hand side e_i of the forward substitution,
// which ends as column i of L^-1 (L = U^T), so the inverse costs no second pass.  A right-looking factorisation in
// four blocks of sixteen columns: the wave that owns a block factors it alone (1 / sqrt(pivot) from v_rsq_f32 plus one
// Newton step; a[i][j] -= L[i][k] L[j][k], s[j] -= L[j][k] x[k] for its own columns j behind k), the waves behind it
// apply the block's sixteen steps to their columns from the copy in LDS.  (With one wave per matrix and all 64 columns
// in a lane's registers a step costs twice 64 - k multiply-adds per lane and the kernel 25-29 us; a barrier per step
// between four waves costs as much in waiting.)
//
// SCALED: `gram` is the Gram matrix S = P^T P of a panel whose columns are not of unit length yet.  The kernel factors
// D^-1 S D^-1 (D = the column lengths, from the diagonal of S) and `inv` receives D^-1 U^-1, so that P inv is the
// orthonormalised panel without a pass that rescales it first; u and panel_inv are not written.  With stand_in != 0
// a column whose squared length is not at least too_short (what projecting the earlier columns out has left of a
// unit column is rounding noise; a NaN counts) is set aside like a dropped one -- it takes no part in the
// factorisation, its column of inv is zero, its bit of set_aside is set -- whatever aside_pivots says; aside_pivots
// == 0 keeps the columns dropped for their pivot where they are (bit 1 of info) and reports only the short ones.
constexpr int LDC = NB + 4;                      // LDS row stride: rows stay 16-byte aligned
constexpr int kCholWaves = 4, kCholCols = NB / kCholWaves;

__device__ __forceinline__ float lane_value(float x, int lane) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(x), lane));
}

template <bool SCALED>
__global__ __launch_bounds__(NB * kCholWaves) void cholesky64_kernel(const float *gram, long long g_stride, int ldg, float *u,
                                                                     long long u_stride, int ldu, float *inv, long long inv_stride,
                                                                     int ldi, float *panel_inv, int *info, float pivot_floor,
                                                                     unsigned long long *set_aside, int aside_stride,
                                                                     float too_short, int stand_in, int aside_pivots) {
    __shared__ __attribute__((aligned(16))) float cols[NB][LDC];
    __shared__ __attribute__((aligned(16))) float handed[NB][2][NB];      // [k][column k of L | x[k] of every row][row]
    __shared__ float lengths[NB];
    __shared__ unsigned long long s_dropped[kCholWaves];
    __shared__ int s_failed[kCholWaves];
    const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c0 = wave * kCholCols;
    const float *G = gram + (long long)b * g_stride;
    for (int r = wave; r < NB; r += kCholWaves) cols[r][lane] = G[(long long)r * ldg + lane];
    __syncthreads();
    float row[kCholCols];                        // columns c0 .. c0 + 15 of row `lane` of the symmetric matrix; end as L[lane][c0 ..]
    float s[kCholCols];                          // the same columns of the right-hand side e_lane; end as L^-1[c0 ..][lane]
    float own_scale = 1.0f;                      // SCALED: 1 / length of column `lane` (0 for a column set aside or of length 0)
    unsigned long long early = 0;                // SCALED: the columns set aside for their length (uniform over the workgroup)
    bool shrunk = false;                         // SCALED: a column kept although the projections left little of it
    if constexpr (SCALED) {
        const float norm2 = cols[lane][lane];
        const bool aside = stand_in != 0 && !(norm2 >= too_short);
        own_scale = 0.0f;
        if (!aside) {
            if (norm2 > 0.0f) {
                const float r = __builtin_amdgcn_rsqf(norm2);
                own_scale = r * __builtin_fmaf(-0.5f * norm2 * r, r, 1.5f);
            } else if (norm2 != norm2) {
                own_scale = norm2;               // a NaN column fails the factorisation, as it did when it was rescaled first
            }
        }
        early = __ballot(aside);
        // Without stand-ins (the last pass over a panel) a column that the projections have shortened that much is
        // kept and lifted back to unit length, and whatever rounding left in it with it: the result can be off by
        // the rounding error over what was left, so the matrix is flagged (bit 1 of info) and the caller tests it.
        // (A column that depends on the ones before it gets here when an earlier pass could not tell: next to an
        // ill-conditioned panel that one Cholesky QR round had not made orthonormal yet.)
        shrunk = stand_in == 0 && __ballot(!(norm2 >= too_short)) != 0;
        if (wave == 0) lengths[lane] = own_scale;
        __syncthreads();
    }
#pragma unroll
    for (int jj = 0; jj < kCholCols; ++jj) {
        const int j = c0 + jj;
        row[jj] = j >= lane ? cols[lane][j] : cols[j][lane];
        if constexpr (SCALED) {
            const bool out = ((early >> j) & 1ull) || ((early >> lane) & 1ull);
            row[jj] = out ? (j == lane ? 1.0f : 0.0f) : row[jj] * own_scale * lengths[j];
        }
        s[jj] = j == lane ? 1.0f : 0.0f;
    }
    bool ok = true;
    uint32_t taken_out = 0;                      // which of its sixteen columns this wave took out of the factorisation (uniform over the wave)
    // Four phases.  In phase p wave p factors its sixteen columns on its own -- step k: pivot, column k of L, then its
    // columns behind k at once, their L[j][k] through v_readlane -- and leaves every column of L, with the
    // substitution's x[k] of every row, in LDS; behind the barrier the waves after it bring their columns up to date
    // with those sixteen steps (the same multiply-adds in the same order as step by step), and the next one goes on.
#pragma unroll
    for (int p = 0; p < kCholWaves; ++p) {
        if (wave == p) {                         // (uniform over the wave)
#pragma unroll
            for (int kk = 0; kk < kCholCols; ++kk) {
                const int k = p * kCholCols + kk;
                float d = lane_value(row[kk], k);
                bool drop = false;
                if (!(d > pivot_floor)) {
                    if (pivot_floor > 0.0f && d == d) { drop = true; taken_out |= 1u << kk; d = pivot_floor; }
                    else { ok = false; d = 1.0f; }
                }
                float r = __builtin_amdgcn_rsqf(d);
                r = r * __builtin_fmaf(-0.5f * d * r, r, 1.5f);
                float l = row[kk] * r;           // L[lane][k] (lanes above k: unused values)
                if (drop) l = lane == k ? d * r : 0.0f;   // sqrt(floor) on the diagonal, nothing below it
                row[kk] = l;
                s[kk] *= r;                      // x[k] = s[k] / L[k][k]
                const float xk = s[kk];
                handed[k][0][lane] = l;
                handed[k][1][lane] = xk;
#pragma unroll
                for (int jj = kk + 1; jj < kCholCols; ++jj) {
                    const float v = lane_value(l, p * kCholCols + jj);     // L[j][k]
                    row[jj] = __builtin_fmaf(-l, v, row[jj]);
                    s[jj] = __builtin_fmaf(-v, xk, s[jj]);
                }
            }
        }
        if (p + 1 == kCholWaves) break;
        __syncthreads();
        if (wave > p) {
#pragma unroll
            for (int kk = 0; kk < kCholCols; ++kk) {
                const int k = p * kCholCols + kk;
                const float l = handed[k][0][lane], xk = handed[k][1][lane];
#pragma unroll
                for (int q = 0; q < kCholCols; q += 4) {
                    const float4 v4 = *reinterpret_cast<const float4 *>(&handed[k][0][c0 + q]);     // L[j][k] for four columns j
                    const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        row[q + e] = __builtin_fmaf(-l, v[e], row[q + e]);
                        s[q + e] = __builtin_fmaf(-v[e], xk, s[q + e]);
                    }
                }
            }
        }
    }
    if (lane == 0) { s_dropped[wave] = (unsigned long long)taken_out << c0; s_failed[wave] = ok ? 0 : 1; }
    __syncthreads();
    unsigned long long dropped = 0;
    int failed = 0;
#pragma unroll
    for (int w = 0; w < kCholWaves; ++w) { dropped |= s_dropped[w]; failed |= s_failed[w]; }
    float *I = inv + (long long)b * inv_stride + (long long)lane * ldi + c0;
    if constexpr (!SCALED) {
        float *U = u + (long long)b * u_stride;
#pragma unroll
        for (int jj = 0; jj < kCholCols; ++jj)                                      // U[r][lane] = L[lane][r]
            U[(long long)(c0 + jj) * ldu + lane] = c0 + jj <= lane ? row[jj] : 0.0f;
    }
    if (set_aside != nullptr) {
        const unsigned long long out = SCALED ? early | (aside_pivots != 0 ? dropped : 0ull) : dropped;
#pragma unroll
        for (int jj = 0; jj < kCholCols; ++jj)
            if ((out >> (c0 + jj)) & 1ull) s[jj] = 0.0f;
        if (threadIdx.x == 0) set_aside[(long long)b * aside_stride] = out;
        if (!SCALED || aside_pivots != 0) dropped = 0;
    }
    if constexpr (SCALED) {
#pragma unroll
        for (int jj = 0; jj < kCholCols; ++jj) s[jj] *= own_scale;                 // row `lane` of D^-1 U^-1
    }
#pragma unroll
    for (int jj = 0; jj < kCholCols; jj += 4)    // U^-1[lane][c] = L^-1[c][lane] = s[c] of this lane (zero for c < lane)
        *reinterpret_cast<float4 *>(I + jj) = make_float4(s[jj], s[jj + 1], s[jj + 2], s[jj + 3]);
    if (!SCALED && panel_inv != nullptr) {
        float *P = panel_inv + (long long)b * inv_stride + (long long)lane * ldi + c0;
#pragma unroll
        for (int jj = 0; jj < kCholCols; jj += 4) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (dropped >> (c0 + jj + e)) & 1ull ? 0.0f : s[jj + e];
            *reinterpret_cast<float4 *>(P + jj) = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
    if ((failed != 0 || dropped != 0 || shrunk) && threadIdx.x == 0) info[b] |= (failed != 0 ? 1 : 0) | (dropped != 0 || shrunk ? 2 : 0);
}

// How far a stack of Gram matrices is from the identity: per matrix max |G - I| and ||G - I||_F^2, in
// one pass over the stack and in a fixed summation order (each block reduces a band of rows, a second
// kernel adds the bands of a matrix in order).  A NaN anywhere gives NaN in both.
constexpr int kBands = 32;

__global__ __launch_bounds__(256) void deviation_bands_kernel(const float *gram, int n, int rows_per_band, float *partial) {
    const int band = blockIdx.x, b = blockIdx.y;
    const float *G = gram + (long long)b * n * n;
    const int r0 = band * rows_per_band, r1 = min(r0 + rows_per_band, n);
    const int quads = n / 4;                                     // n is a multiple of 64
    uint32_t worst = 0;                                          // bits of the largest |e| (a NaN has the largest bits)
    float sum = 0.0f;
    for (int q = threadIdx.x; q < (r1 - r0) * quads; q += 256) {
        const int r = r0 + q / quads, c = (q % quads) * 4;
        const float4 g = *reinterpret_cast<const float4 *>(G + (long long)r * n + c);
        const float e[4] = {g.x - (r == c ? 1.0f : 0.0f), g.y - (r == c + 1 ? 1.0f : 0.0f), g.z - (r == c + 2 ? 1.0f : 0.0f),
                            g.w - (r == c + 3 ? 1.0f : 0.0f)};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            worst = max(worst, __float_as_uint(e[k]) & 0x7fffffffu);
            sum = __builtin_fmaf(e[k], e[k], sum);
        }
    }
    __shared__ uint32_t s_worst[256];
    __shared__ float s_sum[256];
    s_worst[threadIdx.x] = worst;
    s_sum[threadIdx.x] = sum;
    __syncthreads();
    for (int step = 128; step >= 1; step >>= 1) {
        if ((int)threadIdx.x < step) {
            s_worst[threadIdx.x] = max(s_worst[threadIdx.x], s_worst[threadIdx.x + step]);
            s_sum[threadIdx.x] += s_sum[threadIdx.x + step];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partial[((long long)b * kBands + band) * 2] = __uint_as_float(s_worst[0]);
        partial[((long long)b * kBands + band) * 2 + 1] = s_sum[0];
    }
}

__global__ __launch_bounds__(64) void deviation_total_kernel(const float *partial, int bands, int batch, float *out) {
    const int b = blockIdx.x * 64 + threadIdx.x;
    if (b >= batch) return;
    uint32_t worst = 0;
    float sum = 0.0f;
    for (int band = 0; band < bands; ++band) {
        worst = max(worst, __float_as_uint(partial[((long long)b * kBands + band) * 2]));
        sum += partial[((long long)b * kBands + band) * 2 + 1];
    }
    out[2 * b] = __uint_as_float(worst);
    out[2 * b + 1] = sum;
}

// dst[b] = src[b] for the matrices whose flag is set; the blocks of all others leave at once.
__global__ __launch_bounds__(256) void copy_flagged_kernel(float *dst, const float *src, const int *flags, long long quads) {
    const int b = blockIdx.y;
    if (flags[b] == 0) return;
    const float4 *s = reinterpret_cast<const float4 *>(src) + (long long)b * quads;
    float4 *d = reinterpret_cast<float4 *>(dst) + (long long)b * quads;
    for (long long q = blockIdx.x * 256ll + threadIdx.x; q < quads; q += (long long)gridDim.x * 256) d[q] = s[q];
}

// out[b][j] = sum_i A[b][i][j] B[b][i][j] for two stacks of n x n matrices: the diagonal of A^T B without the
// product (the Rayleigh quotients diag(Q^T (L Q)) of a subspace iteration step).  A workgroup takes 64 columns of
// one matrix: 16 lanes cover them with 16-byte loads, the 16 groups of lanes take every sixteenth row, four rows in
// flight per thread, and the partial sums are added in a fixed order.
__global__ __launch_bounds__(256) void column_dots_kernel(const float *A, const float *B, float *out, int n) {
    const int c4 = (threadIdx.x & 15) * 4, g = threadIdx.x >> 4, b = blockIdx.y;
    const long long base = (long long)b * n * n + blockIdx.x * 64 + c4;
    const float *pa = A + base, *pb = B + base;
    float4 part[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) part[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    int r = g;
    for (; r + 48 < n; r += 64) {
        float4 x[4], y[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[i] = *reinterpret_cast<const float4 *>(pa + (long long)(r + 16 * i) * n);
            y[i] = *reinterpret_cast<const float4 *>(pb + (long long)(r + 16 * i) * n);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            part[i].x = __builtin_fmaf(x[i].x, y[i].x, part[i].x);
            part[i].y = __builtin_fmaf(x[i].y, y[i].y, part[i].y);
            part[i].z = __builtin_fmaf(x[i].z, y[i].z, part[i].z);
            part[i].w = __builtin_fmaf(x[i].w, y[i].w, part[i].w);
        }
    }
    for (; r < n; r += 16) {
        const float4 x = *reinterpret_cast<const float4 *>(pa + (long long)r * n), y = *reinterpret_cast<const float4 *>(pb + (long long)r * n);
        part[0].x = __builtin_fmaf(x.x, y.x, part[0].x);
        part[0].y = __builtin_fmaf(x.y, y.y, part[0].y);
        part[0].z = __builtin_fmaf(x.z, y.z, part[0].z);
        part[0].w = __builtin_fmaf(x.w, y.w, part[0].w);
    }
    __shared__ float sums[16][64];
    sums[g][c4 + 0] = (part[0].x + part[1].x) + (part[2].x + part[3].x);
    sums[g][c4 + 1] = (part[0].y + part[1].y) + (part[2].y + part[3].y);
    sums[g][c4 + 2] = (part[0].z + part[1].z) + (part[2].z + part[3].z);
    sums[g][c4 + 3] = (part[0].w + part[1].w) + (part[2].w + part[3].w);
    __syncthreads();
    if (threadIdx.x < 64) {
        const int l = threadIdx.x;
        float total = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) total += sums[k][l];
        out[(long long)b * n + blockIdx.x * 64 + l] = total;
    }
}

// out[b] (64 x 64, rows 64 floats apart) = A_b^T B_b for two panels of 64 columns and n rows (n a multiple of 64, rows
// ld floats apart) of every matrix of a stack: the Gram matrix of a panel (A == B; upper_only: the block below the
// diagonal is not computed) or the coefficients of a panel on its neighbour.  grid (32 x 32 blocks of the result,
// batch); the four waves of a workgroup take a quarter of the rows each and add their blocks up in a fixed order.
// The operands go from memory straight into the fp32 matrix instruction (v_mfma_f32_32x32x2f32: lane l supplies column
// l % 32 of its block and row l / 32 of a pair of rows), 16 rows per group of loads, three groups in flight.
// What bounds it is the number of half rows (128 bytes, 4 KB apart) it asks memory for -- 20 us for 99 panels of 1024
// rows, where one pass over the same bytes in whole rows takes 5: sixteen waves per workgroup (23 us) or one
// workgroup per matrix (33 us: rows 4 KB apart share a set of the first-level cache) do not change that.
constexpr int kNormChunks = 8;
constexpr int kPanelGroup = 8;                   // matrix instructions (pairs of rows) per group of loads

typedef float qt_acc16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void panel_product_kernel(const float *A, const float *B, long long stride, int ld, int n,
                                                            float *out, long long out_stride, int upper_only) {
    const int b = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int bi = upper_only ? (int)(blockIdx.x == 2) : (int)(blockIdx.x >> 1);
    const int bj = upper_only ? (int)(blockIdx.x >= 1) : (int)(blockIdx.x & 1);
    const int rows = n / 4, groups = rows / (2 * kPanelGroup);                 // (n is a multiple of 64)
    const long long first = (long long)b * stride + (long long)(wave * rows + (lane >> 5)) * ld + (lane & 31);
    const float *pa = A + first + 32 * bi, *pb = B + first + 32 * bj;
    // (no branches between the loads and the matrix instructions: the compiler then counts the loads in flight exactly
    // and waits for no more than the group it is about to use)
    float a[4][kPanelGroup], c[4][kPanelGroup];
    auto load = [&](int buf, int group) {
        const long long at = (long long)min(group, groups - 1) * (2 * kPanelGroup) * ld;   // (past the end: a load nobody uses)
#pragma unroll
        for (int m = 0; m < kPanelGroup; ++m) {
            a[buf][m] = pa[at + (long long)(2 * m) * ld];
            c[buf][m] = pb[at + (long long)(2 * m) * ld];
        }
    };
    qt_acc16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    auto multiply = [&](int buf) {
#pragma unroll
        for (int m = 0; m < kPanelGroup; ++m) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[buf][m], c[buf][m], acc, 0, 0, 0);
    };
    load(0, 0);
    load(1, 1);
    load(2, 2);
    int g = 0;
    for (; g + 4 <= groups; g += 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            load((i + 3) & 3, g + i + 3);
            multiply(i);
        }
    }
    if (g < groups) {                                                          // up to three groups are left, in the buffers 0, 1, 2
        multiply(0);
        if (g + 1 < groups) {
            multiply(1);
            if (g + 2 < groups) multiply(2);
        }
    }
    __shared__ float part[4][16][64];
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wave][r][lane] = acc[r];
    __syncthreads();
    float *O = out + (long long)b * out_stride;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int r = 4 * wave + q;                                            // element r of a lane: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
        const float sum = (part[0][r][lane] + part[1][r][lane]) + (part[2][r][lane] + part[3][r][lane]);
        O[(32 * bi + 8 * wave + 4 * (lane >> 5) + q) * NB + 32 * bj + (lane & 31)] = sum;
    }
}

// The columns that the first pass over an outer panel set aside (bit j of aside[b * aside_stride + p]: column 64 p + j of
// the panel, a zero column by now) take the same columns of `fill`; bit 2 of info[b] is set.  Launched over
// (kNormChunks row chunks, batch); threads take a column and every fourth row of the chunk.
__global__ __launch_bounds__(256) void fill_aside_kernel(float *panel, long long stride, int ld, int n, int panels, int aside_stride,
                                                         const unsigned long long *aside, const float *fill, int fill_ld, int *info) {
    const int chunk = blockIdx.x, b = blockIdx.y, c = threadIdx.x & 63, g = threadIdx.x >> 6;
    float *P = panel + (long long)b * stride;
    const int rows = (n + kNormChunks - 1) / kNormChunks, r0 = chunk * rows, r1 = min(r0 + rows, n);
    bool any = false;
    for (int p = 0; p < panels; ++p) {
        const unsigned long long m = aside[(long long)b * aside_stride + p];
        if (m == 0) continue;
        any = true;
        if ((m >> c) & 1ull)
            for (int r = r0 + g; r < r1; r += 4) P[(long long)r * ld + p * NB + c] = fill[(long long)r * fill_ld + p * NB + c];
    }
    if (any && chunk == 0 && threadIdx.x == 0) atomicOr(info + b, 4);
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

// The same with the tile shape chosen here (0 = 128 x 128, 2 = 64 x 128): for the sweep's projections, where measured
// times and the product kernel's cost model part ways.
bool run_tiled(qtensor_gemm_desc &d, hipStream_t stream, int tile) {
    gemm_with_tile(&d, stream, tile);
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

extern "C" void qtensor_hip_cholesky_upper_batched(float *gram, float *u, float *x, int *info, int n, int batch, void *stream_v) {
    qtensor_hip_cholesky_upper_floor_batched(gram, u, x, info, n, batch, 0.0f, stream_v);
}

extern "C" void qtensor_hip_cholesky_upper_floor_batched(float *gram, float *u, float *x, int *info, int n, int batch,
                                                         float pivot_floor, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("cholesky_upper_batched", n, batch, {gram, u, x, info})) return;
    if (!(pivot_floor >= 0.0f)) { set_error(kBadArgument, "cholesky_upper_batched: the pivot floor must not be negative"); return; }
    hipStream_t stream = (hipStream_t)stream_v;
    const long long mat = (long long)n * n;
    // Two levels of blocking: inside a panel of kFactorPanel rows the 64-row steps update only the rest of
    // the panel's rows (thin strips); the matrix below the panel gets the whole panel at once, with a k
    // range four times as long -- a quarter of the passes over the trailing matrix.
    for (int p0 = 0; p0 < n; p0 += kFactorPanel) {
        const int p1 = p0 + kFactorPanel < n ? p0 + kFactorPanel : n;
        for (int j0 = p0; j0 < p1; j0 += NB) {
            const int j1 = j0 + NB, rest = n - j1;
            const long long corner = (long long)j0 * n + j0;
            // (the block of u right below the diagonal block is free: it takes the factor for the block row)
            float *panel_inv = rest > 0 ? u + (long long)j1 * n + j0 : nullptr;
            hipLaunchKernelGGL(cholesky64_kernel<false>, dim3(batch), dim3(NB * kCholWaves), 0, stream, gram + corner, mat, n, u + corner, mat, n,
                               x + corner, mat, n, panel_inv, info, pivot_floor, (unsigned long long *)nullptr, 0, 0.0f, 0, 0);
            if (!launch_ok("cholesky_upper_batched (diagonal block)")) return;
            if (rest == 0) break;
            const long long row = (long long)j0 * n + j1;
            qtensor_gemm_desc d = {};
            // U_j,> = U_jj^-T G_j,>  (zero rows for columns taken out of the factorisation)
            d.M = NB; d.N = rest; d.K = NB; d.batch = batch;
            d.kind_a = QTENSOR_DENSE_T; d.kind_b = QTENSOR_DENSE; d.epilogue = QTENSOR_EPI_STORE;
            d.args.A = strided(panel_inv, mat); d.args.lda = n;
            d.args.B = strided(gram + row, mat); d.args.ldb = n;
            d.args.C = strided(u + row, mat); d.args.ldc = n;
            if (!run(d, stream)) return;
            if (j1 < p1) {
                // the other rows of the panel: G_[j1,p1),[j1,n) -= U_j,[j1,p1)^T U_j,[j1,n)
                qtensor_gemm_desc t = {};
                t.M = p1 - j1; t.N = rest; t.K = NB; t.batch = batch;
                t.kind_a = QTENSOR_DENSE_T; t.kind_b = QTENSOR_DENSE; t.epilogue = QTENSOR_EPI_AXPBY_DENSE;
                t.args.A = strided(u + row, mat); t.args.lda = n;
                t.args.B = strided(u + row, mat); t.args.ldb = n;
                const long long next = (long long)j1 * n + j1;
                t.args.C = strided(gram + next, mat); t.args.ldc = n;
                t.args.E = strided(gram + next, mat); t.args.lde = n;
                t.args.alpha = -1.0f; t.args.beta = 1.0f;
                if (!run(t, stream)) return;
            }
        }
        if (p1 < n) {
            // below the panel: G_>,> -= U_P,>^T U_P,>   (symmetric: upper tiles, mirrored)
            qtensor_gemm_desc t = {};
            t.M = n - p1; t.N = n - p1; t.K = p1 - p0; t.batch = batch;
            t.kind_a = QTENSOR_DENSE_T; t.kind_b = QTENSOR_DENSE; t.epilogue = QTENSOR_EPI_AXPBY_DENSE;
            const long long rows = (long long)p0 * n + p1;
            t.args.A = strided(u + rows, mat); t.args.lda = n;
            t.args.B = strided(u + rows, mat); t.args.ldb = n;
            const long long next = (long long)p1 * n + p1;
            t.args.C = strided(gram + next, mat); t.args.ldc = n;
            t.args.E = strided(gram + next, mat); t.args.lde = n;
            t.args.alpha = -1.0f; t.args.beta = 1.0f;
            t.args.symmetric = 1;
            if (!run(t, stream)) return;
        }
    }
}

namespace qt {
namespace {

// State of one block Gram-Schmidt sweep over a stack (see qtensor_hip_block_gram_schmidt_batched).
struct Sweep {
    float *q, *w, *gram, *u, *x;
    const float *fill;
    int *info;
    int n, batch, w_cols;
    float pivot_floor, null_norm2;
    hipStream_t stream;
    bool replace;                                             // columns a first pass finds dependent inside their panel are replaced too
    long long mat() const { return (long long)n * n; }
    // With stand-in columns the tail of w holds, per matrix and 64-column panel of the current outer panel, which
    // columns the pass before set aside (w_cols / 64 words of 64 bits per matrix)
    long long w_floats() const { return (long long)batch * n * w_cols - (fill != nullptr ? 2LL * batch * (w_cols / NB) : 0); }
    unsigned long long *aside_words() const { return reinterpret_cast<unsigned long long *>(w + w_floats()); }

    // columns [c0, c0 + width) -= Q[:, a0:c0] (Q[:, a0:c0]^T columns): the columns a0..c0 are orthonormal
    bool project(int a0, int c0, int width) {
        const int k = c0 - a0;
        if (k <= 0) return true;
        // The coefficients of matrix b sit k * width floats apart; what is left of w behind them takes the partial
        // products when the product is cut along k (one 64 x 64 tile per matrix and a k range of n: few, long workgroups).
        // Only for a panel against its neighbour: cutting the products against all earlier panels as well is a little
        // faster for one stack alone and costs the optimizer step, where three stacks share the device, a third.
        const long long w_stride = (long long)k * width, w_used = w_stride * batch, w_all = w_floats();
        qtensor_gemm_desc p = {};                             // W = Q_a^T Y
        p.M = k; p.N = width; p.K = n; p.batch = batch;
        p.kind_a = QTENSOR_DENSE_T; p.kind_b = QTENSOR_DENSE; p.epilogue = QTENSOR_EPI_STORE;
        p.args.A = strided(q + a0, mat()); p.args.lda = n;
        p.args.B = strided(q + c0, mat()); p.args.ldb = n;
        p.args.C = strided(w, w_stride); p.args.ldc = width;
        if (k <= NB && width <= NB && w_all > w_used) {
            p.args.workspace = w + w_used;
            p.args.workspace_floats = w_all - w_used;
        }
        // Tile shapes by measurement (a stack of 99 matrices of order 1024, seven outer panels of a pass): the coefficients
        // -- few output tiles, a long k -- take 685 us with tiles of 128 x 128 (cut along k where that shape leaves units
        // idle) against 773 with what the product's cost model picks; the application 771 us with tiles of 64 rows and the
        // panel's full width against 800 (136 of order 768: 389 against 441 and 424 against 448; 50 of order 1024: 384
        // against 419 and 388 against 435).  Smaller stacks are left to the model, which is as good or better there.
        const bool wide = width == 2 * NB && (long long)batch * n >= 49152;
        if (!(wide ? run_tiled(p, stream, 0) : run(p, stream))) return false;
        qtensor_gemm_desc r = {};                             // Y -= Q_a W
        r.M = n; r.N = width; r.K = k; r.batch = batch;
        r.kind_a = QTENSOR_DENSE; r.kind_b = QTENSOR_DENSE; r.epilogue = QTENSOR_EPI_AXPBY_DENSE;
        r.args.A = strided(q + a0, mat()); r.args.lda = n;
        r.args.B = strided(w, w_stride); r.args.ldb = width;
        r.args.C = strided(q + c0, mat()); r.args.ldc = n;
        r.args.E = strided(q + c0, mat()); r.args.lde = n;
        r.args.alpha = -1.0f; r.args.beta = 1.0f;
        return wide ? run_tiled(r, stream, 2) : run(r, stream);
    }

    // The 64 columns from c0 on, in pass `pass` of `passes` over their outer panel (which starts at column a0): take the
    // columns a0..c0 out, then one Cholesky QR round inside -- Gram matrix of the panel as it is (one launch that reads
    // it once), factorisation of that matrix scaled to a unit diagonal (the columns' lengths are on the diagonal), and
    // the panel times D^-1 U^-1: three launches, two passes over the panel.
    // Stand-in columns: in every pass but the last a column that the projections have left shorter than a threshold
    // -- sqrt(null_norm2) in the first pass, where it was a unit column before them and what is left is rounding
    // noise; a half in the later ones, where it was orthonormalised a pass earlier and losing most of its length again
    // means it was noise then -- leaves the pass as a zero column and comes back as its column of `fill` before the
    // next pass (fill_aside_kernel).  In replace mode so do the columns whose pivot inside the panel is at or below
    // the floor.
    bool panel(int a0, int c0, int pass, int passes) {
        float *panel_ptr = q + c0;
        const bool more = pass + 1 < passes;
        const bool stand_in = fill != nullptr && more;
        // (word (c0 - a0) / 64 of the outer panel, matrices w_cols / 64 words apart -- see fill_aside_kernel)
        unsigned long long *aside = stand_in ? aside_words() + (c0 - a0) / NB : nullptr;
        const float too_short = pass == 0 ? null_norm2 : 0.25f;
        // The last pass of replace mode normalises whatever has a pivot above the noise of the Gram matrix: a stand-in
        // column for one of the last columns of a matrix has little room left (the complement of a thousand columns in
        // a space of as many dimensions), which is a small pivot and no dependence.
        const float floor_here = replace && !more && pivot_floor > 1e-6f ? 1e-6f : pivot_floor;
        const long long small = (long long)NB * NB;
        if (c0 - a0 == NB) {
            // against the one neighbour inside the outer panel: coefficients in one launch, straight from the panels
            hipLaunchKernelGGL(panel_product_kernel, dim3(4, batch), dim3(256), 0, stream, q + a0, panel_ptr, mat(), n, n, w, small, 0);
            if (!launch_ok("block_gram_schmidt_batched (coefficients)")) return false;
            qtensor_gemm_desc r = {};                         // Y -= Q_a W
            r.M = n; r.N = NB; r.K = NB; r.batch = batch;
            r.kind_a = QTENSOR_DENSE; r.kind_b = QTENSOR_DENSE; r.epilogue = QTENSOR_EPI_AXPBY_DENSE;
            r.args.A = strided(q + a0, mat()); r.args.lda = n;
            r.args.B = strided(w, small); r.args.ldb = NB;
            r.args.C = strided(panel_ptr, mat()); r.args.ldc = n;
            r.args.E = strided(panel_ptr, mat()); r.args.lde = n;
            r.args.alpha = -1.0f; r.args.beta = 1.0f;
            if (!run(r, stream)) return false;
        } else if (!project(a0, c0, NB)) {
            return false;
        }
        hipLaunchKernelGGL(panel_product_kernel, dim3(3, batch), dim3(256), 0, stream, panel_ptr, panel_ptr, mat(), n, n, gram, small, 1);
        hipLaunchKernelGGL(cholesky64_kernel<true>, dim3(batch), dim3(NB * kCholWaves), 0, stream, gram, small, NB, (float *)nullptr, small, NB, x,
                           small, NB, (float *)nullptr, info, floor_here, aside, w_cols / NB, too_short, stand_in ? 1 : 0,
                           replace && more ? 1 : 0);
        if (!launch_ok("block_gram_schmidt_batched (panel factor)")) return false;
        qtensor_gemm_desc t = {};                             // Y_p <- Y_p D^-1 U^-1 (one tile column: in place is safe)
        t.M = n; t.N = NB; t.K = NB; t.batch = batch;
        t.kind_a = QTENSOR_DENSE; t.kind_b = QTENSOR_DENSE; t.epilogue = QTENSOR_EPI_STORE;
        t.args.A = strided(panel_ptr, mat()); t.args.lda = n;
        t.args.B = strided(x, small); t.args.ldb = NB;
        t.args.C = strided(panel_ptr, mat()); t.args.ldc = n;
        t.args.triangular = 2;
        return run(t, stream);
    }
};

}  // namespace
}  // namespace qt

extern "C" int qtensor_hip_block_gram_schmidt_width(void) {
    // QT_BGS_PANEL (a tuning knob, only in builds made with -DQT_TUNING_KNOBS): another width of the outer panels,
    // a multiple of 64
    static const int width = [] {
#ifdef QT_TUNING_KNOBS
        const char *env = getenv("QT_BGS_PANEL");
#else
        const char *env = nullptr;
#endif
        const int asked = env != nullptr ? atoi(env) : 0;
        return asked >= qt::NB && asked % qt::NB == 0 && asked <= 1024 ? asked : 128;
    }();
    return width;
}

extern "C" void qtensor_hip_block_gram_schmidt_batched(float *q, float *w, float *gram, float *u, float *x, const float *fill,
                                                       int *info, int n, int batch, float pivot_floor, float null_norm2,
                                                       void *stream_v) {
    qtensor_hip_block_gram_schmidt_replacing_batched(q, w, gram, u, x, fill, info, n, batch, pivot_floor, null_norm2, 0, stream_v);
}

extern "C" void qtensor_hip_block_gram_schmidt_replacing_batched(float *q, float *w, float *gram, float *u, float *x,
                                                                 const float *fill, int *info, int n, int batch, float pivot_floor,
                                                                 float null_norm2, int replace_dependent, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("block_gram_schmidt_batched", n, batch, {q, w, gram, u, x, info})) return;
    if (!(pivot_floor >= 0.0f) || !(null_norm2 >= 0.0f)) { set_error(kBadArgument, "block_gram_schmidt_batched: negative threshold"); return; }
    if (replace_dependent != 0 && (fill == nullptr || !(pivot_floor > 0.0f))) {
        set_error(kBadArgument, "block_gram_schmidt_batched: replacing dependent columns needs fill columns and a pivot floor");
        return;
    }
    const int outer = qtensor_hip_block_gram_schmidt_width();
    Sweep s = {q, w, gram, u, x, fill, info, n, batch, outer, pivot_floor, null_norm2, (hipStream_t)stream_v, replace_dependent != 0};
    // Two levels.  An outer panel of `outer` columns has the finished columns taken out of it as a whole (the
    // bulk of the arithmetic, as products with a wide right-hand side) and is then swept inside -- every
    // 64-column panel: take the earlier panels of the same outer panel out, unit columns, one Cholesky QR
    // round -- and all of that is done twice.  The second pass acts on a panel that is orthonormal up to what
    // the rounding of the first one left, so nothing amplifies its own rounding: the panel ends orthonormal,
    // and orthogonal to the earlier columns, to fp32 rounding whatever the conditioning of the matrix (block
    // classical Gram-Schmidt with reorthogonalisation; the Cholesky QR inside a 64-column panel sees at most
    // that panel's own conditioning, and its pivot floor takes care of columns that depend on each other).
    // replace_dependent: three passes instead of two.  A column that the first or the second pass finds dependent on
    // the columns before it inside its 64-column panel (pivot at or below the floor) is not handed to the next pass as
    // it is -- where it is rounding noise it depends on them again -- but leaves the pass as a zero column and enters
    // the next one as a stand-in column from `fill`; so does a column that the second pass's projections shorten to
    // less than half.  Every stand-in column is orthogonalised against everything before it at least once after it
    // came in, every other column three times.
    const int passes = s.replace ? 3 : 2;
    for (int o0 = 0; o0 < n; o0 += outer) {
        const int width = n - o0 < outer ? n - o0 : outer;
        for (int pass = 0; pass < passes; ++pass) {
            if (pass >= 1 && fill != nullptr) {
                // what the pass before set aside comes back as stand-in columns, ahead of everything this pass does
                hipLaunchKernelGGL(fill_aside_kernel, dim3(kNormChunks, batch), dim3(256), 0, s.stream, q + o0, s.mat(), n, n, width / NB,
                                   outer / NB, s.aside_words(), fill + o0, n, info);
                if (!launch_ok("block_gram_schmidt_batched (stand-in columns)")) return;
            }
            if (!s.project(0, o0, width)) return;
            for (int c0 = o0; c0 < o0 + width; c0 += NB)
                if (!s.panel(o0, c0, pass, passes)) return;
        }
    }
}

extern "C" void qtensor_hip_solve_upper_right_batched(const float *q, const float *u, float *x, float *work, float *out,
                                                      int rows, int n, int batch, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("solve_upper_right_batched", n, batch, {q, u, x, work, out})) return;
    if (rows < 1) { set_error(kBadArgument, "solve_upper_right_batched: rows must be positive"); return; }
    hipStream_t stream = (hipStream_t)stream_v;
    const long long mat = (long long)n * n, tall = (long long)rows * n;
    // QT_SOLVE_PANEL (a tuning knob, only in builds made with -DQT_TUNING_KNOBS): another panel width, 64 times a
    // power of two
    static const int top = [] {
#ifdef QT_TUNING_KNOBS
        const char *env = getenv("QT_SOLVE_PANEL");
#else
        const char *env = nullptr;
#endif
        const int asked = env != nullptr ? atoi(env) : 0;
        const bool usable = asked >= NB && asked % NB == 0 && ((asked / NB) & (asked / NB - 1)) == 0;
        return usable ? asked : kSolvePanel;
    }();
    // x holds the inverses of the 64 x 64 diagonal blocks; every level doubles the size of the inverted blocks
    for (int s = NB; s < n && s < top; s *= 2) {
        const int full = n / (2 * s), rem = n % (2 * s);
        for (int part = 0; part < 2; ++part) {
            // part 0: the `full` pairs of two s-blocks of every matrix; part 1: a last pair whose second block is shorter
            if (part == 0 ? full == 0 : rem <= s) continue;
            const int c = part == 0 ? s : rem - s;
            const long long first = part == 0 ? 0 : (long long)full * 2 * s * (n + 1);     // corner of the (first) pair
            const int pairs = part == 0 ? full : 1;
            if ((long long)batch * pairs > 65535) { set_error(kBadArgument, "solve_upper_right_batched: too many blocks"); return; }
            const long long step = (long long)2 * s * (n + 1);
            // work_B = U_B X_C
            qtensor_gemm_desc w = {};
            w.M = s; w.N = c; w.K = c; w.batch = batch * pairs;
            w.kind_a = QTENSOR_DENSE; w.kind_b = QTENSOR_DENSE; w.epilogue = QTENSOR_EPI_STORE;
            w.args.A = strided(u + first + s, mat); w.args.lda = n;
            w.args.B = strided(x + first + (long long)s * (n + 1), mat); w.args.ldb = n;
            w.args.C = strided(work + first + s, mat); w.args.ldc = n;
            w.args.batch_inner = pairs;
            w.args.inner_a = w.args.inner_b = w.args.inner_c = step;
            w.args.triangular = 2;
            if (!run(w, stream)) return;
            // X_B = -X_A work_B
            qtensor_gemm_desc v = {};
            v.M = s; v.N = c; v.K = s; v.batch = batch * pairs;
            v.kind_a = QTENSOR_DENSE; v.kind_b = QTENSOR_DENSE; v.epilogue = QTENSOR_EPI_AXPBY_DENSE;
            v.args.A = strided(x + first, mat); v.args.lda = n;
            v.args.B = strided(work + first + s, mat); v.args.ldb = n;
            v.args.C = strided(x + first + s, mat); v.args.ldc = n;
            v.args.E = strided(work + first + s, mat); v.args.lde = n;       // finite values; beta = 0
            v.args.alpha = -1.0f; v.args.beta = 0.0f;
            v.args.batch_inner = pairs;
            v.args.inner_a = v.args.inner_b = v.args.inner_c = v.args.inner_e = step;
            v.args.triangular = 1;
            if (!run(v, stream)) return;
        }
    }
    // block back-substitution over column panels whose diagonal blocks of x are now inverted:
    //   out_j = (q_j - out_<j U_<j,j) X_jj
    const int width = top < n ? top : n;
    for (int j0 = 0; j0 < n; j0 += width) {
        const int w = n - j0 < width ? n - j0 : width;
        const float *rhs = q + j0;
        long long rhs_stride = tall;
        int rhs_ld = n;
        if (j0 > 0) {
            qtensor_gemm_desc d = {};
            d.M = rows; d.N = w; d.K = j0; d.batch = batch;
            d.kind_a = QTENSOR_DENSE; d.kind_b = QTENSOR_DENSE; d.epilogue = QTENSOR_EPI_AXPBY_DENSE;
            d.args.A = strided(out, tall); d.args.lda = n;
            d.args.B = strided(u + j0, mat); d.args.ldb = n;
            d.args.E = strided(q + j0, tall); d.args.lde = n;
            d.args.C = strided(work, (long long)rows * width); d.args.ldc = width;
            d.args.alpha = -1.0f; d.args.beta = 1.0f;
            if (!run(d, stream)) return;
            rhs = work; rhs_stride = (long long)rows * width; rhs_ld = width;
        }
        qtensor_gemm_desc t = {};
        t.M = rows; t.N = w; t.K = w; t.batch = batch;
        t.kind_a = QTENSOR_DENSE; t.kind_b = QTENSOR_DENSE; t.epilogue = QTENSOR_EPI_STORE;
        t.args.A = strided(rhs, rhs_stride); t.args.lda = rhs_ld;
        t.args.B = strided(x + (long long)j0 * (n + 1), mat); t.args.ldb = n;
        t.args.C = strided(out + j0, tall); t.args.ldc = n;
        t.args.triangular = 2;
        if (!run(t, stream)) return;
    }
}

extern "C" void qtensor_hip_gram_deviation_batched(const float *gram, float *partial, float *out, int n, int batch, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("gram_deviation_batched", n, batch, {gram, partial, out})) return;
    hipStream_t stream = (hipStream_t)stream_v;
    const int bands = n / 16 < kBands ? n / 16 : kBands;         // at least 16 rows per band
    const int rows_per_band = (n + bands - 1) / bands;
    hipLaunchKernelGGL(deviation_bands_kernel, dim3(bands, batch), dim3(256), 0, stream, gram, n, rows_per_band, partial);
    if (!launch_ok("gram_deviation_batched (bands)")) return;
    hipLaunchKernelGGL(deviation_total_kernel, dim3((batch + 63) / 64), dim3(64), 0, stream, partial, bands, batch, out);
    launch_ok("gram_deviation_batched (totals)");
}

extern "C" void qtensor_hip_column_dots_batched(const float *a, const float *b, float *out, int n, int batch, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("column_dots_batched", n, batch, {a, b, out})) return;
    hipLaunchKernelGGL(column_dots_kernel, dim3(n / 64, batch), dim3(256), 0, (hipStream_t)stream_v, a, b, out, n);
    launch_ok("column_dots_batched");
}

extern "C" void qtensor_hip_copy_flagged_batched(float *dst, const float *src, const int *flags, int n, int batch, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!stack_args_ok("copy_flagged_batched", n, batch, {dst, src, flags})) return;
    const long long quads = (long long)n * n / 4;
    hipLaunchKernelGGL(copy_flagged_kernel, dim3(64, batch), dim3(256), 0, (hipStream_t)stream_v, dst, src, flags, quads);
    launch_ok("copy_flagged_batched");
}
