// The elementwise end of a Shampoo optimizer step for all parameters in two launches:
//   1. per tensor, |grad|^2 and |direction|^2 (deterministic two-level sums);
//   2. direction *= |grad| / (|direction| + 1e-12)   (layer-wise grafting, optimizers/shampoo1.py:421
//      and shampoo2.py:453 of the reference), followed by the AdamW update (shampoo1.py:405-427,
//      shampoo2.py:446-468) or the SGD-with-momentum update (shampoo1.py:310-331, shampoo2.py:346-367).
// The reference does this with a dozen small torch kernels per parameter.
//
// Work is cut into chunks of kChunk consecutive elements of one tensor, one workgroup each;
// the table of tensors and the chunk -> tensor map live in device memory and are written by
// the caller once (they only change when a buffer moves).
#include "qt_common.h"

namespace qt {

struct TailTensor {            // one row of the device table: 8 x 64 bit
    float *param;
    const float *dir;          // preconditioned gradient (or the gradient itself)
    const float *grad;         // only read when the row is grafted
    float *m;                  // AdamW: exp_avg, SGD: momentum buffer
    float *v;                  // AdamW: exp_avg_sq, SGD: unused
    long long n;               // elements
    long long first_chunk;     // index of this tensor's first chunk
    long long flags;           // bit 0: rescale dir to the norm of grad
};

namespace {

constexpr int kChunk = 16384;  // elements per workgroup: sixteen float4 per thread
constexpr int kThreads = 256;

#define QT_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ float4 g4(const float *p) {
    const qt_f32x4 v = *(const QT_GLOBAL qt_f32x4 *)p;
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void s4(float *p, float4 y) {
    qt_f32x4 v;
    v.x = y.x; v.y = y.y; v.z = y.z; v.w = y.w;
    *(QT_GLOBAL qt_f32x4 *)p = v;
}
__device__ __forceinline__ float g1(const float *p) { return *(const QT_GLOBAL float *)p; }
__device__ __forceinline__ void s1(float *p, float y) { *(QT_GLOBAL float *)p = y; }

__device__ __forceinline__ float block_sum(float x, float *s_part) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) s_part[wave] = x;
    __syncthreads();
    const float total = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    __syncthreads();
    return total;
}

// partial[2c] = sum grad^2, partial[2c+1] = sum dir^2 over chunk c (rows without graft: untouched)
__global__ __launch_bounds__(kThreads) void tail_norms_kernel(const TailTensor *table, const int *chunk_tensor,
                                                              float *partial) {
    __shared__ float s_part[4];
    const int c = blockIdx.x;
    const TailTensor t = table[chunk_tensor[c]];
    if (!(t.flags & 1)) return;
    const long long start = ((long long)c - t.first_chunk) * kChunk;
    const long long left = t.n - start;
    const int len = left < kChunk ? (int)left : kChunk;
    const float *g = t.grad + start, *d = t.dir + start;
    float sg = 0.f, sd = 0.f;
    if (is_aligned16(g) && is_aligned16(d)) {
        for (int i = threadIdx.x * 4; i < len; i += kThreads * 4) {
            if (i + 3 < len) {
                const float4 a = g4(g + i), b = g4(d + i);
                sg += (a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w);
                sd += (b.x * b.x + b.y * b.y) + (b.z * b.z + b.w * b.w);
            } else {
                for (int e = i; e < len; ++e) { const float a = g1(g + e), b = g1(d + e); sg += a * a; sd += b * b; }
            }
        }
    } else {
        for (int i = threadIdx.x; i < len; i += kThreads) { const float a = g1(g + i), b = g1(d + i); sg += a * a; sd += b * b; }
    }
    sg = block_sum(sg, s_part);
    sd = block_sum(sd, s_part);
    if (threadIdx.x == 0) { s1(partial + 2 * c, sg); s1(partial + 2 * c + 1, sd); }
}

// |grad| / (|dir| + 1e-12) of the tensor that owns this chunk, summed in chunk order (the same
// value in every workgroup of the tensor)
__device__ __forceinline__ float graft_scale(const TailTensor &t, const float *partial, float *s_scale) {
    if (!(t.flags & 1)) return 1.0f;
    if (threadIdx.x == 0) {
        const long long chunks = (t.n + kChunk - 1) / kChunk;
        double sg = 0.0, sd = 0.0;
        for (long long c = t.first_chunk; c < t.first_chunk + chunks; ++c) {
            sg += (double)g1(partial + 2 * c);
            sd += (double)g1(partial + 2 * c + 1);
        }
        const float gn = (float)sqrt(sg), dn = (float)sqrt(sd);
        *s_scale = gn / (dn + 1e-12f);
    }
    __syncthreads();
    return *s_scale;
}

struct AdamW {
    float decay, beta1, alpha1, beta2, alpha2, sqrt_c2, eps, neg_step;
    const float *row_corrections;      // optional: {sqrt(1 - beta2^t), -lr / (1 - beta1^t)} per table row (its own step count t)
    __device__ __forceinline__ void bind(int row) {
        if (row_corrections != nullptr) { sqrt_c2 = g1(row_corrections + 2 * row); neg_step = g1(row_corrections + 2 * row + 1); }
    }
    __device__ __forceinline__ void operator()(float &p, float &m, float &v, float d) const {
        p = p * decay;
        m = m * beta1 + alpha1 * d;
        v = v * beta2 + (alpha2 * d) * d;
        const float denom = sqrtf(v) / sqrt_c2 + eps;
        p = p + neg_step * (m / denom);
    }
};

struct Sgd {
    float momentum, weight_decay, neg_lr;
    int nesterov;
    __device__ __forceinline__ void bind(int) {}
    __device__ __forceinline__ void operator()(float &p, float &m, float &v, float d) const {
        (void)v;
        if (weight_decay != 0.0f) d = d + weight_decay * p;
        m = m * momentum + d;
        const float u = nesterov ? d + momentum * m : m;
        p = p + neg_lr * u;
    }
};

template <typename RULE, bool HAS_V>
__global__ __launch_bounds__(kThreads) void tail_update_kernel(const TailTensor *table, const int *chunk_tensor,
                                                               const float *partial, const RULE launch_rule) {
    __shared__ float s_scale;
    const int c = blockIdx.x;
    const TailTensor t = table[chunk_tensor[c]];
    RULE rule = launch_rule;
    rule.bind(chunk_tensor[c]);
    const float scale = graft_scale(t, partial, &s_scale);
    const bool graft = (t.flags & 1) != 0;
    const long long start = ((long long)c - t.first_chunk) * kChunk;
    const long long left = t.n - start;
    const int len = left < kChunk ? (int)left : kChunk;
    float *p = t.param + start, *m = t.m + start, *v = HAS_V ? t.v + start : nullptr;
    const float *d = t.dir + start;
    const bool vec = is_aligned16(p) && is_aligned16(m) && is_aligned16(d) && (!HAS_V || is_aligned16(v));
    if (vec) {
        for (int i = threadIdx.x * 4; i < len; i += kThreads * 4) {
            if (i + 3 < len) {
                float4 P = g4(p + i), M = g4(m + i), D = g4(d + i), V = HAS_V ? g4(v + i) : make_float4(0.f, 0.f, 0.f, 0.f);
                if (graft) { D.x *= scale; D.y *= scale; D.z *= scale; D.w *= scale; }
                rule(P.x, M.x, V.x, D.x);
                rule(P.y, M.y, V.y, D.y);
                rule(P.z, M.z, V.z, D.z);
                rule(P.w, M.w, V.w, D.w);
                s4(p + i, P);
                s4(m + i, M);
                if (HAS_V) s4(v + i, V);
            } else {
                for (int e = i; e < len; ++e) {
                    float P = g1(p + e), M = g1(m + e), V = HAS_V ? g1(v + e) : 0.f, D = g1(d + e);
                    if (graft) D *= scale;
                    rule(P, M, V, D);
                    s1(p + e, P); s1(m + e, M);
                    if (HAS_V) s1(v + e, V);
                }
            }
        }
    } else {
        for (int e = threadIdx.x; e < len; e += kThreads) {
            float P = g1(p + e), M = g1(m + e), V = HAS_V ? g1(v + e) : 0.f, D = g1(d + e);
            if (graft) D *= scale;
            rule(P, M, V, D);
            s1(p + e, P); s1(m + e, M);
            if (HAS_V) s1(v + e, V);
        }
    }
}

bool tail_args_ok(const void *table, const void *chunk_tensor, int n_chunks, const void *partial, int graft, const char *what) {
    if (!table || !chunk_tensor || (graft && !partial)) { set_error(kNullPointer, "%s: null table, chunk map or partial-sum buffer", what); return false; }
    if (n_chunks < 0) { set_error(kBadArgument, "%s: negative chunk count", what); return false; }
    return true;
}

}  // namespace
}  // namespace qt

extern "C" int qtensor_hip_tail_chunk(void) { return qt::kChunk; }

namespace qt {
namespace {
void adamw_tail(const void *table, const int *chunk_tensor, int n_chunks, float *partial, int graft, double lr, double beta1,
                double beta2, double eps, double weight_decay, long long step, const float *row_corrections, void *stream) {
    clear_error();
    if (!tail_args_ok(table, chunk_tensor, n_chunks, partial, graft, "adamw_tail")) return;
    if (row_corrections == nullptr && step < 1) { set_error(kBadArgument, "adamw_tail: step counts from 1"); return; }
    if (n_chunks == 0) return;
    const TailTensor *tab = static_cast<const TailTensor *>(table);
    if (graft) {
        hipLaunchKernelGGL(tail_norms_kernel, dim3(n_chunks), dim3(kThreads), 0, (hipStream_t)stream, tab, chunk_tensor, partial);
        if (!launch_ok("adamw_tail (norms)")) return;
    }
    AdamW rule;
    rule.decay = (float)(1.0 - lr * weight_decay);
    rule.beta1 = (float)beta1;
    rule.alpha1 = (float)(1.0 - beta1);
    rule.beta2 = (float)beta2;
    rule.alpha2 = (float)(1.0 - beta2);
    rule.sqrt_c2 = row_corrections != nullptr ? 1.0f : (float)sqrt(1.0 - pow(beta2, (double)step));
    rule.eps = (float)eps;
    rule.neg_step = row_corrections != nullptr ? 0.0f : (float)(-lr / (1.0 - pow(beta1, (double)step)));
    rule.row_corrections = row_corrections;
    hipLaunchKernelGGL((tail_update_kernel<AdamW, true>), dim3(n_chunks), dim3(kThreads), 0, (hipStream_t)stream, tab,
                       chunk_tensor, partial, rule);
    launch_ok("adamw_tail");
}
}  // namespace
}  // namespace qt

extern "C" void qtensor_hip_adamw_tail(const void *table, const int *chunk_tensor, int n_chunks, float *partial, int graft,
                                       double lr, double beta1, double beta2, double eps, double weight_decay,
                                       long long step, void *stream) {
    qt::adamw_tail(table, chunk_tensor, n_chunks, partial, graft, lr, beta1, beta2, eps, weight_decay, step, nullptr, stream);
}

extern "C" void qtensor_hip_adamw_tail_rows(const void *table, const int *chunk_tensor, int n_chunks, float *partial, int graft,
                                            double lr, double beta1, double beta2, double eps, double weight_decay,
                                            const float *row_corrections, void *stream) {
    if (row_corrections == nullptr) {
        qt::clear_error();
        qt::set_error(qt::kNullPointer, "adamw_tail_rows: null row_corrections");
        return;
    }
    qt::adamw_tail(table, chunk_tensor, n_chunks, partial, graft, lr, beta1, beta2, eps, weight_decay, 0, row_corrections, stream);
}

extern "C" void qtensor_hip_sgd_tail(const void *table, const int *chunk_tensor, int n_chunks, float *partial, int graft,
                                     double lr, double momentum, double weight_decay, int nesterov, void *stream) {
    using namespace qt;
    clear_error();
    if (!tail_args_ok(table, chunk_tensor, n_chunks, partial, graft, "sgd_tail")) return;
    if (n_chunks == 0) return;
    const TailTensor *tab = static_cast<const TailTensor *>(table);
    if (graft) {
        hipLaunchKernelGGL(tail_norms_kernel, dim3(n_chunks), dim3(kThreads), 0, (hipStream_t)stream, tab, chunk_tensor, partial);
        if (!launch_ok("sgd_tail (norms)")) return;
    }
    Sgd rule;
    rule.momentum = (float)momentum;
    rule.weight_decay = (float)weight_decay;
    rule.neg_lr = (float)(-lr);
    rule.nesterov = nesterov != 0;
    hipLaunchKernelGGL((tail_update_kernel<Sgd, false>), dim3(n_chunks), dim3(kThreads), 0, (hipStream_t)stream, tab,
                       chunk_tensor, partial, rule);
    launch_ok("sgd_tail");
}
