// Blockwise dequantize kernels for gfx950 and their launchers.
//
// out[r,c] = fl32(code[idx] * absmax[segment]) -- except +0.0 for a zero-maximum segment --
// then rounded to the output type; the diagreal form overwrites the diagonal with diag[]
// (qtensor/functional.py:618-688 and :738-746 of the reference).
//
// flat path (blocksize divides order): one lane turns 2 bytes (4-bit) or 4 bytes (8-bit) of
// codes into one 16-byte (fp32) or 8-byte (bf16) store, so the store stream -- eight ninths of
// the traffic -- is perfectly coalesced.  general path: one thread per code byte.
#include "qt_common.h"

namespace qt {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

template <typename T> struct Vec4Store;
template <> struct Vec4Store<float> {
    static __device__ __forceinline__ void store(float *base, uint32_t k, float4 y) {
        *reinterpret_cast<float4 *>(base + k) = y;
    }
    static __device__ __forceinline__ void store1(float *base, size_t k, float y) { base[k] = y; }
};
template <> struct Vec4Store<uint16_t> {
    static __device__ __forceinline__ void store(uint16_t *base, uint32_t k, float4 y) {
        uint2 w;
        w.x = (uint32_t)float_to_bf16_bits(y.x) | ((uint32_t)float_to_bf16_bits(y.y) << 16);
        w.y = (uint32_t)float_to_bf16_bits(y.z) | ((uint32_t)float_to_bf16_bits(y.w) << 16);
        *reinterpret_cast<uint2 *>(base + k) = w;
    }
    static __device__ __forceinline__ void store1(uint16_t *base, size_t k, float y) { base[k] = float_to_bf16_bits(y); }
};

template <typename T, int BITS, bool DIAG>
__global__ __launch_bounds__(kThreads) void dequantize_flat_kernel(
    const uint8_t *__restrict__ q, const float *__restrict__ code, uint32_t n_vec, uint32_t bs_shift,
    FastDiv row_div, const float *__restrict__ absmax, const float *__restrict__ diag, T *__restrict__ out) {
    constexpr int NCODE = 1 << BITS;
    __shared__ float s_code[NCODE];
    for (int i = threadIdx.x; i < NCODE; i += kThreads) s_code[i] = code[i];
    __syncthreads();

    const uint32_t stride = gridDim.x * kThreads;
    for (uint32_t base = blockIdx.x * kThreads + threadIdx.x; base < n_vec; base += stride * kUnroll) {
        uint32_t packed[kUnroll];
        float scale[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t i = base + (uint32_t)u * stride;
            if (i < n_vec) {
                packed[u] = BITS == 4 ? (uint32_t) reinterpret_cast<const uint16_t *>(q)[i]
                                      : reinterpret_cast<const uint32_t *>(q)[i];
                scale[u] = absmax[(i << 2) >> bs_shift];
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t i = base + (uint32_t)u * stride;
            if (i >= n_vec) break;
            uint32_t id0, id1, id2, id3;
            if (BITS == 4) {
                id0 = (packed[u] >> 4) & 15u; id1 = packed[u] & 15u;
                id2 = (packed[u] >> 12) & 15u; id3 = (packed[u] >> 8) & 15u;
            } else {
                id0 = packed[u] & 255u; id1 = (packed[u] >> 8) & 255u;
                id2 = (packed[u] >> 16) & 255u; id3 = packed[u] >> 24;
            }
            const float a = scale[u];
            float4 y;
            if (a == 0.0f) {
                y = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            } else {
                y = make_float4(s_code[id0] * a, s_code[id1] * a, s_code[id2] * a, s_code[id3] * a);
            }
            if (DIAG) {
                const uint32_t row = fastdiv(i, row_div);
                const uint32_t col4 = i - row * row_div.divisor;
                if ((row >> 2) == col4) {
                    const float d = diag[row];
                    const uint32_t e = row & 3u;
                    if (e == 0) y.x = d; else if (e == 1) y.y = d; else if (e == 2) y.z = d; else y.w = d;
                }
            }
            Vec4Store<T>::store(out, i << 2, y);
        }
    }
}

template <typename T, int BITS, bool DIAG>
__global__ __launch_bounds__(kThreads) void dequantize_general_kernel(
    const uint8_t *__restrict__ q, const float *__restrict__ code, uint32_t order, uint32_t bs, uint32_t nb,
    uint32_t total, const float *__restrict__ absmax, const float *__restrict__ diag, T *__restrict__ out) {
    constexpr int NCODE = 1 << BITS;
    constexpr uint32_t EPB = 8 / BITS;
    __shared__ float s_code[NCODE];
    for (int i = threadIdx.x; i < NCODE; i += kThreads) s_code[i] = code[i];
    __syncthreads();
    const uint32_t n_bytes = (total + EPB - 1) / EPB;
    for (uint32_t j = blockIdx.x * kThreads + threadIdx.x; j < n_bytes; j += gridDim.x * kThreads) {
        const uint32_t byte = q[j];
#pragma unroll
        for (uint32_t e = 0; e < EPB; ++e) {
            const uint32_t k = j * EPB + e;
            if (k >= total) break;
            const uint32_t id = BITS == 8 ? byte : (e == 0 ? byte >> 4 : byte & 15u);
            const uint32_t r = k / order, c = k - r * order;
            const float a = absmax[r * nb + c / bs];
            float y = a == 0.0f ? 0.0f : s_code[id] * a;
            if (DIAG && r == c) y = diag[r];
            Vec4Store<T>::store1(out, k, y);
        }
    }
}

int capped_grid(uint32_t blocks_needed, int blocks_per_cu) {
    const uint32_t cap = (uint32_t)(compute_units() * blocks_per_cu);
    return (int)(blocks_needed < 1 ? 1 : (blocks_needed < cap ? blocks_needed : cap));
}

template <typename T, int BITS, bool DIAG>
void dequantize_dispatch(const uint8_t *q, const float *code, int order_i, const float *absmax, const float *diag,
                         T *out, int blocksize, hipStream_t stream) {
    clear_error();
    int bs_shift = 0;
    switch (blocksize) {
        case 64: bs_shift = 6; break;
        case 128: bs_shift = 7; break;
        case 256: bs_shift = 8; break;
        case 512: bs_shift = 9; break;
        case 1024: bs_shift = 10; break;
        case 2048: bs_shift = 11; break;
        default:
            set_error(kBadBlocksize, "dequantize_blockwise: blocksize %d is not one of 64,128,256,512,1024,2048", blocksize);
            return;
    }
    if (order_i < 1 || (int64_t)order_i * order_i >= (int64_t(1) << 31)) {
        set_error(kBadOrder, "dequantize_blockwise: order %d out of range (need 1 <= order and order*order < 2^31)", order_i);
        return;
    }
    if (!q || !code || !absmax || !out || (DIAG && !diag)) {
        set_error(kNullPointer, "dequantize_blockwise: null device pointer");
        return;
    }
    const uint32_t order = (uint32_t)order_i, bs = (uint32_t)blocksize;
    const uint32_t total = order * order;
    const bool flat = order % bs == 0 && is_aligned(out, 4 * sizeof(T)) && is_aligned(q, BITS == 4 ? 2 : 4) && is_aligned(absmax, 4);
    if (flat) {
        const uint32_t n_vec = total / 4;
        const uint32_t blocks = (n_vec + kThreads * kUnroll - 1) / (kThreads * kUnroll);
        hipLaunchKernelGGL((dequantize_flat_kernel<T, BITS, DIAG>), dim3(capped_grid(blocks, 16)), dim3(kThreads), 0, stream,
                           q, code, n_vec, (uint32_t)bs_shift, make_fastdiv(order / 4), absmax, diag, out);
    } else {
        const uint32_t nb = (order + bs - 1) / bs;
        const uint32_t n_bytes = (total * BITS + 7) / 8;
        hipLaunchKernelGGL((dequantize_general_kernel<T, BITS, DIAG>), dim3(capped_grid((n_bytes + kThreads - 1) / kThreads, 16)),
                           dim3(kThreads), 0, stream, q, code, order, bs, nb, total, absmax, diag, out);
    }
    launch_ok("dequantize_blockwise");
}

}  // namespace
}  // namespace qt

#define QT_DEFINE_DEQUANT(NAME, T, BITS)                                                                                  \
    extern "C" void cdequantize_blockwise_##NAME##_stream(unsigned char *A, float *code, int order, float *absmax,       \
                                                          T *out, int blocksize, void *stream) {                         \
        qt::dequantize_dispatch<T, BITS, false>(A, code, order, absmax, nullptr, out, blocksize, (hipStream_t)stream);   \
    }                                                                                                                    \
    extern "C" void cdequantize_blockwise_##NAME(unsigned char *A, float *code, int order, float *absmax, T *out,        \
                                                 int blocksize) {                                                        \
        qt::dequantize_dispatch<T, BITS, false>(A, code, order, absmax, nullptr, out, blocksize, nullptr);               \
    }                                                                                                                    \
    extern "C" void cdequantize_blockwise_diagreal_##NAME##_stream(unsigned char *A, float *code, int order,             \
                                                                   float *absmax, float *diag, T *out, int blocksize,    \
                                                                   void *stream) {                                       \
        qt::dequantize_dispatch<T, BITS, true>(A, code, order, absmax, diag, out, blocksize, (hipStream_t)stream);       \
    }                                                                                                                    \
    extern "C" void cdequantize_blockwise_diagreal_##NAME(unsigned char *A, float *code, int order, float *absmax,       \
                                                          float *diag, T *out, int blocksize) {                          \
        qt::dequantize_dispatch<T, BITS, true>(A, code, order, absmax, diag, out, blocksize, nullptr);                   \
    }

QT_DEFINE_DEQUANT(8bit_fp32, float, 8)
QT_DEFINE_DEQUANT(8bit_bf16, uint16_t, 8)
QT_DEFINE_DEQUANT(4bit_fp32, float, 4)
QT_DEFINE_DEQUANT(4bit_bf16, uint16_t, 4)
