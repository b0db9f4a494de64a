// Blockwise dequantize kernels for gfx950 and their launchers.
//
// out[r,c] = fl32(code[idx] * absmax[segment]) -- except +0.0 for a zero-maximum segment --
// then rounded to the output type; the diagreal form overwrites the diagonal with diag[]
// (qtensor/functional.py:618-688 and :738-746 of the reference).
//
// flat path (blocksize divides order): codes are fetched 16 bytes per lane, turned around in
// LDS, and written out as fully coalesced 16-byte (fp32) or 8-byte (bf16) stores per lane -- the
// store stream is eight ninths of the traffic.  general path: one thread per code byte.
#include "qt_common.h"

namespace qt {
namespace {

#ifndef QT_D_THREADS
#define QT_D_THREADS 128
#endif
#ifndef QT_D_BLOCKS_PER_CU
#define QT_D_BLOCKS_PER_CU 3
#endif
#ifndef QT_D_CHUNKED
#define QT_D_CHUNKED 0
#endif
constexpr int kThreads = 256;             // general-path kernel
constexpr int kFlatThreads = QT_D_THREADS;
constexpr int kFlatBlocksPerCU = QT_D_BLOCKS_PER_CU;
constexpr int kSuper = 2048;              // elements a wave turns around per step

template <typename T> struct Vec4Store;
template <> struct Vec4Store<float> {
    template <bool STREAM>
    static __device__ __forceinline__ void store(float *base, uint32_t k, float4 y) {
        store_f32x4<STREAM>(base + k, y);
    }
    static __device__ __forceinline__ void store1(float *base, size_t k, float y) { base[k] = y; }
};
template <> struct Vec4Store<uint16_t> {
    template <bool STREAM>
    static __device__ __forceinline__ void store(uint16_t *base, uint32_t k, float4 y) {
        uint2 w;
        w.x = (uint32_t)float_to_bf16_bits(y.x) | ((uint32_t)float_to_bf16_bits(y.y) << 16);
        w.y = (uint32_t)float_to_bf16_bits(y.z) | ((uint32_t)float_to_bf16_bits(y.w) << 16);
        store_u32x2<STREAM>(base + k, w);
    }
    static __device__ __forceinline__ void store1(uint16_t *base, size_t k, float y) { base[k] = float_to_bf16_bits(y); }
};

// Flat path.  Per step a wave takes 2048 consecutive elements: their packed codes arrive with
// one 16-byte (4-bit) or two 16-byte (8-bit) loads per lane and the segment maxima with one
// 4-byte load on the first lanes; both are parked in the wave's private LDS area and read back
// in the order that makes every one of the 8 output stores a fully coalesced 1 KiB (fp32) run.
// The loads of the next step are issued before the stores of the current one.  Big outputs are written
// with the streaming hint, but the codes are always read with plain loads: on an MI355X the hint on this
// thin read stream beside the wide write stream costs a tenth of the bandwidth (0.224 -> 0.199 ms for the
// 16384^2 tensor), and six waves per compute unit in workgroups of two do better than twelve in
// workgroups of four (0.199 -> 0.185 ms).
template <typename T, int BITS, bool DIAG, bool STREAM>
__global__ __launch_bounds__(kFlatThreads) void dequantize_flat_kernel(
    const uint8_t *__restrict__ q, const float *__restrict__ code, uint32_t n_super, uint32_t bs_shift,
    FastDiv row_div, FastDiv order_div, const float *__restrict__ absmax, const float *__restrict__ diag, T *__restrict__ out) {
    constexpr int NCODE = 1 << BITS;
    constexpr int kWaves = kFlatThreads / 64;
    constexpr int CODE_VECS = BITS == 4 ? 1 : 2;            // uint4 loads per lane per step
    __shared__ float s_code[NCODE];
    __shared__ uint4 s_stage[kWaves][CODE_VECS * 64];
    __shared__ float s_scale[kWaves][32];
    for (int i = threadIdx.x; i < NCODE; i += kFlatThreads) s_code[i] = code[i];
    __syncthreads();

    const uint32_t lane = threadIdx.x & 63u, w = threadIdx.x >> 6;
    const uint32_t wave = blockIdx.x * kWaves + w;
    const uint32_t n_waves = gridDim.x * kWaves;
#if QT_D_CHUNKED
    const uint32_t per = (n_super + n_waves - 1) / n_waves;
    uint32_t st = wave * per;
    const uint32_t end = min(st + per, n_super);
    const uint32_t step = 1;
#else
    uint32_t st = wave;
    const uint32_t end = n_super;
    const uint32_t step = n_waves;
#endif
    if (st >= end) return;
    const uint32_t last = end - 1;
    const uint32_t seg_per_super = (uint32_t)kSuper >> bs_shift;   // 32 .. 1
    const uint4 *q16 = reinterpret_cast<const uint4 *>(q);

    uint4 c[CODE_VECS];
    float a = 0.0f;
    auto fetch = [&](uint32_t s) {
#pragma unroll
        for (int v = 0; v < CODE_VECS; ++v) c[v] = load_u32x4<false>(q16 + (size_t)s * (CODE_VECS * 64) + v * 64 + lane);
        if (lane < seg_per_super) a = absmax[s * seg_per_super + lane];
    };
    fetch(st);
    const uint16_t *stage16 = reinterpret_cast<const uint16_t *>(&s_stage[w][0]);
    const uint32_t *stage32 = reinterpret_cast<const uint32_t *>(&s_stage[w][0]);

    for (; st < end; st += step) {
#pragma unroll
        for (int v = 0; v < CODE_VECS; ++v) s_stage[w][v * 64 + lane] = c[v];
        if (lane < seg_per_super) s_scale[w][lane] = a;
        fetch(min(st + step, last));
        wave_lds_sync();

        const uint32_t k4_0 = st * (uint32_t)(kSuper / 4) + lane;   // index of this lane's first 4-vector
        uint32_t row = 0, col4 = 0, lrow = 0;                        // row of the stack, and inside its matrix
        if (DIAG) {
            row = fastdiv(k4_0, row_div);
            col4 = k4_0 - row * row_div.divisor;
            lrow = row - fastdiv(row, order_div) * order_div.divisor;
        }
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t v4 = j * 64u + lane;                 // 4-vector inside the step
            uint32_t id0, id1, id2, id3;
            if (BITS == 4) {
                const uint32_t p = stage16[v4];
                id0 = (p >> 4) & 15u; id1 = p & 15u; id2 = (p >> 12) & 15u; id3 = (p >> 8) & 15u;
            } else {
                const uint32_t p = stage32[v4];
                id0 = p & 255u; id1 = (p >> 8) & 255u; id2 = (p >> 16) & 255u; id3 = p >> 24;
            }
            const float scale = s_scale[w][(v4 << 2) >> bs_shift];
            float4 y;
            if (scale == 0.0f) {
                y = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            } else {
                y = make_float4(s_code[id0] * scale, s_code[id1] * scale, s_code[id2] * scale, s_code[id3] * scale);
            }
            if (DIAG) {
                if ((lrow >> 2) == col4) {
                    const float d = diag[row];
                    const uint32_t e = lrow & 3u;
                    if (e == 0) y.x = d; else if (e == 1) y.y = d; else if (e == 2) y.z = d; else y.w = d;
                }
                col4 += 64u;
                while (col4 >= row_div.divisor) {
                    col4 -= row_div.divisor;
                    ++row;
                    if (++lrow == order_div.divisor) lrow = 0;
                }
            }
            Vec4Store<T>::template store<STREAM>(out, (k4_0 + j * 64u) << 2, y);
        }
        wave_lds_sync();   // the staging area is rewritten at the top of the next step
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
    // blockIdx.y = matrix of a stack (its own run of code bytes, maxima and diagonal entries)
    q += (size_t)blockIdx.y * n_bytes;
    absmax += (size_t)blockIdx.y * order * nb;
    if (DIAG) diag += (size_t)blockIdx.y * order;
    out += (size_t)blockIdx.y * total;
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
                         T *out, int blocksize, hipStream_t stream, int batch = 1) {
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
    if (order_i < 1 || batch < 1 || (int64_t)order_i * order_i * batch >= (int64_t(1) << 31)) {
        set_error(kBadOrder, "dequantize_blockwise: order %d (batch %d) out of range (need order >= 1 and batch*order*order < 2^31)",
                  order_i, batch);
        return;
    }
    if (!q || !code || !absmax || !out || (DIAG && !diag)) {
        set_error(kNullPointer, "dequantize_blockwise: null device pointer");
        return;
    }
    const uint32_t order = (uint32_t)order_i, bs = (uint32_t)blocksize;
    const uint32_t total = order * order * (uint32_t)batch;
    const bool flat = order % bs == 0 && is_aligned(out, 4 * sizeof(T)) && is_aligned(q, 16) && is_aligned(absmax, 4);
    if (batch > 65535 && !flat) {
        set_error(kBadArgument, "dequantize_blockwise: a stack whose order the blocksize does not divide (or with unaligned buffers) "
                                "takes at most 65535 matrices per launch");
        return;
    }
    if (flat) {
        constexpr uint32_t kWaves = kFlatThreads / 64;
        const uint32_t n_super = total / kSuper;
        const uint32_t blocks = (n_super + kWaves - 1) / kWaves;
        const dim3 grid(capped_grid(blocks, kFlatBlocksPerCU));
        // Outputs far beyond the 256 MB last-level cache are written with the streaming hint.
        if (total >= (1u << 25)) {
            hipLaunchKernelGGL((dequantize_flat_kernel<T, BITS, DIAG, true>), grid, dim3(kFlatThreads), 0, stream,
                               q, code, n_super, (uint32_t)bs_shift, make_fastdiv(order / 4), make_fastdiv(order), absmax, diag, out);
        } else {
            hipLaunchKernelGGL((dequantize_flat_kernel<T, BITS, DIAG, false>), grid, dim3(kFlatThreads), 0, stream,
                               q, code, n_super, (uint32_t)bs_shift, make_fastdiv(order / 4), make_fastdiv(order), absmax, diag, out);
        }
    } else {
        const uint32_t nb = (order + bs - 1) / bs;
        const uint32_t one = order * order;
        const uint32_t n_bytes = (one * BITS + 7) / 8;
        hipLaunchKernelGGL((dequantize_general_kernel<T, BITS, DIAG>), dim3(capped_grid((n_bytes + kThreads - 1) / kThreads, 16), batch),
                           dim3(kThreads), 0, stream, q, code, order, bs, nb, one, absmax, diag, out);
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

extern "C" void qtensor_hip_dequantize_batched(const unsigned char *q, const float *code, int bits, int order, int batch,
                                               const float *absmax, const float *diag, void *out, int out_is_bf16,
                                               int blocksize, void *stream) {
    using namespace qt;
    hipStream_t st = (hipStream_t)stream;
    if (bits != 4 && bits != 8) { clear_error(); set_error(kBadArgument, "dequantize_batched: bits must be 4 or 8"); return; }
#define QT_DB(T, BITS)                                                                                           \
    (diag ? dequantize_dispatch<T, BITS, true>(q, code, order, absmax, diag, (T *)out, blocksize, st, batch)       \
          : dequantize_dispatch<T, BITS, false>(q, code, order, absmax, nullptr, (T *)out, blocksize, st, batch))
    if (out_is_bf16) { if (bits == 4) QT_DB(uint16_t, 4); else QT_DB(uint16_t, 8); }
    else { if (bits == 4) QT_DB(float, 4); else QT_DB(float, 8); }
#undef QT_DB
}
