// Blockwise quantize kernels for gfx950 (wave64) and their launchers.
//
// Two paths:
//  * flat path -- blocksize divides order.  The matrix is then a flat stream of whole segments
//    (segment s = elements [s*BS, (s+1)*BS), absmax index s).  Each lane owns one 16-byte vector
//    per 256-element slice, the segment maximum is a DPP butterfly over 16/32/64 lanes, the
//    quotient is a correctly rounded fp32 division (one exact reciprocal per segment, then the
//    multiply / residual-fma / correction-fma sequence), and the index is a threshold count
//    done either through a bucket table in LDS (large inputs) or a binary search in LDS.
//  * general path -- any order/blocksize (ragged last segment, odd order with nibble pairs that
//    straddle rows): one pass for the maxima (a wave per segment), one pass per output byte.
//
// Arithmetic follows qtensor/functional.py:526-615 and :703-735 of the reference.
#include "qt_common.h"
#include "qt_tables.h"

namespace qt {
namespace {

constexpr int kThreads = 256;

template <typename T> struct Vec4Loader;
template <> struct Vec4Loader<float> {
    static __device__ __forceinline__ float4 load(const float *base, uint32_t k) {
        return *reinterpret_cast<const float4 *>(base + k);
    }
    static __device__ __forceinline__ float load1(const float *base, size_t k) { return base[k]; }
};
template <> struct Vec4Loader<uint16_t> {
    static __device__ __forceinline__ float4 load(const uint16_t *base, uint32_t k) {
        const uint2 w = *reinterpret_cast<const uint2 *>(base + k);
        return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
                           __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u));
    }
    static __device__ __forceinline__ float load1(const uint16_t *base, size_t k) { return bf16_bits_to_float(base[k]); }
};

__device__ __forceinline__ uint32_t abs_bits(float x) { return __float_as_uint(x) & 0x7fffffffu; }

// Index by the exact route: IEEE division, then the threshold count.  amax_bits == 0 -> 0.
template <int NCODE>
__device__ __forceinline__ uint32_t exact_index(float x, uint32_t amax_bits, const CodeTables<NCODE> &t) {
    if (amax_bits == 0u) return 0u;
    const float q = x / __uint_as_float(amax_bits);
    return t.perm[count_thresholds<NCODE>(q, t.thr)];
}

// Correctly rounded x / a for a in [2^-60, 2^60] and |x/a| >= 2^-40 (or x == 0), given
// r = fl(1/a): q0 = fl(x*r) is within one ulp, the residual x - q0*a is exact in fp32, and one
// more fma lands on the correctly rounded quotient (Markstein's division theorem).
__device__ __forceinline__ float quotient(float x, float a, float r) {
    const float q0 = x * r;
    const float rem = __builtin_fmaf(-q0, a, x);
    return __builtin_fmaf(rem, r, q0);
}

template <int NCODE, bool USE_LUT>
__device__ __forceinline__ uint32_t fast_index(float x, float a, float r, const CodeTables<NCODE> &t, const uint2 *lut) {
    const float q = quotient(x, a, r);
    if (USE_LUT) {
        const uint2 e = lut[lut_bucket(q)];
        return e.y + (uint32_t)!(q < __uint_as_float(e.x));
    }
    return (uint32_t)count_thresholds<NCODE>(q, t.thr);
}

// One wave handles TILE = max(BS, 256) consecutive elements per iteration; VPT 16-byte
// vectors per lane.  Segment = G lanes when BS <= 256, the whole wave otherwise.
template <typename T, int BITS, int BS, bool DIAG, bool USE_LUT>
__global__ __launch_bounds__(kThreads) void quantize_flat_kernel(
    const T *__restrict__ A, const float *__restrict__ code, uint32_t n_tiles, FastDiv row_div,
    float *__restrict__ absmax, float *__restrict__ diag, uint8_t *__restrict__ out) {
    constexpr int NCODE = 1 << BITS;
    constexpr int TILE = BS > 256 ? BS : 256;
    constexpr int VPT = TILE / 256;
    constexpr int G = BS >= 256 ? 64 : BS / 4;

    __shared__ CodeTables<NCODE> tab;
    __shared__ uint2 lut_mem[USE_LUT ? kLutEntries : 1];
    uint2 *lut = USE_LUT ? lut_mem : nullptr;
    build_code_tables<NCODE>(code, tab, lut);
    const int flags = tab.flags;
    const bool fast_ok = (flags & kFlagLut) != 0;
    const bool ascending = (flags & kFlagAscending) != 0;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * (kThreads / 64);

    for (uint32_t tile = wave; tile < n_tiles; tile += n_waves) {
        const uint32_t k0 = tile * (uint32_t)TILE + lane * 4u;
        float4 v[VPT];
#pragma unroll
        for (int j = 0; j < VPT; ++j) v[j] = Vec4Loader<T>::load(A, k0 + (uint32_t)j * 256u);

        if (DIAG) {
#pragma unroll
            for (int j = 0; j < VPT; ++j) {
                const uint32_t k4 = (k0 + (uint32_t)j * 256u) >> 2;
                const uint32_t row = fastdiv(k4, row_div);
                const uint32_t col4 = k4 - row * row_div.divisor;
                if ((row >> 2) == col4) {
                    const uint32_t e = row & 3u;
                    const float d = e == 0 ? v[j].x : e == 1 ? v[j].y : e == 2 ? v[j].z : v[j].w;
                    diag[row] = d;
                    if (e == 0) v[j].x = 0.0f; else if (e == 1) v[j].y = 0.0f; else if (e == 2) v[j].z = 0.0f; else v[j].w = 0.0f;
                }
            }
        }

        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < VPT; ++j)
            m = max(max(m, max(abs_bits(v[j].x), abs_bits(v[j].y))), max(abs_bits(v[j].z), abs_bits(v[j].w)));
        m = group_max_u32<G>(m);
        if (m > 0x7f800000u) m = 0x7fc00000u;   // any NaN in the segment -> canonical NaN
        const float amax = __uint_as_float(m);
        if ((lane & (G - 1)) == 0) absmax[tile * (uint32_t)(TILE / BS) + lane / G] = amax;

        // 2^-60 <= amax <= 2^60, else (zero, huge, tiny, inf, NaN) take the exact route
        const bool special = !fast_ok || (m - 0x21800000u) > (0x5d800000u - 0x21800000u);
        uint32_t idx[VPT][4];
        if (__any(special)) {
#pragma unroll
            for (int j = 0; j < VPT; ++j) {
                idx[j][0] = exact_index<NCODE>(v[j].x, m, tab);
                idx[j][1] = exact_index<NCODE>(v[j].y, m, tab);
                idx[j][2] = exact_index<NCODE>(v[j].z, m, tab);
                idx[j][3] = exact_index<NCODE>(v[j].w, m, tab);
            }
        } else {
            const float r = 1.0f / amax;
#pragma unroll
            for (int j = 0; j < VPT; ++j) {
                idx[j][0] = fast_index<NCODE, USE_LUT>(v[j].x, amax, r, tab, lut);
                idx[j][1] = fast_index<NCODE, USE_LUT>(v[j].y, amax, r, tab, lut);
                idx[j][2] = fast_index<NCODE, USE_LUT>(v[j].z, amax, r, tab, lut);
                idx[j][3] = fast_index<NCODE, USE_LUT>(v[j].w, amax, r, tab, lut);
            }
            if (!ascending) {
#pragma unroll
                for (int j = 0; j < VPT; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) idx[j][e] = tab.perm[idx[j][e]];
            }
        }

#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            const uint32_t k = k0 + (uint32_t)j * 256u;
            if (BITS == 4) {
                const uint32_t h = ((idx[j][0] << 4) | idx[j][1]) | (((idx[j][2] << 4) | idx[j][3]) << 8);
                *reinterpret_cast<uint16_t *>(out + (k >> 1)) = (uint16_t)h;
            } else {
                const uint32_t w = idx[j][0] | (idx[j][1] << 8) | (idx[j][2] << 16) | (idx[j][3] << 24);
                *reinterpret_cast<uint32_t *>(out + k) = w;
            }
        }
    }
}

// ---- general path ----------------------------------------------------------------------
// One wave per segment; writes absmax (and diag).
template <typename T, bool DIAG>
__global__ __launch_bounds__(kThreads) void segment_max_kernel(
    const T *__restrict__ A, uint32_t order, uint32_t bs, uint32_t nb, uint32_t n_segments,
    float *__restrict__ absmax, float *__restrict__ diag) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * (kThreads / 64);
    for (uint32_t seg = wave; seg < n_segments; seg += n_waves) {
        const uint32_t r = seg / nb, b = seg - r * nb;
        const uint32_t c0 = b * bs, c1 = min(c0 + bs, order);
        const size_t row0 = (size_t)r * order;
        uint32_t m = 0;
        for (uint32_t c = c0 + lane; c < c1; c += 64u) {
            float x = Vec4Loader<T>::load1(A, row0 + c);
            if (DIAG && c == r) { diag[r] = x; x = 0.0f; }
            m = max(m, abs_bits(x));
        }
        m = group_max_u32<64>(m);
        if (m > 0x7f800000u) m = 0x7fc00000u;
        if (lane == 0) absmax[seg] = __uint_as_float(m);
    }
}

// One thread per output byte; reads the maxima written by segment_max_kernel.
template <typename T, int BITS, bool DIAG>
__global__ __launch_bounds__(kThreads) void encode_kernel(
    const T *__restrict__ A, const float *__restrict__ code, uint32_t order, uint32_t bs, uint32_t nb,
    uint32_t total, const float *__restrict__ absmax, uint8_t *__restrict__ out) {
    constexpr int NCODE = 1 << BITS;
    constexpr uint32_t EPB = 8 / BITS;
    __shared__ CodeTables<NCODE> tab;
    build_code_tables<NCODE>(code, tab, nullptr);
    const uint32_t n_bytes = (total + EPB - 1) / EPB;
    for (uint32_t j = blockIdx.x * kThreads + threadIdx.x; j < n_bytes; j += gridDim.x * kThreads) {
        uint32_t byte = 0;
#pragma unroll
        for (uint32_t e = 0; e < EPB; ++e) {
            const uint32_t k = j * EPB + e;
            uint32_t id = 0;
            if (k < total) {
                const uint32_t r = k / order, c = k - r * order;
                float x = Vec4Loader<T>::load1(A, k);
                if (DIAG && r == c) x = 0.0f;
                id = exact_index<NCODE>(x, __float_as_uint(absmax[r * nb + c / bs]), tab);
            }
            byte = (byte << BITS) | id;
        }
        out[j] = (uint8_t)byte;
    }
}

int grid_for(uint32_t work_items_per_block_unit, int blocks_per_cu) {
    const int cap = compute_units() * blocks_per_cu;
    const int need = (int)work_items_per_block_unit;
    return need < 1 ? 1 : (need < cap ? need : cap);
}

template <typename T, int BITS, int BS, bool DIAG>
void launch_flat(const T *A, const float *code, uint32_t order, float *absmax, float *diag, uint8_t *out, hipStream_t stream) {
    constexpr uint32_t TILE = BS > 256 ? BS : 256;
    const uint32_t total = order * order;
    const uint32_t n_tiles = total / TILE;
    const FastDiv rd = make_fastdiv(order / 4);
    const uint32_t blocks_needed = (n_tiles + 3) / 4;
    // The bucket table costs a few microseconds of set-up per workgroup; it pays from about
    // a million elements on.
    if (total >= (1u << 20)) {
        const int grid = grid_for(blocks_needed, 5);
        hipLaunchKernelGGL((quantize_flat_kernel<T, BITS, BS, DIAG, true>), dim3(grid), dim3(kThreads), 0, stream,
                           A, code, n_tiles, rd, absmax, diag, out);
    } else {
        const int grid = grid_for(blocks_needed, 8);
        hipLaunchKernelGGL((quantize_flat_kernel<T, BITS, BS, DIAG, false>), dim3(grid), dim3(kThreads), 0, stream,
                           A, code, n_tiles, rd, absmax, diag, out);
    }
}

template <typename T, int BITS, bool DIAG>
void launch_general(const T *A, const float *code, uint32_t order, uint32_t bs, float *absmax, float *diag, uint8_t *out, hipStream_t stream) {
    const uint32_t nb = (order + bs - 1) / bs;
    const uint32_t n_segments = order * nb;
    const uint32_t total = order * order;
    hipLaunchKernelGGL((segment_max_kernel<T, DIAG>), dim3(grid_for((n_segments + 3) / 4, 8)), dim3(kThreads), 0, stream,
                       A, order, bs, nb, n_segments, absmax, diag);
    if (!launch_ok("segment_max_kernel")) return;
    const uint32_t n_bytes = (total * BITS + 7) / 8;
    hipLaunchKernelGGL((encode_kernel<T, BITS, DIAG>), dim3(grid_for((n_bytes + kThreads - 1) / kThreads, 8)), dim3(kThreads), 0, stream,
                       A, code, order, bs, nb, total, absmax, out);
}

template <typename T, int BITS, bool DIAG>
void quantize_dispatch(const T *A, const float *code, int order_i, float *absmax, float *diag, uint8_t *out, int blocksize, hipStream_t stream) {
    clear_error();
    if (!(blocksize == 64 || blocksize == 128 || blocksize == 256 || blocksize == 512 || blocksize == 1024 || blocksize == 2048)) {
        set_error(kBadBlocksize, "quantize_blockwise: blocksize %d is not one of 64,128,256,512,1024,2048", blocksize);
        return;
    }
    if (order_i < 1 || (int64_t)order_i * order_i >= (int64_t(1) << 31)) {
        set_error(kBadOrder, "quantize_blockwise: order %d out of range (need 1 <= order and order*order < 2^31)", order_i);
        return;
    }
    if (!A || !code || !absmax || !out || (DIAG && !diag)) {
        set_error(kNullPointer, "quantize_blockwise: null device pointer");
        return;
    }
    const uint32_t order = (uint32_t)order_i, bs = (uint32_t)blocksize;
    const bool flat = order % bs == 0 && is_aligned(A, 4 * sizeof(T)) && is_aligned(out, 4) && is_aligned(absmax, 4);
    if (flat) {
        switch (blocksize) {
            case 64: launch_flat<T, BITS, 64, DIAG>(A, code, order, absmax, diag, out, stream); break;
            case 128: launch_flat<T, BITS, 128, DIAG>(A, code, order, absmax, diag, out, stream); break;
            case 256: launch_flat<T, BITS, 256, DIAG>(A, code, order, absmax, diag, out, stream); break;
            case 512: launch_flat<T, BITS, 512, DIAG>(A, code, order, absmax, diag, out, stream); break;
            case 1024: launch_flat<T, BITS, 1024, DIAG>(A, code, order, absmax, diag, out, stream); break;
            default: launch_flat<T, BITS, 2048, DIAG>(A, code, order, absmax, diag, out, stream); break;
        }
    } else {
        launch_general<T, BITS, DIAG>(A, code, order, bs, absmax, diag, out, stream);
    }
    launch_ok("quantize_blockwise");
}

}  // namespace
}  // namespace qt

#define QT_DEFINE_QUANT(NAME, T, BITS)                                                                                   \
    extern "C" void cquantize_blockwise_##NAME##_stream(T *A, float *code, int order, float *absmax, unsigned char *out, \
                                                        int blocksize, void *stream) {                                   \
        qt::quantize_dispatch<T, BITS, false>(A, code, order, absmax, nullptr, out, blocksize, (hipStream_t)stream);     \
    }                                                                                                                    \
    extern "C" void cquantize_blockwise_##NAME(T *A, float *code, int order, float *absmax, unsigned char *out,          \
                                               int blocksize) {                                                          \
        qt::quantize_dispatch<T, BITS, false>(A, code, order, absmax, nullptr, out, blocksize, nullptr);                 \
    }                                                                                                                    \
    extern "C" void cquantize_blockwise_diagreal_##NAME##_stream(T *A, float *code, int order, float *absmax,            \
                                                                 float *diag, unsigned char *out, int blocksize,         \
                                                                 void *stream) {                                         \
        qt::quantize_dispatch<T, BITS, true>(A, code, order, absmax, diag, out, blocksize, (hipStream_t)stream);         \
    }                                                                                                                    \
    extern "C" void cquantize_blockwise_diagreal_##NAME(T *A, float *code, int order, float *absmax, float *diag,        \
                                                        unsigned char *out, int blocksize) {                             \
        qt::quantize_dispatch<T, BITS, true>(A, code, order, absmax, diag, out, blocksize, nullptr);                     \
    }

QT_DEFINE_QUANT(8bit_fp32, float, 8)
QT_DEFINE_QUANT(8bit_bf16, uint16_t, 8)
QT_DEFINE_QUANT(4bit_fp32, float, 4)
QT_DEFINE_QUANT(4bit_bf16, uint16_t, 4)
