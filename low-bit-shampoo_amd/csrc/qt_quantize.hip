// Blockwise quantize kernels for gfx950 (wave64) and their launchers.
//
// Two paths:
//  * flat path -- blocksize divides order.  The matrix is then a flat stream of whole segments
//    (segment s = elements [s*BS, (s+1)*BS), absmax index s).  A wave takes 2048 elements per
//    step as 8 coalesced 16-byte loads per lane, the segment maximum is a DPP butterfly, the
//    quotient is a correctly rounded fp32 division (one exact reciprocal per segment, then the
//    multiply / residual-fma / correction-fma sequence), and the index is a threshold count
//    done either through a bucket table in LDS (large inputs) or a binary search in LDS.
//  * general path -- any order/blocksize (ragged last segment, odd order with nibble pairs that
//    straddle rows): one pass for the maxima (a wave per segment), one pass per output byte.
//
// Arithmetic follows qtensor/functional.py:526-615 and :703-735 of the reference.
#include "qt_common.h"
#include "qt_tables.h"
#include "qt_divide.h"

namespace qt {
namespace {

#ifndef QT_Q_THREADS
#define QT_Q_THREADS 256
#endif
#ifndef QT_Q_BLOCKS_PER_CU
#define QT_Q_BLOCKS_PER_CU 3
#endif
constexpr int kThreads = 256;            // general-path kernels
constexpr int kFlatThreads = QT_Q_THREADS;
constexpr int kFlatBlocksPerCU = QT_Q_BLOCKS_PER_CU;
constexpr int kStep = 2048;              // elements a wave takes per step on the flat path

template <typename T> struct ElementLoader;
template <> struct ElementLoader<float> {
    template <bool STREAM>
    static __device__ __forceinline__ float4 load4(const float *base, uint32_t k) {
        return load_f32x4<STREAM>(base + k);
    }
    static __device__ __forceinline__ float load1(const float *base, size_t k) { return base[k]; }
};
template <> struct ElementLoader<uint16_t> {
    template <bool STREAM>
    static __device__ __forceinline__ float4 load4(const uint16_t *base, uint32_t k) {
        const uint2 w = load_u32x2<STREAM>(base + k);
        return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
                           __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u));
    }
    static __device__ __forceinline__ float load1(const uint16_t *base, size_t k) { return bf16_bits_to_float(base[k]); }
};

// Per-wave staging area: packed codes of one step in element order, and its segment maxima.
template <int BITS>
struct WaveStage {
    uint4 codes[BITS == 4 ? 64 : 128];
    float maxima[32];
};

// One step of a wave = 2048 consecutive elements, fetched as J = 8 fully coalesced 16-byte
// loads per lane (vector j of lane L covers elements 256 j + 4 L .. +3).  A segment is G = BS/4
// lanes of one vector for BS <= 256, and JS = BS/256 whole vectors of the wave above that.  The
// packed codes and the maxima are parked in LDS so that they leave as one contiguous 1 KiB
// (4-bit) or 2 KiB (8-bit) run and one run of 2048/BS floats per step.
template <typename T, int BITS, int BS, bool DIAG, bool USE_LUT, bool STREAM>
struct FlatQuantizer {
    static constexpr int NCODE = 1 << BITS;
    static constexpr int J = 8;
    static constexpr int JS = BS > 256 ? BS / 256 : 1;
    static constexpr int G = BS >= 256 ? 64 : BS / 4;
    static constexpr int SEGS = kStep / BS;

    const T *__restrict__ A;
    float *__restrict__ absmax;
    float *__restrict__ diag;
    uint8_t *__restrict__ out;
    const CodeTables<NCODE> &tab;
    const uint2 *lut;
    WaveStage<BITS> &stage;
    FastDiv row_div;                                        // by order/4
    FastDiv order_div;                                      // by order (rows of a stack -> row inside its matrix)
    bool fast_ok, ascending;
    uint32_t lane;

    struct Step {
        float4 v[J];
    };

    __device__ __forceinline__ void load(Step &s, uint32_t step) const {
        const uint32_t k0 = step * (uint32_t)kStep + lane * 4u;
#pragma unroll
        for (int j = 0; j < J; ++j) s.v[j] = ElementLoader<T>::template load4<STREAM>(A, k0 + (uint32_t)j * 256u);
    }

    __device__ __forceinline__ void process(Step &s, uint32_t step) const {
        if (DIAG) {
            const uint32_t k4 = step * (uint32_t)(kStep / 4) + lane;
            uint32_t row = fastdiv(k4, row_div);            // row of the stack of matrices
            uint32_t col4 = k4 - row * row_div.divisor;
            uint32_t lrow = row - fastdiv(row, order_div) * order_div.divisor;   // row inside its matrix
#pragma unroll
            for (int j = 0; j < J; ++j) {
                if ((lrow >> 2) == col4) {                  // this vector holds a diagonal element
                    const uint32_t e = lrow & 3u;
                    float4 &v = s.v[j];
                    diag[row] = e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w;
                    if (e == 0) v.x = 0.0f; else if (e == 1) v.y = 0.0f; else if (e == 2) v.z = 0.0f; else v.w = 0.0f;
                }
                col4 += 64u;
                while (col4 >= row_div.divisor) {
                    col4 -= row_div.divisor;
                    ++row;
                    if (++lrow == order_div.divisor) lrow = 0;
                }
            }
        }

        uint16_t *stage16 = reinterpret_cast<uint16_t *>(stage.codes);
        uint32_t *stage32 = reinterpret_cast<uint32_t *>(stage.codes);
#pragma unroll
        for (int jg = 0; jg < J; jg += JS) {
            uint32_t m = 0;
#pragma unroll
            for (int jj = 0; jj < JS; ++jj) {
                const float4 v = s.v[jg + jj];
                m = max(max(m, max(abs_bits(v.x), abs_bits(v.y))), max(abs_bits(v.z), abs_bits(v.w)));
            }
            m = group_max_u32<G>(m);

            // 2^-60 <= amax <= 2^60, else (zero, huge, tiny, inf, NaN) take the exact route
            const bool special = !fast_ok || (m - kFastDivLo) > (kFastDivHi - kFastDivLo);
            uint32_t idx[JS][4];
            if (__any(special)) {
                if (m > 0x7f800000u) m = 0x7fc00000u;       // any NaN in the segment -> canonical NaN
#pragma unroll
                for (int jj = 0; jj < JS; ++jj) {
                    const float4 v = s.v[jg + jj];
                    idx[jj][0] = exact_index<NCODE>(v.x, m, tab);
                    idx[jj][1] = exact_index<NCODE>(v.y, m, tab);
                    idx[jj][2] = exact_index<NCODE>(v.z, m, tab);
                    idx[jj][3] = exact_index<NCODE>(v.w, m, tab);
                }
            } else {
                const float amax = __uint_as_float(m);
                const float r = exact_reciprocal(amax);
#pragma unroll
                for (int jj = 0; jj < JS; ++jj) {
                    const float4 v = s.v[jg + jj];
                    idx[jj][0] = fast_index<NCODE, USE_LUT>(v.x, amax, r, tab, lut);
                    idx[jj][1] = fast_index<NCODE, USE_LUT>(v.y, amax, r, tab, lut);
                    idx[jj][2] = fast_index<NCODE, USE_LUT>(v.z, amax, r, tab, lut);
                    idx[jj][3] = fast_index<NCODE, USE_LUT>(v.w, amax, r, tab, lut);
                }
                if (!ascending) {
#pragma unroll
                    for (int jj = 0; jj < JS; ++jj)
#pragma unroll
                        for (int e = 0; e < 4; ++e) idx[jj][e] = tab.perm[idx[jj][e]];
                }
            }
            if ((lane & (G - 1)) == 0) stage.maxima[(jg * 256 + (int)lane * 4) / BS] = __uint_as_float(m);
#pragma unroll
            for (int jj = 0; jj < JS; ++jj) {
                const uint32_t *i = idx[jj];
                if (BITS == 4)
                    stage16[(jg + jj) * 64 + lane] = (uint16_t)(((i[0] << 4) | i[1]) | (((i[2] << 4) | i[3]) << 8));
                else
                    stage32[(jg + jj) * 64 + lane] = i[0] | (i[1] << 8) | (i[2] << 16) | (i[3] << 24);
            }
        }
        wave_lds_sync();
        uint4 *dst = reinterpret_cast<uint4 *>(out + (size_t)step * (kStep * BITS / 8));
        dst[lane] = stage.codes[lane];
        if (BITS == 8) dst[64 + lane] = stage.codes[64 + lane];
        if (lane < SEGS) absmax[step * (uint32_t)SEGS + lane] = stage.maxima[lane];
        wave_lds_sync();                                    // the next step rewrites the staging area
    }
};

template <typename T, int BITS, int BS, bool DIAG, bool USE_LUT, bool STREAM>
__global__ __launch_bounds__(kFlatThreads) void quantize_flat_kernel(
    const T *__restrict__ A, const float *__restrict__ code, uint32_t n_steps, FastDiv row_div, FastDiv order_div,
    float *__restrict__ absmax, float *__restrict__ diag, uint8_t *__restrict__ out) {
    using Q = FlatQuantizer<T, BITS, BS, DIAG, USE_LUT, STREAM>;
    constexpr int NCODE = Q::NCODE;
    constexpr int kWaves = kFlatThreads / 64;

    __shared__ CodeTables<NCODE> tab;
    __shared__ uint2 lut_mem[USE_LUT ? kLutEntries : 1];
    __shared__ WaveStage<BITS> stages[kWaves];
    uint2 *lut = USE_LUT ? lut_mem : nullptr;
    build_code_tables<NCODE>(code, tab, lut);
    const int flags = tab.flags;

    const uint32_t w = threadIdx.x >> 6;
    const Q q{A, absmax, diag, out, tab, lut, stages[w], row_div, order_div, (flags & kFlagLut) != 0,
              (flags & kFlagAscending) != 0, threadIdx.x & 63u};
    const uint32_t n_waves = gridDim.x * kWaves;
    uint32_t step = blockIdx.x * kWaves + w;
    if (step >= n_steps) return;
    // Two register buffers in ping-pong: the loads of the next step are in flight while the
    // current one is processed.  Look-ahead indices are clamped so every load is unconditional.
    const uint32_t last = n_steps - 1;
    typename Q::Step a, b;
    q.load(a, step);
    while (true) {
        q.load(b, min(step + n_waves, last));
        q.process(a, step);
        step += n_waves;
        if (step >= n_steps) break;
        q.load(a, min(step + n_waves, last));
        q.process(b, step);
        step += n_waves;
        if (step >= n_steps) break;
    }
}

// ---- general path ----------------------------------------------------------------------
// (blockIdx.y = matrix of a stack: every matrix has its own run of maxima, diagonal entries and code bytes, the
// codes of an odd order padded to a whole byte per matrix as the single-matrix format has them)
// One wave per segment; writes absmax (and diag).
template <typename T, bool DIAG>
__global__ __launch_bounds__(kThreads) void segment_max_kernel(
    const T *__restrict__ A, uint32_t order, uint32_t bs, uint32_t nb, uint32_t n_segments,
    float *__restrict__ absmax, float *__restrict__ diag) {
    A += (size_t)blockIdx.y * order * order;
    absmax += (size_t)blockIdx.y * n_segments;
    if (DIAG) diag += (size_t)blockIdx.y * order;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * (kThreads / 64);
    for (uint32_t seg = wave; seg < n_segments; seg += n_waves) {
        const uint32_t r = seg / nb, b = seg - r * nb;
        const uint32_t c0 = b * bs, c1 = min(c0 + bs, order);
        const size_t row0 = (size_t)r * order;
        uint32_t m = 0;
        for (uint32_t c = c0 + lane; c < c1; c += 64u) {
            float x = ElementLoader<T>::load1(A, row0 + c);
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
    A += (size_t)blockIdx.y * total;
    absmax += (size_t)blockIdx.y * order * nb;
    out += (size_t)blockIdx.y * n_bytes;
    for (uint32_t j = blockIdx.x * kThreads + threadIdx.x; j < n_bytes; j += gridDim.x * kThreads) {
        uint32_t byte = 0;
#pragma unroll
        for (uint32_t e = 0; e < EPB; ++e) {
            const uint32_t k = j * EPB + e;
            uint32_t id = 0;
            if (k < total) {
                const uint32_t r = k / order, c = k - r * order;
                float x = ElementLoader<T>::load1(A, k);
                if (DIAG && r == c) x = 0.0f;
                id = exact_index<NCODE>(x, __float_as_uint(absmax[r * nb + c / bs]), tab);
            }
            byte = (byte << BITS) | id;
        }
        out[j] = (uint8_t)byte;
    }
}

// ---- transposed source -----------------------------------------------------------------
// Quantizes the transpose of every matrix of a stack without writing the transpose out (the
// reference transposes first: V.T.contiguous() at qtensor/utils.py:169, then the plain quantizer).
// A workgroup takes BS input rows x 64 input columns, turns the tile around in LDS (row stride
// BS + 1: the scalar writes and reads below hit distinct banks for BS = 64), and every group of
// BS/4 lanes encodes one segment of an output row with the arithmetic of the flat path.
template <int BITS, int BS>
__global__ __launch_bounds__(kThreads) void quantize_transposed_kernel(
    const float *__restrict__ A, const float *__restrict__ code, uint32_t order, uint32_t n_tiles, uint32_t tiles_r, uint32_t tiles_c,
    float *__restrict__ absmax, uint8_t *__restrict__ out) {
    constexpr int NCODE = 1 << BITS;
    constexpr int LD = BS + 1;
    constexpr int G = BS / 4;                    // lanes per segment
    constexpr int SEGS = 64 / G;                 // segments a wave encodes at a time
    static_assert(BS == 64 || BS == 128 || BS == 256, "segment of 64, 128 or 256 elements");
    __shared__ CodeTables<NCODE> tab;
    __shared__ float tile[64 * LD];
    build_code_tables<NCODE>(code, tab, nullptr);
    const bool fast_ok = (tab.flags & kFlagLut) != 0, ascending = (tab.flags & kFlagAscending) != 0;
    const uint32_t t = threadIdx.x, lane = t & 63u, w = t >> 6;
    const uint32_t per_matrix = tiles_r * tiles_c;
    for (uint32_t id = blockIdx.x; id < n_tiles; id += gridDim.x) {
        const uint32_t b = id / per_matrix, rem = id - b * per_matrix;
        const uint32_t rb = rem / tiles_c, cb = rem - rb * tiles_c;
        const float *src = A + ((size_t)b * order + (size_t)rb * BS) * order + cb * 64u;
        const uint32_t c4 = (t & 15u) * 4u;
#pragma unroll
        for (int p = 0; p < BS / 16; ++p) {
            const uint32_t r = (uint32_t)p * 16u + (t >> 4);
            const float4 v = *reinterpret_cast<const float4 *>(src + (size_t)r * order + c4);
            tile[(c4 + 0) * LD + r] = v.x;
            tile[(c4 + 1) * LD + r] = v.y;
            tile[(c4 + 2) * LD + r] = v.z;
            tile[(c4 + 3) * LD + r] = v.w;
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 16 / SEGS; ++q) {
            const uint32_t cl = w * 16u + (uint32_t)q * SEGS + lane / G;       // output row inside the tile
            const uint32_t e0 = (lane % G) * 4u;                               // first of this lane's four elements
            float x[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = tile[cl * LD + e0 + e];
            uint32_t m = max(max(abs_bits(x[0]), abs_bits(x[1])), max(abs_bits(x[2]), abs_bits(x[3])));
            m = group_max_u32<G>(m);
            const bool special = !fast_ok || (m - kFastDivLo) > (kFastDivHi - kFastDivLo);
            uint32_t idx[4];
            if (__any(special)) {
                if (m > 0x7f800000u) m = 0x7fc00000u;
#pragma unroll
                for (int e = 0; e < 4; ++e) idx[e] = exact_index<NCODE>(x[e], m, tab);
            } else {
                const float amax = __uint_as_float(m);
                const float r = exact_reciprocal(amax);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    idx[e] = fast_index<NCODE, false>(x[e], amax, r, tab, nullptr);
                    if (!ascending) idx[e] = tab.perm[idx[e]];
                }
            }
            const size_t orow = (size_t)b * order + cb * 64u + cl;            // row of the stack of transposes
            if (lane % G == 0) absmax[orow * tiles_r + rb] = __uint_as_float(m);
            const size_t k = orow * order + (size_t)rb * BS + e0;             // flat element index of x[0]
            if (BITS == 4)
                *reinterpret_cast<uint16_t *>(out + (k >> 1)) = (uint16_t)(((idx[0] << 4) | idx[1]) | (((idx[2] << 4) | idx[3]) << 8));
            else
                *reinterpret_cast<uint32_t *>(out + k) = idx[0] | (idx[1] << 8) | (idx[2] << 16) | (idx[3] << 24);
        }
        __syncthreads();                                                       // the next tile rewrites the LDS copy
    }
}

int grid_for(uint32_t work_items_per_block_unit, int blocks_per_cu) {
    const int cap = compute_units() * blocks_per_cu;
    const int need = (int)work_items_per_block_unit;
    return need < 1 ? 1 : (need < cap ? need : cap);
}

template <typename T, int BITS, int BS, bool DIAG>
void launch_flat(const T *A, const float *code, uint32_t order, uint32_t batch, float *absmax, float *diag, uint8_t *out, hipStream_t stream) {
    constexpr uint32_t kWaves = kFlatThreads / 64;
    const uint32_t total = order * order * batch;
    const uint32_t n_steps = total / kStep;
    const FastDiv rd = make_fastdiv(order / 4), od = make_fastdiv(order);
    const uint32_t blocks_needed = (n_steps + kWaves - 1) / kWaves;
    const int grid = grid_for(blocks_needed, kFlatBlocksPerCU);
    // The bucket table costs a few microseconds of set-up per workgroup; it pays from about
    // a million elements on.  Inputs far beyond the 256 MB last-level cache are read with the
    // streaming hint.
    if (total >= (1u << 25)) {
        hipLaunchKernelGGL((quantize_flat_kernel<T, BITS, BS, DIAG, true, true>), dim3(grid), dim3(kFlatThreads), 0, stream,
                           A, code, n_steps, rd, od, absmax, diag, out);
    } else if (total >= (1u << 20)) {
        hipLaunchKernelGGL((quantize_flat_kernel<T, BITS, BS, DIAG, true, false>), dim3(grid), dim3(kFlatThreads), 0, stream,
                           A, code, n_steps, rd, od, absmax, diag, out);
    } else {
        hipLaunchKernelGGL((quantize_flat_kernel<T, BITS, BS, DIAG, false, false>), dim3(grid), dim3(kFlatThreads), 0, stream,
                           A, code, n_steps, rd, od, absmax, diag, out);
    }
}

template <typename T, int BITS, bool DIAG>
void launch_general(const T *A, const float *code, uint32_t order, uint32_t bs, uint32_t batch, float *absmax, float *diag, uint8_t *out,
                    hipStream_t stream) {
    const uint32_t nb = (order + bs - 1) / bs;
    const uint32_t n_segments = order * nb;
    const uint32_t total = order * order;
    hipLaunchKernelGGL((segment_max_kernel<T, DIAG>), dim3(grid_for((n_segments + 3) / 4, 8), batch), dim3(kThreads), 0, stream,
                       A, order, bs, nb, n_segments, absmax, diag);
    if (!launch_ok("segment_max_kernel")) return;
    const uint32_t n_bytes = (total * BITS + 7) / 8;
    hipLaunchKernelGGL((encode_kernel<T, BITS, DIAG>), dim3(grid_for((n_bytes + kThreads - 1) / kThreads, 8), batch), dim3(kThreads), 0, stream,
                       A, code, order, bs, nb, total, absmax, out);
}

template <typename T, int BITS, bool DIAG>
void quantize_dispatch(const T *A, const float *code, int order_i, float *absmax, float *diag, uint8_t *out, int blocksize, hipStream_t stream,
                       int batch = 1) {
    clear_error();
    if (!(blocksize == 64 || blocksize == 128 || blocksize == 256 || blocksize == 512 || blocksize == 1024 || blocksize == 2048)) {
        set_error(kBadBlocksize, "quantize_blockwise: blocksize %d is not one of 64,128,256,512,1024,2048", blocksize);
        return;
    }
    if (order_i < 1 || batch < 1 || (int64_t)order_i * order_i * batch >= (int64_t(1) << 31)) {
        set_error(kBadOrder, "quantize_blockwise: order %d (batch %d) out of range (need order >= 1 and batch*order*order < 2^31)",
                  order_i, batch);
        return;
    }
    if (!A || !code || !absmax || !out || (DIAG && !diag)) {
        set_error(kNullPointer, "quantize_blockwise: null device pointer");
        return;
    }
    const uint32_t order = (uint32_t)order_i, bs = (uint32_t)blocksize;
    const bool flat = order % bs == 0 && is_aligned(A, 4 * sizeof(T)) && is_aligned(out, 16) && is_aligned(absmax, 4);
    if (batch > 65535 && !flat) {
        set_error(kBadArgument, "quantize_blockwise: a stack whose order the blocksize does not divide (or with unaligned buffers) "
                                "takes at most 65535 matrices per launch");
        return;
    }
    if (flat) {
        switch (blocksize) {
            case 64: launch_flat<T, BITS, 64, DIAG>(A, code, order, (uint32_t)batch, absmax, diag, out, stream); break;
            case 128: launch_flat<T, BITS, 128, DIAG>(A, code, order, (uint32_t)batch, absmax, diag, out, stream); break;
            case 256: launch_flat<T, BITS, 256, DIAG>(A, code, order, (uint32_t)batch, absmax, diag, out, stream); break;
            case 512: launch_flat<T, BITS, 512, DIAG>(A, code, order, (uint32_t)batch, absmax, diag, out, stream); break;
            case 1024: launch_flat<T, BITS, 1024, DIAG>(A, code, order, (uint32_t)batch, absmax, diag, out, stream); break;
            default: launch_flat<T, BITS, 2048, DIAG>(A, code, order, (uint32_t)batch, absmax, diag, out, stream); break;
        }
    } else {
        launch_general<T, BITS, DIAG>(A, code, order, bs, (uint32_t)batch, absmax, diag, out, stream);
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

extern "C" void qtensor_hip_quantize_batched(const void *A, int a_is_bf16, const float *code, int bits, int order, int batch,
                                             float *absmax, float *diag, unsigned char *out, int blocksize, void *stream) {
    using namespace qt;
    hipStream_t st = (hipStream_t)stream;
    float *c = const_cast<float *>(code);
    (void)c;
    if (bits != 4 && bits != 8) { clear_error(); set_error(kBadArgument, "quantize_batched: bits must be 4 or 8"); return; }
#define QT_QB(T, BITS)                                                                                        \
    (diag ? quantize_dispatch<T, BITS, true>((const T *)A, code, order, absmax, diag, out, blocksize, st, batch)    \
          : quantize_dispatch<T, BITS, false>((const T *)A, code, order, absmax, nullptr, out, blocksize, st, batch))
    if (a_is_bf16) { if (bits == 4) QT_QB(uint16_t, 4); else QT_QB(uint16_t, 8); }
    else { if (bits == 4) QT_QB(float, 4); else QT_QB(float, 8); }
#undef QT_QB
}

extern "C" void qtensor_hip_quantize_transposed_batched(const float *A, const float *code, int bits, int order, int batch,
                                                        float *absmax, unsigned char *out, int blocksize, void *stream) {
    using namespace qt;
    clear_error();
    if (bits != 4 && bits != 8) { set_error(kBadArgument, "quantize_transposed: bits must be 4 or 8"); return; }
    if (blocksize != 64 && blocksize != 128 && blocksize != 256) {
        set_error(kBadBlocksize, "quantize_transposed: blocksize %d is not one of 64,128,256", blocksize);
        return;
    }
    if (order < 1 || batch < 1 || (int64_t)order * order * batch >= (int64_t(1) << 31) || order % blocksize != 0 || order % 64 != 0) {
        set_error(kBadOrder, "quantize_transposed: order %d (batch %d) must be a multiple of 64 and of the blocksize, batch*order*order < 2^31",
                  order, batch);
        return;
    }
    if (!A || !code || !absmax || !out) { set_error(kNullPointer, "quantize_transposed: null device pointer"); return; }
    if (!is_aligned(A, 16) || !is_aligned(out, 4) || !is_aligned(absmax, 4)) {
        set_error(kBadArgument, "quantize_transposed: A needs 16-byte, out and absmax 4-byte alignment");
        return;
    }
    const uint32_t tiles_r = (uint32_t)(order / blocksize), tiles_c = (uint32_t)(order / 64);
    const uint32_t n_tiles = tiles_r * tiles_c * (uint32_t)batch;
    const int grid = grid_for(n_tiles, blocksize == 256 ? 2 : 4);
#define QT_QT(BITS, BS)                                                                                                  \
    hipLaunchKernelGGL((quantize_transposed_kernel<BITS, BS>), dim3(grid), dim3(kThreads), 0, (hipStream_t)stream, A, code, \
                       (uint32_t)order, n_tiles, tiles_r, tiles_c, absmax, out)
    if (bits == 4) { if (blocksize == 64) QT_QT(4, 64); else if (blocksize == 128) QT_QT(4, 128); else QT_QT(4, 256); }
    else { if (blocksize == 64) QT_QT(8, 64); else if (blocksize == 128) QT_QT(8, 128); else QT_QT(8, 256); }
#undef QT_QT
    launch_ok("quantize_transposed");
}
