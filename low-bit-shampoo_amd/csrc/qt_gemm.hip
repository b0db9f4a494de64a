// Products of fp32 matrices on the gfx950 matrix cores, with blockwise quantized operands expanded on their
// way into LDS and the Shampoo epilogues fused in.  Two pipes: the fp32 one (v_mfma_f32_32x32x2_f32) and, by
// default, the bf16 one on operands split into three bf16 pieces each (v_mfma_f32_32x32x16_bf16, six products
// per fp32 product, fp32 accumulation: fp32-grade results at a multiple of the rate; see kPipeSplit below).
//
// What the reference does with separate steps
//   P = dequantize(Pq);  out = P @ G            (optimizers/shampoo2.py:255-268, shampoo1.py:224-237)
//   S = G @ G.T;  L = dequantize(Lq);  L.mul_(b).add_(S, alpha=1-b)   (shampoo1.py:164-178)
//   the matmuls of the coupled Newton iteration  (optimizers/matrix_functions.py:131-140)
// is done here as one launch per product over a whole batch of equally shaped problems.
//
// C[b] = epilogue( opA(A[b]) * opB(B[b]) ), b = blockIdx.z.  Row-major everywhere.
//   operand kinds: dense (k contiguous for A, n contiguous for B), dense transposed, or a
//   square 4/8-bit blockwise-quantized matrix (flat layout: blocksize divides the order).
//   epilogues: plain store | beta * E + alpha * acc with E dense or quantized |
//              Newton: C = acc, T = (1 - w) I + w * acc, err = max |acc - I|.
//
// Tiling: workgroup = 4 waves in a 2 x 2 grid, block tile BM x BN x 16, each wave owns
// (BM/2) x (BN/2) as 32 x 32 MFMA blocks.  An operand tile sits in LDS the way its source is
// contiguous -- [row][k] (stride 20) when k is, [k][row] (stride rows + 4) otherwise -- so every
// commit is a 16-byte store; fragments come out as one 16-byte read per four MFMA steps or as
// consecutive words per step.  Global loads run two tiles ahead of the MFMAs; the LDS commit sits
// in the middle of the MFMA stream.  (Split pipe: three bf16 planes per operand tile, [half of k][row][8].)
#include "qt_common.h"
#include "qt_tables.h"

#include <atomic>
#include <cmath>
#include <cstring>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#ifndef QT_STREAMK
#define QT_STREAMK 1
#endif
// Tuning knobs of the tile / k-cut choice (environment variables QT_GEMM_TILE, QT_GEMM_SPLIT, QT_GEMM_STREAM_WGS,
// QT_GEMM_STREAM_MIN) exist only in builds made with -DQT_TUNING_KNOBS: they change the summation order of a
// product, which a release build promises not to depend on anything but the operands' shapes.
#ifdef QT_TUNING_KNOBS
#define QT_KNOB(name) getenv(name)
#else
#define QT_KNOB(name) (static_cast<const char *>(nullptr))
#endif

namespace qt {

enum OperandKind : int { kDense = 0, kDenseT = 1, kQuant4 = 2, kQuant8 = 3 };
enum EpilogueKind : int { kStore = 0, kAxpbyDense = 1, kAxpbyQuant4 = 2, kAxpbyQuant8 = 3, kNewton = 4, kRequant4 = 5, kRequant8 = 6 };

// One matrix argument over the batch: either base + b * stride, or list[b] when list != nullptr.
struct BatchPtr {
    const void *base;
    const void *const *list;
    long long stride;   // in elements of the pointee type
};

struct QuantRef {       // a square blockwise-quantized matrix per batch entry
    BatchPtr codes;     // uint8
    BatchPtr absmax;    // float
    BatchPtr diag;      // float, base == nullptr and list == nullptr: plain (no exact diagonal)
    int order;
    int bs_shift;       // log2(blocksize)
};

struct GemmArgs {
    int M, N, K;
    BatchPtr A; int lda;          // dense A: M x K (lda) or, transposed, K x M (lda)
    BatchPtr B; int ldb;          // dense B: K x N (ldb) or, transposed, N x K (ldb)
    QuantRef Aq, Bq;              // used when the operand kind is quantized
    BatchPtr C; int ldc;
    float alpha, beta;
    BatchPtr E; int lde;          // dense addend for kAxpbyDense
    QuantRef Eq;                  // quantized addend for kAxpbyQuant*
    BatchPtr T; int ldt;          // kNewton: second output
    float newton_w;               // kNewton: T = (1 - w) I + w acc
    float *err;                   // kNewton: err[b] = max |acc - I| (must be zeroed by the caller)
    const int *skip;              // optional: skip[b] != 0 -> this batch entry is left untouched
    const float *code;            // code table for quantized operands / addend
    int symmetric;                // != 0: the product is symmetric (M == N); only tiles on or above the
                                  // diagonal are computed and every off-diagonal tile is also written mirrored
    float *workspace;             // optional scratch for splitting k (plain-store products only)
    long long workspace_floats;
    int split_k;                  // set by the library: slices of the k range (1 = no split)
    int batch_count;              // set by the library: batch entries of this launch
    int stream_per, stream_lcm;   // set by the library: > 0 = the k tiles of all output tiles, laid end to end, are dealt
                                  // out in runs of stream_per to the workgroups (a run may end inside one output tile and
                                  // go on in the next); stream_lcm = lcm(stream_per, k tiles per output tile)
    int batch_inner;              // > 1: batch entry b of the strided dense operands A, B, C, E lives at
    long long inner_a, inner_b, inner_c, inner_e;   // base + (b / batch_inner) * stride + (b % batch_inner) * inner_x
    int triangular;               // bit 0: A is upper triangular (A[m][k] = 0 for k < m): k starts at the tile's first row;
                                  // bit 1: B is upper triangular (B[k][n] = 0 for k > n): k ends with the tile's last column
    int pipe;                     // 0: the process-wide choice (qtensor_hip_gemm_pipe); 1: the fp32 pipe; 2: the split bf16 pipe
};

namespace {

constexpr int BK = 16;
// Which matrix pipe multiplies.  kPipeF32: v_mfma_f32_32x32x2_f32 on the operands as they are.  kPipeSplit: every fp32
// operand element is written as the sum of three bf16 numbers (x = h + m + l, each the rounding of what the ones before
// leave over: |x - h - m - l| <= 2^-24 |x|) and a product a b is the six bf16 products a_h b_h + a_h b_m + a_m b_h +
// a_h b_l + a_l b_h + a_m b_m, each exact in fp32, accumulated in fp32 by v_mfma_f32_32x32x16_bf16.  The terms left out
// are below 2^-24 |a b|: the error of a dot product stays that of fp32 arithmetic, and the bf16 pipe does sixteen times
// the multiply-adds per cycle of the fp32 pipe, six of which make one fp32 multiply-add.
constexpr int kPipeF32 = 0, kPipeSplit = 1;
constexpr uint32_t kDies = 8;          // accelerator dies (XCDs) of an MI355X
constexpr int LDS_PAD = 4;   // k-major tiles ([k][row]): row stride = rows + 4 floats, 16-byte aligned rows
constexpr int LDK = BK + 4;  // row-major tiles ([row][k], for sources whose k is contiguous): 20 floats per row, so
                             // that the 16-byte fragment reads of 8 consecutive lanes cover all 32 banks
typedef float f32x16 __attribute__((ext_vector_type(16)));
// Pointers that arrive inside a by-value struct or from a pointer table are "generic" to the
// compiler, which then emits flat_* instructions (slower, and they also count on the LDS wait
// counter).  Everything here lives in global memory: say so.
#define QT_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ float gload(const float *p) { return *(const QT_GLOBAL float *)p; }
__device__ __forceinline__ float4 gload4(const float *p) {
    const qt_f32x4 v = *(const QT_GLOBAL qt_f32x4 *)p;
    return make_float4(v.x, v.y, v.z, v.w);
}
// A word or four at `base` (the same for the whole wave) plus a byte offset of 32 bits per lane: the form of the
// load instruction that takes the base from scalar registers, so that moving the base costs no vector arithmetic.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t whole_range(const float *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, -1, 0x00020000);
}
// A pointer that is the same in every lane, as a value the compiler knows to be: without that it wraps every buffer
// load into a loop over the distinct values of its base.
__device__ __forceinline__ const float *wave_uniform(const float *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return reinterpret_cast<const float *>(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ float gload_at(const float *base, uint32_t byte_off) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(whole_range(base), (int)byte_off, 0, 0));
}
__device__ __forceinline__ float4 gload4_at(const float *base, uint32_t byte_off) {
    const qt_u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(whole_range(base), (int)byte_off, 0, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ uint32_t gload_u32(const void *p) { return *(const QT_GLOBAL uint32_t *)p; }
__device__ __forceinline__ uint2 gload_u32x2(const void *p) {
    const qt_u32x2 v = *(const QT_GLOBAL qt_u32x2 *)p;
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t gload_u8(const uint8_t *p) { return *(const QT_GLOBAL uint8_t *)p; }
__device__ __forceinline__ uint32_t gload_u16(const void *p) { return *(const QT_GLOBAL uint16_t *)p; }
__device__ __forceinline__ void gstore(float *p, float v) { *(QT_GLOBAL float *)p = v; }
__device__ __forceinline__ void gstore4(float *p, const float v[4]) {
    qt_f32x4 x;
    x.x = v[0]; x.y = v[1]; x.z = v[2]; x.w = v[3];
    *(QT_GLOBAL qt_f32x4 *)p = x;
}

template <typename T>
__device__ __forceinline__ const T *batch_ptr(const BatchPtr &p, int b) {
    return p.list ? reinterpret_cast<const T *>(p.list[b]) : reinterpret_cast<const T *>(p.base) + (long long)b * p.stride;
}

// Dense operand of batch entry b when the batch has two levels (blocks inside the matrices of a stack).
__device__ __forceinline__ const float *dense_ptr(const BatchPtr &p, int b, int inner, long long inner_stride) {
    if (p.list || inner <= 1) return batch_ptr<float>(p, b);
    const int outer = b / inner;
    return reinterpret_cast<const float *>(p.base) + outer * p.stride + (b - outer * inner) * inner_stride;
}

__device__ __forceinline__ bool has_ptr(const BatchPtr &p) { return p.base != nullptr || p.list != nullptr; }
inline bool has_host_ptr(const BatchPtr &p) { return p.base != nullptr || p.list != nullptr; }

// Dequantized element (r, c) of a flat-layout quantized matrix.
template <int BITS>
__device__ __forceinline__ float dequant_element(const uint8_t *codes, const float *absmax, const float *diag,
                                                 const float *s_code, int order, int bs_shift, int r, int c) {
    if (diag != nullptr && r == c) return gload(diag + r);
    const long long k = (long long)r * order + c;
    uint32_t id;
    if (BITS == 8) id = gload_u8(codes + k);
    else { const uint32_t byte = gload_u8(codes + (k >> 1)); id = (k & 1) ? (byte & 15u) : (byte >> 4); }
    const float a = gload(absmax + (k >> bs_shift));
    return a == 0.0f ? 0.0f : s_code[id] * a;
}

// Four consecutive off-diagonal elements (r, c0 .. c0+3), c0 a multiple of 4, of the same matrix.
template <int BITS>
__device__ __forceinline__ void dequant_four(const uint8_t *codes, const float *absmax, const float *s_code, int order,
                                             int bs_shift, int r, int c0, float out[4]) {
    const long long k = (long long)r * order + c0;
    uint32_t id[4];
    if (BITS == 8) {
        const uint32_t w = gload_u32(codes + k);
#pragma unroll
        for (int e = 0; e < 4; ++e) id[e] = (w >> (8 * e)) & 255u;
    } else {
        const uint32_t w = gload_u16(codes + (k >> 1));
        id[0] = (w >> 4) & 15u; id[1] = w & 15u; id[2] = (w >> 12) & 15u; id[3] = (w >> 8) & 15u;
    }
    const float a = gload(absmax + (k >> bs_shift));
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = a == 0.0f ? 0.0f : s_code[id[e]] * a;
}

// ---- tile loaders: global -> registers -> LDS ([k][row], row stride rows + LDS_PAD) -------------
// Every loader covers ROWS x BK elements with 256 threads and keeps them in registers between
// `fetch` (global loads, issued early) and `commit` (LDS stores, after the barrier).

// Dense, k contiguous in memory: element (row, k) at base[row * ld + k].
template <int ROWS>
struct LoadKContig {
    static constexpr bool kRowMajor = true;                  // lands in LDS as [row][k]
    static constexpr int VEC = ROWS * BK / 4 / 256;          // float4 per thread
    float4 v[VEC];
    int off[VEC];
    // Fast path (whole k tiles, 16-byte aligned rows): per-thread offsets are fixed for the whole
    // product, rows beyond the matrix are clamped (their results are never stored), and a tile
    // load is `uniform tile base + offset` with no predicate.
    __device__ __forceinline__ void prepare(int ld, int row0, int rows) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int f = threadIdx.x + i * 256;
            const int r = f / (BK / 4), kq = (f % (BK / 4)) << 2;
            off[i] = min(row0 + r, rows - 1) * ld + kq;
        }
    }
    __device__ __forceinline__ void fetch_fast(const float *tile_base) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = gload4(tile_base + off[i]);
    }
    __device__ __forceinline__ void fetch(const float *base, int ld, int row0, int k0, int rows, int K, bool vec_ok) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int f = threadIdx.x + i * 256;
            const int r = f / (BK / 4), kq = (f % (BK / 4)) << 2;
            const int gr = row0 + r, gk = k0 + kq;
            float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
            if (gr < rows) {
                const float *p = base + (long long)gr * ld + gk;
                if (vec_ok && gk + 3 < K) x = gload4(p);
                else {
                    if (gk < K) x.x = gload(p);
                    if (gk + 1 < K) x.y = gload(p + 1);
                    if (gk + 2 < K) x.z = gload(p + 2);
                    if (gk + 3 < K) x.w = gload(p + 3);
                }
            }
            v[i] = x;
        }
    }
    __device__ __forceinline__ void commit(float *lds, const float *) const {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int f = threadIdx.x + i * 256;
            const int r = f / (BK / 4), kq = (f % (BK / 4)) << 2;
            *reinterpret_cast<float4 *>(lds + r * LDK + kq) = v[i];
        }
    }
};

// Dense, row index contiguous in memory: element (row, k) at base[k * ld + row].
template <int ROWS>
struct LoadRowContig {
    static constexpr bool kRowMajor = false;                 // lands in LDS as [k][row]
    static constexpr int VEC = ROWS * BK / 4 / 256;
    float4 v[VEC];
    int off[VEC];
    __device__ __forceinline__ void prepare(int ld, int row0, int rows) {      // rows is a multiple of 4 here
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int f = threadIdx.x + i * 256;
            const int kk = f / (ROWS / 4), rq = (f % (ROWS / 4)) << 2;
            off[i] = kk * ld + min(row0 + rq, rows - 4);
        }
    }
    __device__ __forceinline__ void fetch_fast(const float *tile_base) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = gload4(tile_base + off[i]);
    }
    __device__ __forceinline__ void fetch(const float *base, int ld, int row0, int k0, int rows, int K, bool vec_ok) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int f = threadIdx.x + i * 256;
            const int kk = f / (ROWS / 4), rq = (f % (ROWS / 4)) << 2;
            const int gk = k0 + kk, gr = row0 + rq;
            float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
            if (gk < K) {
                const float *p = base + (long long)gk * ld + gr;
                if (vec_ok && gr + 3 < rows) x = gload4(p);
                else {
                    if (gr < rows) x.x = gload(p);
                    if (gr + 1 < rows) x.y = gload(p + 1);
                    if (gr + 2 < rows) x.z = gload(p + 2);
                    if (gr + 3 < rows) x.w = gload(p + 3);
                }
            }
            v[i] = x;
        }
    }
    __device__ __forceinline__ void commit(float *lds, const float *) const {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int f = threadIdx.x + i * 256;
            const int kk = f / (ROWS / 4), rq = (f % (ROWS / 4)) << 2;
            *reinterpret_cast<float4 *>(lds + kk * (ROWS + LDS_PAD) + rq) = v[i];
        }
    }
};

// ---- loaders of the split pipe: global -> registers (fp32) -> LDS (three bf16 planes) -----------
// A plane of an operand tile of ROWS rows holds, for each half of the 16 k of a tile, the 8 values of every row as 16
// bytes: [half][row][8 bf16], the halves kSplitHalfPad bytes further apart than they need be so that the 16-byte
// stores of two threads that differ in the half fall into different banks.  A lane's MFMA fragment (8 consecutive k of
// one row) is then one 16-byte read, and the 32 lanes of a half read 512 contiguous bytes.
typedef __bf16 qt_bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 qt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float qt_f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t qt_u32x4 __attribute__((ext_vector_type(4)));
constexpr int kSplitHalfPad = 64;
template <int ROWS> struct SplitLayout {
    static constexpr int kHalf = ROWS * 16 + kSplitHalfPad, kPlane = 2 * kHalf, kOperand = 3 * kPlane;   // bytes
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {       // round to nearest even, a in the low half
    const qt_f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, qt_bf16x2));
}
__device__ __forceinline__ float low_bf16(uint32_t p) { return __builtin_bit_cast(float, p << 16); }
__device__ __forceinline__ float high_bf16(uint32_t p) { return __builtin_bit_cast(float, p & 0xffff0000u); }

// 8 floats -> their three bf16 planes (4 packed words each); the subtractions are exact
__device__ __forceinline__ void split_eight(const float x[8], qt_u32x4 &h, qt_u32x4 &m, qt_u32x4 &l) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float a = x[2 * i], b = x[2 * i + 1];
        const uint32_t ph = pack_bf16(a, b);
        const float ra = a - low_bf16(ph), rb = b - high_bf16(ph);
        const uint32_t pm = pack_bf16(ra, rb);
        const float sa = ra - low_bf16(pm), sb = rb - high_bf16(pm);
        h[i] = ph; m[i] = pm; l[i] = pack_bf16(sa, sb);
    }
}

template <int ROWS>
__device__ __forceinline__ void commit_split_eight(unsigned char *operand, int row, int half, const float x[8]) {
    using L = SplitLayout<ROWS>;
    qt_u32x4 h, m, l;
    split_eight(x, h, m, l);
    unsigned char *at = operand + half * L::kHalf + row * 16;
    *reinterpret_cast<qt_u32x4 *>(at) = h;
    *reinterpret_cast<qt_u32x4 *>(at + L::kPlane) = m;
    *reinterpret_cast<qt_u32x4 *>(at + 2 * L::kPlane) = l;
}

// 4 floats -> their three bf16 planes (2 packed words each)
__device__ __forceinline__ void split_four(const float x[4], uint2 &h, uint2 &m, uint2 &l) {
    uint32_t hh[2], mm[2], ll[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const float a = x[2 * i], b = x[2 * i + 1];
        const uint32_t ph = pack_bf16(a, b);
        const float ra = a - low_bf16(ph), rb = b - high_bf16(ph);
        const uint32_t pm = pack_bf16(ra, rb);
        const float sa = ra - low_bf16(pm), sb = rb - high_bf16(pm);
        hh[i] = ph; mm[i] = pm; ll[i] = pack_bf16(sa, sb);
    }
    h = make_uint2(hh[0], hh[1]); m = make_uint2(mm[0], mm[1]); l = make_uint2(ll[0], ll[1]);
}

template <int ROWS>
__device__ __forceinline__ void commit_split_four(unsigned char *operand, int row, int quarter, const float x[4]) {
    using L = SplitLayout<ROWS>;
    uint2 h, m, l;
    split_four(x, h, m, l);
    unsigned char *at = operand + (quarter >> 1) * L::kHalf + row * 16 + (quarter & 1) * 8;
    *reinterpret_cast<uint2 *>(at) = h;
    *reinterpret_cast<uint2 *>(at + L::kPlane) = m;
    *reinterpret_cast<uint2 *>(at + 2 * L::kPlane) = l;
}

// Dense, k contiguous in memory (element (row, k) at base[row * ld + k]); whole k tiles.  128 rows: thread t takes 8
// consecutive k (half t & 1) of row t >> 1; 64 rows: 4 consecutive k (quarter t & 3) of row t >> 2.  Rows beyond the
// matrix are clamped (their products are never stored).  `vec`: rows are 16-byte aligned (the same for the whole
// workgroup); otherwise word loads.
// The loads take the tile's base from scalar registers and a byte offset of 32 bits per lane that stays the same from
// tile to tile (buffer loads), so that moving on to the next tile costs no vector arithmetic: with a pointer per lane the
// compiler advances one 64-bit address per load and tile.
template <int ROWS>
struct SplitKContig {
    static_assert(ROWS == 128 || ROWS == 64, "tile rows");
    static constexpr int PER = ROWS * BK / 256;
    float v[PER];
    long long first;                    // elements from the operand's origin to the tile's first row (the same for all lanes)
    uint32_t off;                       // bytes from there to this lane's first word (the host keeps 128 rows inside 32 bits)
    bool vec = true;
    __device__ __forceinline__ void prepare(int ld, int row0, int rows) {
        const int row = ROWS == 128 ? threadIdx.x >> 1 : threadIdx.x >> 2, part = ROWS == 128 ? threadIdx.x & 1 : threadIdx.x & 3;
        first = (long long)row0 * ld;
        off = (uint32_t)((min(row0 + row, rows - 1) - row0) * ld + part * PER) * 4u;
    }
    __device__ __forceinline__ void fetch_fast(const float *tile_base) {
        const float *base = tile_base + first;
        if (vec) {
#pragma unroll
            for (int q = 0; q < PER / 4; ++q) {
                const float4 x = gload4_at(base, off + 16u * q);
                v[4 * q] = x.x; v[4 * q + 1] = x.y; v[4 * q + 2] = x.z; v[4 * q + 3] = x.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < PER; ++j) v[j] = gload_at(base, off + 4u * j);
        }
    }
    __device__ __forceinline__ void commit_split(unsigned char *operand) const {
        if constexpr (ROWS == 128) commit_split_eight<ROWS>(operand, threadIdx.x >> 1, threadIdx.x & 1, v);
        else commit_split_four<ROWS>(operand, threadIdx.x >> 2, threadIdx.x & 3, v);
    }
};

// Dense, row index contiguous in memory (element (row, k) at base[k * ld + row]); whole k tiles.  128 rows: thread t
// takes row t & 127 and the 8 k of half t >> 7; 64 rows: row t & 63 and the 4 k of quarter t >> 6; one word per load,
// a wave's load covers 64 consecutive words.  Scalar base and per-lane byte offsets as above.
template <int ROWS>
struct SplitRowContig {
    static_assert(ROWS == 128 || ROWS == 64, "tile rows");
    static constexpr int PER = ROWS * BK / 256;
    float v[PER];
    int first;                          // the tile's first row (the same for all lanes)
    uint32_t off[PER];                  // bytes from there to each of this lane's words
    __device__ __forceinline__ void prepare(int ld, int row0, int rows) {
        const int row = threadIdx.x & (ROWS - 1), part = ROWS == 128 ? threadIdx.x >> 7 : threadIdx.x >> 6;
        first = row0;
#pragma unroll
        for (int j = 0; j < PER; ++j) off[j] = (uint32_t)((part * PER + j) * ld + (min(row0 + row, rows - 1) - row0)) * 4u;
    }
    __device__ __forceinline__ void fetch_fast(const float *tile_base) {
        const float *base = tile_base + first;
#pragma unroll
        for (int j = 0; j < PER; ++j) v[j] = gload_at(base, off[j]);
    }
    __device__ __forceinline__ void commit_split(unsigned char *operand) const {
        if constexpr (ROWS == 128) commit_split_eight<ROWS>(operand, threadIdx.x & 127, threadIdx.x >> 7, v);
        else commit_split_four<ROWS>(operand, threadIdx.x & 63, threadIdx.x >> 6, v);
    }
};

// Quantized square matrix (order x order, flat layout).  ALONG_K: the tile's k runs along the
// matrix columns (left factor); otherwise the tile's rows run along the matrix columns (right
// factor).  Each thread expands 8 consecutive codes of one matrix row.
// TURNED (split pipe, right factor): the 8 lanes of a group take 8 consecutive k, so that a group holds an 8 x 8 square
// (k x tile row) which one pass through LDS turns around into 8 consecutive k per tile row.
template <int ROWS, int BITS, bool ALONG_K, bool TURNED = false>
struct LoadQuant {
    static_assert(!(TURNED && ALONG_K), "only the right factor is turned");
    static constexpr bool kRowMajor = ALONG_K;               // 8 consecutive k of one row: [row][k]; else [k][row]
    static constexpr int TOTAL = ROWS * BK / 8;              // 8-element groups in the tile
    static constexpr int GROUPS = (TOTAL + 255) / 256;       // per thread
    // `fetch` only issues the global loads (packed codes, the segment maximum, the exact diagonal
    // entry); the table lookups wait until `commit`, one tile later, when the loads have long
    // landed.  The order is a multiple of 64, hence of the tile depth: no k bounds; groups beyond the
    // matrix are clamped into it (their products are never stored).  Offsets are split into a fixed
    // per-thread part (`prepare`) and a part that is uniform over the workgroup per tile.
    uint2 raw[GROUPS];
    float amax[GROUPS];
    float dval[GROUPS];
    int dpos[GROUPS];                                        // element of the group on the diagonal, if in 0..7
    int code_off[GROUPS], amax_off[GROUPS], d0[GROUPS], drow[GROUPS];
    const uint8_t *codes;
    const float *absmax, *diag;
    int order, per_row, shift, first_row;
    bool on_diagonal;                                        // the fetched tile holds diagonal entries (uniform over the workgroup)
    __device__ __forceinline__ bool active(int g) const { return (int)threadIdx.x + g * 256 < TOTAL; }
    __device__ __forceinline__ void locate(int g, int &mr, int &mc) const {
        const int f = threadIdx.x + g * 256;
        if (ALONG_K) { mr = f % ROWS; mc = (f / ROWS) << 3; }               // tile row = matrix row, 2 groups per row
        else if (TURNED) {                                                  // wave: half of k and 64 tile rows; lane: k and group
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
            mr = 8 * (wave & 1) + (lane & 7);
            mc = (8 * (wave >> 1) + ((lane >> 3) & 7)) << 3;
        }
        else { mr = f / (ROWS / 8); mc = (f % (ROWS / 8)) << 3; }           // tile k = matrix row
    }
    __device__ __forceinline__ void prepare(const QuantRef &q, int b, int row0) {
        codes = batch_ptr<uint8_t>(q.codes, b);
        absmax = batch_ptr<float>(q.absmax, b);
        diag = has_ptr(q.diag) ? batch_ptr<float>(q.diag, b) : nullptr;
        order = q.order; shift = q.bs_shift; per_row = q.order >> q.bs_shift;
        first_row = row0;
        on_diagonal = false;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            int tr, tc;
            locate(g, tr, tc);
            // matrix row / first column of the group at k0 = 0
            const int mr = ALONG_K ? min(row0 + tr, order - 1) : tr;
            const int mc = ALONG_K ? tc : min(row0 + tc, order - 8);
            const int k = mr * order + mc;                   // below 2^31: checked on the host
            code_off[g] = BITS == 4 ? k >> 1 : k;
            amax_off[g] = mr * per_row + (mc >> shift);
            d0[g] = mr - mc;
            drow[g] = mr;
            if (ALONG_K) dval[g] = diag != nullptr ? gload(diag + mr) : 0.0f;
        }
    }
    __device__ __forceinline__ void fetch(int k0) {
        // uniform parts of the addresses for this tile
        const long long step = ALONG_K ? k0 : (long long)k0 * order;
        const uint8_t *c = codes + (BITS == 4 ? step >> 1 : step);
        const float *a = absmax + (ALONG_K ? k0 >> shift : k0 * per_row);
        // the tile spans BK of one index and ROWS of the other: only the few tiles that cross the diagonal
        // need the exact diagonal entries
        on_diagonal = diag != nullptr && k0 + BK > first_row && k0 < first_row + ROWS;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            if (!active(g)) continue;
            amax[g] = gload(a + amax_off[g]);
            if (BITS == 4) raw[g].x = gload_u32(c + code_off[g]);
            else raw[g] = gload_u32x2(c + code_off[g]);
            if (!on_diagonal) continue;
            if (ALONG_K) {
                dpos[g] = d0[g] - k0;
            } else {
                dpos[g] = d0[g] + k0;
                dval[g] = gload(diag + min(drow[g] + k0, order - 1));
            }
        }
    }
    __device__ __forceinline__ void expand(int g, const float *s_code, float v[8]) const {
        uint32_t id[8];
        if (BITS == 4) {
            const uint32_t w = raw[g].x;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t byte = (w >> (8 * e)) & 255u;
                id[2 * e] = byte >> 4;
                id[2 * e + 1] = byte & 15u;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) { id[e] = (raw[g].x >> (8 * e)) & 255u; id[4 + e] = (raw[g].y >> (8 * e)) & 255u; }
        }
        // (a zero maximum gives +-0 here where the dequantizer writes +0: the same contribution to a product)
        const float a = amax[g];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = s_code[id[e]] * a;
        if (on_diagonal) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = e == dpos[g] ? dval[g] : v[e];
        }
    }
    __device__ __forceinline__ void commit(float *lds, const float *s_code) const {
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            if (!active(g)) continue;
            int tr, tc;
            locate(g, tr, tc);
            float v[8];
            expand(g, s_code, v);
            constexpr int LD = ALONG_K ? LDK : ROWS + LDS_PAD;
            float4 *d = reinterpret_cast<float4 *>(lds + tr * LD + tc);
            d[0] = make_float4(v[0], v[1], v[2], v[3]);
            d[1] = make_float4(v[4], v[5], v[6], v[7]);
        }
    }
    // Split pipe.  Left factor: a group is 8 consecutive k of one tile row, which is what a lane's fragment reads.
    // Right factor (TURNED): a group is 8 consecutive tile rows at one k; the 8 lanes of a group write their 8 x 8 square
    // into the wave's own part of the operand (64 tile rows of one half of k: 1 KiB in each of the three planes, used
    // as fp32 scratch first), read it back the other way round, and only then split and store: all inside the wave.
    __device__ __forceinline__ void commit_split(unsigned char *operand, const float *s_code) {
        static_assert(ALONG_K || TURNED, "the right factor's groups must be turned");
        static_assert(GROUPS == 1, "one group per thread");
        if (!active(0)) return;                               // whole waves
        int tr, tc;
        locate(0, tr, tc);
        float v[8];
        expand(0, s_code, v);
        if constexpr (ALONG_K) {
            commit_split_eight<ROWS>(operand, tr, tc >> 3, v);
        } else {
            stage_values(operand, v);
            turn(operand);
            finish(operand);
        }
    }
    // The three phases of the turned commit, so that the caller can put matrix instructions between them (each phase
    // starts by waiting for the LDS traffic of the one before): stage = expand and write the 8 x 8 squares, turn = read
    // them back the other way round, finish = split and store.
    float turned[8];
    __device__ __forceinline__ float *scratch_word(unsigned char *operand, int i) const {
        using L = SplitLayout<ROWS>;
        const int wave = threadIdx.x >> 6;
        unsigned char *mine = operand + (wave & 1) * L::kHalf + 64 * (wave >> 1) * 16;
        return reinterpret_cast<float *>(mine + (i >> 8) * L::kPlane) + (i & 255);
    }
    __device__ __forceinline__ void stage_values(unsigned char *operand, const float v[8]) const {
        const int lane = threadIdx.x & 63, kk = lane & 7, gg = (lane >> 3) & 7;
#pragma unroll
        for (int e = 0; e < 8; ++e) *scratch_word(operand, 72 * gg + 8 * e + kk) = v[e];   // [group][tile row][k], groups 72 words apart
    }
    __device__ __forceinline__ void stage(unsigned char *operand, const float *s_code) const {
        if (!active(0)) return;
        float v[8];
        expand(0, s_code, v);
        stage_values(operand, v);
    }
    __device__ __forceinline__ void turn(unsigned char *operand) {
        if (!active(0)) return;
        const int lane = threadIdx.x & 63, kk = lane & 7, gg = (lane >> 3) & 7;
        wave_lds_sync();
        const float4 lo = *reinterpret_cast<const float4 *>(scratch_word(operand, 72 * gg + 8 * kk));
        const float4 hi = *reinterpret_cast<const float4 *>(scratch_word(operand, 72 * gg + 8 * kk + 4));
        turned[0] = lo.x; turned[1] = lo.y; turned[2] = lo.z; turned[3] = lo.w;
        turned[4] = hi.x; turned[5] = hi.y; turned[6] = hi.z; turned[7] = hi.w;                // tile row 8 gg + kk of the wave's 64, its 8 k
    }
    __device__ __forceinline__ void finish(unsigned char *operand) const {
        if (!active(0)) return;
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, kk = lane & 7, gg = (lane >> 3) & 7;
        wave_lds_sync();
        commit_split_eight<ROWS>(operand, 64 * (wave >> 1) + 8 * gg + kk, wave & 1, turned);
    }
};

template <int BM, int BN, int KA, int KB, int EPI, int PREC>
constexpr int kWavesPerSimd = (PREC == kPipeSplit && BM == 128 && BN == 128 &&
                               (KA >= kQuant4 || KB >= kQuant4 || EPI == kRequant8)) ? 2 : 3;   // (the 256-entry tables of the 8-bit re-encoding leave LDS for two)

template <int BM, int BN, int KA, int KB, int EPI, int PREC = kPipeF32>
__global__ __launch_bounds__(256, (kWavesPerSimd<BM, BN, KA, KB, EPI, PREC>)) void gemm_kernel(const GemmArgs args) {   // three waves per SIMD mean at most 168 registers, two 256
    constexpr int WM = BM / 2, WN = BN / 2, MI = WM / 32, NI = WN / 32;
    // Workgroups are dealt round-robin to the 8 accelerator dies, each with its own L2.  Renumber
    // them so that every die works through one contiguous run of (batch entry, tile row, tile
    // column): the tiles that share operand panels then share an L2 as well.
    const int tiles_n = (args.N + BN - 1) / BN, tiles_m = (args.M + BM - 1) / BM;
    const uint32_t total = gridDim.x;
    const uint32_t die = blockIdx.x % kDies, slot = blockIdx.x / kDies;
    const uint32_t per = total / kDies, extra = total % kDies;
    uint32_t id = die * per + min(die, extra) + slot;
    // Plain-store products with few output tiles and a long k range run in one of two ways that cut k:
    // equal slices per output tile (split_k), or runs of stream_per k tiles dealt out over the k tiles of all
    // output tiles laid end to end (every workgroup the same share of the arithmetic, whatever the number of
    // tiles).  Either way a part of a tile's k range goes to the workspace and a second kernel adds the parts
    // of a tile in order.
    // (only built into the products with a quantized operand: the loop around the tile costs the plain
    // products of the big stacks, which never need it, a percent)
    constexpr bool kCanStream = QT_STREAMK && EPI == kStore && (KA >= kQuant4 || KB >= kQuant4);
    const bool streamed = kCanStream && args.stream_per > 0;
    const int k_tiles_all = args.K / BK;                 // (only used when streamed: K is then a multiple of BK)
    long long run_at = 0, run_end = 0;                   // streamed: this workgroup's run of k tiles, [run_at, run_end)
    if (streamed) {
        run_at = (long long)id * args.stream_per;
        run_end = min(run_at + args.stream_per, (long long)tiles_m * tiles_n * args.batch_count * k_tiles_all);
        if (run_at >= run_end) return;
    }
    const int slices = EPI == kStore && !streamed ? args.split_k : 1;
    const int slice = id % slices;
    id /= slices;
    constexpr bool kSplit = PREC == kPipeSplit;

    using PlainA = typename std::conditional<KA == kDense, LoadKContig<BM>,
        typename std::conditional<KA == kDenseT, LoadRowContig<BM>,
            LoadQuant<BM, KA == kQuant4 ? 4 : 8, true>>::type>::type;
    using PlainB = typename std::conditional<KB == kDense, LoadRowContig<BN>,
        typename std::conditional<KB == kDenseT, LoadKContig<BN>,
            LoadQuant<BN, KB == kQuant4 ? 4 : 8, false>>::type>::type;
    using LoaderA = typename std::conditional<!kSplit || KA >= kQuant4, PlainA,
        typename std::conditional<KA == kDense, SplitKContig<BM>, SplitRowContig<BM>>::type>::type;
    using LoaderB = typename std::conditional<!kSplit, PlainB,
        typename std::conditional<KB >= kQuant4, LoadQuant<BN, KB == kQuant4 ? 4 : 8, false, true>,
            typename std::conditional<KB == kDense, SplitRowContig<BN>, SplitKContig<BN>>::type>::type>::type;
    // An operand whose k is contiguous at the source sits in LDS as [row][k] (16-byte commits, one
    // 16-byte fragment read per four MFMA steps); the others as [k][row] (16-byte commits, one word
    // per step).  Which k a lane feeds into which step is free as long as both operands agree:
    // step s of a tile takes k = 8 (s / 4) + 4 (lane / 32) + s % 4.
    constexpr bool A_RM = PlainA::kRowMajor, B_RM = PlainB::kRowMajor;
    constexpr int LDA = BM + LDS_PAD, LDB = BN + LDS_PAD;
    constexpr int SIZE_A = A_RM ? BM * LDK : BK * LDA, SIZE_B = B_RM ? BN * LDK : BK * LDB;
    // one buffer: the two stages of both operand tiles during the main loop, then (symmetric products)
    // a 32 x 32 staging square per wave that turns accumulator blocks around for the mirrored stores
    constexpr bool kRequant = EPI == kRequant4 || EPI == kRequant8;
    constexpr int SPLIT_A = SplitLayout<BM>::kOperand, SPLIT_STAGE = SPLIT_A + SplitLayout<BN>::kOperand;     // bytes
    constexpr int STAGE_LD = 36, REQUANT_LD = 68, SIZE_MAIN = kSplit ? 2 * SPLIT_STAGE / 4 : 2 * SIZE_A + 2 * SIZE_B;
    constexpr int SIZE_STAGE = kRequant ? 4 * 32 * REQUANT_LD : 4 * 32 * STAGE_LD;
    __shared__ __attribute__((aligned(16))) float s_mem[SIZE_MAIN > SIZE_STAGE ? SIZE_MAIN : SIZE_STAGE];
    float (*s_a)[SIZE_A] = reinterpret_cast<float (*)[SIZE_A]>(s_mem);
    float (*s_b)[SIZE_B] = reinterpret_cast<float (*)[SIZE_B]>(s_mem + 2 * SIZE_A);
    __shared__ float s_code[256];
    constexpr bool kNeedCode = KA >= kQuant4 || KB >= kQuant4 || EPI == kAxpbyQuant4 || EPI == kAxpbyQuant8 || kRequant;
    // a requantizing epilogue searches the table like the quantizer does: thresholds per workgroup
    constexpr int RCODE = EPI == kRequant8 ? 256 : 16;
    __shared__ CodeTables<kRequant ? RCODE : 1> tab;
    if constexpr (kRequant) build_code_tables<RCODE>(args.code, tab, nullptr);
    if (kNeedCode) {
        constexpr int NCODE = (KA == kQuant8 || KB == kQuant8 || EPI == kAxpbyQuant8 || EPI == kRequant8) ? 256 : 16;
        if ((int)threadIdx.x < NCODE) s_code[threadIdx.x] = args.code[threadIdx.x];
        __syncthreads();
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

  for (;;) {                                   // one pass, or one per piece of this workgroup's run when streamed
    int tile_m, tile_n, b;
    int seg_first = 0, seg_tiles = 0;          // streamed: first k tile and number of k tiles of this piece
    long long seg_slot = -1;                   // streamed: workspace slot of a piece that is not a whole tile
    uint32_t tile_id = id;
    if (streamed) {
        const long long t = run_at / k_tiles_all;
        seg_first = (int)(run_at - t * k_tiles_all);
        seg_tiles = (int)min((long long)(k_tiles_all - seg_first), run_end - run_at);
        tile_id = (uint32_t)t;
        // pieces are numbered in the order of their first k tile: one starts at every multiple of stream_per
        // and at every multiple of the k tiles per output tile
        if (seg_tiles != k_tiles_all) seg_slot = run_at / args.stream_per + t - run_at / args.stream_lcm;
    }
    if (args.symmetric) {                  // row-major walk over the tiles on and above the diagonal
        const uint32_t upper = (uint32_t)tiles_n * (tiles_n + 1) / 2;
        b = tile_id / upper;
        uint32_t rest = tile_id % upper, width = tiles_n;
        tile_m = 0;
        while (rest >= width) { rest -= width; --width; ++tile_m; }
        tile_n = tile_m + rest;
    } else {
        tile_n = tile_id % tiles_n;
        tile_id /= tiles_n;
        tile_m = tile_id % tiles_m;
        b = tile_id / tiles_m;
    }
    if (args.skip != nullptr && args.skip[b] != 0) return;       // (never set together with `streamed`)
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const float *A = (KA < kQuant4) ? dense_ptr(args.A, b, args.batch_inner, args.inner_a) : nullptr;
    const float *B = (KB < kQuant4) ? dense_ptr(args.B, b, args.batch_inner, args.inner_b) : nullptr;
    if constexpr (kSplit) {                    // the same for the whole workgroup: say so, the loads take them from scalar registers
        A = wave_uniform(A);
        B = wave_uniform(B);
    }
    const bool a_vec = KA < kQuant4 && (args.lda & 3) == 0 && is_aligned16(A);
    const bool b_vec = KB < kQuant4 && (args.ldb & 3) == 0 && is_aligned16(B);

    LoaderA la;
    LoaderB lb;

    // whole k tiles, aligned rows, extents that keep a clamped 16-byte load inside the matrix and
    // offsets inside 31 bits: the loads of the main loop then need no predicates at all
    const bool whole_k = args.K % BK == 0;
    bool a_fast = false, b_fast = false;
    if constexpr (kSplit) {                    // the host only picks this pipe where the fast loads apply
        if constexpr (KA >= kQuant4) la.prepare(args.Aq, b, m0);
        else la.prepare(args.lda, m0, args.M);
        if constexpr (KB >= kQuant4) lb.prepare(args.Bq, b, n0);
        else lb.prepare(args.ldb, n0, args.N);
        if constexpr (KA == kDense) la.vec = a_vec;
        if constexpr (KB == kDenseT) lb.vec = b_vec;
    } else {
        if constexpr (KA < kQuant4) {
            a_fast = whole_k && a_vec && (KA == kDense || (args.M & 3) == 0) &&
                     (long long)(KA == kDense ? args.M : args.K) * args.lda < 0x7fffffffLL;
            if (a_fast) la.prepare(args.lda, m0, args.M);
        }
        if constexpr (KB < kQuant4) {
            b_fast = whole_k && b_vec && (KB == kDenseT || (args.N & 3) == 0) &&
                     (long long)(KB == kDenseT ? args.N : args.K) * args.ldb < 0x7fffffffLL;
            if (b_fast) lb.prepare(args.ldb, n0, args.N);
        }
        if constexpr (KA >= kQuant4) la.prepare(args.Aq, b, m0);
        if constexpr (KB >= kQuant4) lb.prepare(args.Bq, b, n0);
    }
    auto fetch = [&](int k0) {
        if constexpr (kSplit) {
            if constexpr (KA >= kQuant4) la.fetch(k0);
            else la.fetch_fast(A + (KA == kDense ? (long long)k0 : (long long)k0 * args.lda));
            if constexpr (KB >= kQuant4) lb.fetch(k0);
            else lb.fetch_fast(B + (KB == kDenseT ? (long long)k0 : (long long)k0 * args.ldb));
        } else {
            if constexpr (KA < kQuant4) {
                if (a_fast) la.fetch_fast(A + (KA == kDense ? (long long)k0 : (long long)k0 * args.lda));
                else la.fetch(A, args.lda, m0, k0, args.M, args.K, a_vec);
            } else la.fetch(k0);
            if constexpr (KB < kQuant4) {
                if (b_fast) lb.fetch_fast(B + (KB == kDenseT ? (long long)k0 : (long long)k0 * args.ldb));
                else lb.fetch(B, args.ldb, n0, k0, args.N, args.K, b_vec);
            } else lb.fetch(k0);
        }
    };
    auto commit = [&](int stage, bool right_in_phases = false) {
        if constexpr (kSplit) {
            unsigned char *at = reinterpret_cast<unsigned char *>(s_mem) + stage * SPLIT_STAGE;
            if constexpr (KA >= kQuant4) la.commit_split(at, s_code);
            else la.commit_split(at);
            if constexpr (KB >= kQuant4) { if (!right_in_phases) lb.commit_split(at + SPLIT_A, s_code); }
            else lb.commit_split(at + SPLIT_A);
        } else {
            la.commit(s_a[stage], s_code);
            lb.commit(s_b[stage], s_code);
        }
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // Pipeline: tile t is multiplied out of one LDS buffer while tile t+1 (already in registers,
    // its loads were issued a whole tile earlier) is written to the other buffer half-way through
    // the MFMA stream and the loads of tile t+2 are issued right after.  One barrier per tile.
    // (with k split into slices -- the host makes them equal -- this workgroup owns one of them)
    // (a triangular operand shortens the range to where it is not zero: tile origins are multiples of BK)
    const int k_first = (args.triangular & 1) ? min(m0, args.K) : 0;
    const int k_last = (args.triangular & 2) ? min(n0 + BN, args.K) : args.K;
    const int n_tiles = streamed ? seg_tiles : max((k_last - k_first + BK - 1) / BK, 1) / slices;
    const int k_begin = streamed ? seg_first * BK : k_first + slice * n_tiles * BK;
    fetch(k_begin);
    commit(0);
    if (n_tiles > 1) fetch(k_begin + BK);
    __syncthreads();
    const int frag_row = lane & 31, half = lane >> 5;
    constexpr int STEPS = BK / 2;
    if constexpr (kSplit) {
        using LA = SplitLayout<BM>;
        using LB = SplitLayout<BN>;
        // products in the order of their size, smallest first: (h, l), (l, h), (m, m), (h, m), (m, h), (h, h)
        constexpr int pa_of[6] = {0, 2, 1, 0, 1, 0}, pb_of[6] = {2, 0, 1, 1, 0, 0};
        for (int t = 0; t < n_tiles; ++t) {
            const int cur = t & 1;
            const unsigned char *sa = reinterpret_cast<const unsigned char *>(s_mem) + cur * SPLIT_STAGE + half * LA::kHalf + (wm + frag_row) * 16;
            const unsigned char *sb = reinterpret_cast<const unsigned char *>(s_mem) + cur * SPLIT_STAGE + SPLIT_A + half * LB::kHalf + (wn + frag_row) * 16;
            qt_bf16x8 fa[3][MI], fb[3][NI];
#pragma unroll
            for (int p = 0; p < 3; ++p) {
#pragma unroll
                for (int i = 0; i < MI; ++i) fa[p][i] = *reinterpret_cast<const qt_bf16x8 *>(sa + p * LA::kPlane + i * 32 * 16);
#pragma unroll
                for (int j = 0; j < NI; ++j) fb[p][j] = *reinterpret_cast<const qt_bf16x8 *>(sb + p * LB::kPlane + j * 32 * 16);
            }
#pragma unroll
            for (int q = 0; q < 6; ++q) {
                if constexpr (KB >= kQuant4) {        // the turned commit of the right factor, spread over the products
                    unsigned char *next_b = reinterpret_cast<unsigned char *>(s_mem) + (cur ^ 1) * SPLIT_STAGE + SPLIT_A;
                    if (t + 1 < n_tiles) {
                        if (q == 1) lb.stage(next_b, s_code);
                        if (q == 2) lb.turn(next_b);
                        if (q == 4) lb.finish(next_b);
                    }
                }
                if constexpr (KA < kQuant4 && KB < kQuant4) {
                    // dense operands: the split of the next tile in two halves between the product groups (A, then B),
                    // each followed by its loads of the tile after
                    unsigned char *next = reinterpret_cast<unsigned char *>(s_mem) + (cur ^ 1) * SPLIT_STAGE;
                    if (q == 2 && t + 1 < n_tiles) {
                        la.commit_split(next);
                        if (t + 2 < n_tiles) la.fetch_fast(A + (KA == kDense ? (long long)(k_begin + (t + 2) * BK) : (long long)(k_begin + (t + 2) * BK) * args.lda));
                    }
                    if (q == 4 && t + 1 < n_tiles) {
                        lb.commit_split(next + SPLIT_A);
                        if (t + 2 < n_tiles) lb.fetch_fast(B + (KB == kDenseT ? (long long)(k_begin + (t + 2) * BK) : (long long)(k_begin + (t + 2) * BK) * args.ldb));
                    }
                } else if (q == 3 && t + 1 < n_tiles) {
                    commit(cur ^ 1, true);
                    if (t + 2 < n_tiles) fetch(k_begin + (t + 2) * BK);
                }
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[pa_of[q]][i], fb[pb_of[q]][j], acc[i][j], 0, 0, 0);
            }
            __syncthreads();
        }
    } else
    for (int t = 0; t < n_tiles; ++t) {
        const int cur = t & 1;
        const float *pa = s_a[cur] + (A_RM ? (wm + frag_row) * LDK + 4 * half : 4 * half * LDA + wm + frag_row);
        const float *pb = s_b[cur] + (B_RM ? (wn + frag_row) * LDK + 4 * half : 4 * half * LDB + wn + frag_row);
        // fragments are read from LDS ahead of the MFMAs that use them: the next step's words for a
        // [k][row] operand, the next group of four steps for a [row][k] operand
        float fa[2][MI], fb[2][NI];
        qt_f32x4 qa[2][MI], qb[2][NI];
        auto load_a = [&](int step) {
            if constexpr (A_RM) {
                if (step % 4 == 0)
#pragma unroll
                    for (int i = 0; i < MI; ++i)
                        qa[(step / 4) & 1][i] = *reinterpret_cast<const qt_f32x4 *>(pa + i * 32 * LDK + 8 * (step / 4));
            } else {
#pragma unroll
                for (int i = 0; i < MI; ++i) fa[step & 1][i] = pa[i * 32 + (8 * (step / 4) + step % 4) * LDA];
            }
        };
        auto load_b = [&](int step) {
            if constexpr (B_RM) {
                if (step % 4 == 0)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        qb[(step / 4) & 1][j] = *reinterpret_cast<const qt_f32x4 *>(pb + j * 32 * LDK + 8 * (step / 4));
            } else {
#pragma unroll
                for (int j = 0; j < NI; ++j) fb[step & 1][j] = pb[j * 32 + (8 * (step / 4) + step % 4) * LDB];
            }
        };
        load_a(0);
        load_b(0);
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            // [row][k] operands fetch a whole group ahead (at the first step of the previous group)
            if (A_RM && s % 4 == 0 && s + 4 < STEPS) load_a(s + 4);
            if (B_RM && s % 4 == 0 && s + 4 < STEPS) load_b(s + 4);
            if (!A_RM && s + 1 < STEPS) load_a(s + 1);
            if (!B_RM && s + 1 < STEPS) load_b(s + 1);
            if (s == STEPS / 2 && t + 1 < n_tiles) {
                commit(cur ^ 1);
                if (t + 2 < n_tiles) fetch(k_begin + (t + 2) * BK);
            }
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const float av = A_RM ? qa[(s / 4) & 1][i][s % 4] : fa[s & 1][i];
                    const float bv = B_RM ? qb[(s / 4) & 1][j][s % 4] : fb[s & 1][j];
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                }
        }
        __syncthreads();
    }

    // Split pipe, diagonal tile of a symmetric product: a b and b a add the pieces of a product in different orders,
    // so an element below the diagonal that is multiplied out differs in its last bits from the mirror image of
    // its partner above -- and which of the two a tile shape produces depends on the shape.  Every element below
    // the diagonal therefore takes the value of its partner above, here as in the mirrored tiles: the result is
    // exactly symmetric and does not depend on the tiling.  (On the fp32 pipe the products of G G^T commute.)
    if constexpr (kSplit && BM == BN) {
        if (args.symmetric && tile_m == tile_n) {
            constexpr int XLD = WN + 1;
            float *X = s_mem;                                   // one quadrant (WM x WN) at a time; the operand tiles are done with
            auto put = [&](bool turned) {
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int lr = i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, lc = j * 32 + (lane & 31);
                            X[turned ? lc * XLD + lr : lr * XLD + lc] = acc[i][j][r];
                        }
            };
            if (wm < wn) put(true);                             // the quadrant above the diagonal, turned around ...
            __syncthreads();
            if (wm > wn) {                                      // ... is the one below
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int lr = i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, lc = j * 32 + (lane & 31);
                            acc[i][j][r] = X[lr * XLD + lc];
                        }
            }
            __syncthreads();
#pragma unroll
            for (int w = 0; w < 2; ++w) {                       // the two quadrants on the diagonal, one after the other
                if (wm == wn && (wm != 0) == (w == 1)) {
                    put(false);
                    wave_lds_sync();
#pragma unroll
                    for (int i = 0; i < MI; ++i)
#pragma unroll
                        for (int j = 0; j < NI; ++j)
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int lr = i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, lc = j * 32 + (lane & 31);
                                if (lr > lc) acc[i][j][r] = X[lc * XLD + lr];
                            }
                }
                __syncthreads();
            }
        }
    }

    // ---- epilogue
    float *C = const_cast<float *>(dense_ptr(args.C, b, args.batch_inner, args.inner_c));
    int ldc = args.ldc;
    if (slices > 1) {                              // partial product of this slice: summed by reduce_slices_kernel
        C = args.workspace + ((long long)b * slices + slice) * args.M * args.N;
        ldc = args.N;
    }
    if (seg_slot >= 0) {                           // a piece of a tile: kept as a BM x BN square, summed by reduce_pieces_kernel
        C = args.workspace + seg_slot * (BM * BN) - ((long long)m0 * BN + n0);
        ldc = BN;
    }
    float *T = EPI == kNewton ? const_cast<float *>(batch_ptr<float>(args.T, b)) : nullptr;
    const float *E = EPI == kAxpbyDense ? dense_ptr(args.E, b, args.batch_inner, args.inner_e) : nullptr;
    constexpr bool kQuantAddend = EPI == kAxpbyQuant4 || EPI == kAxpbyQuant8 || kRequant;
    constexpr int EBITS = (EPI == kAxpbyQuant8 || EPI == kRequant8) ? 8 : 4;
    const uint8_t *e_codes = kQuantAddend ? batch_ptr<uint8_t>(args.Eq.codes, b) : nullptr;
    const float *e_absmax = kQuantAddend ? batch_ptr<float>(args.Eq.absmax, b) : nullptr;
    const float *e_diag = kQuantAddend && has_ptr(args.Eq.diag) ? batch_ptr<float>(args.Eq.diag, b) : nullptr;
    // an off-diagonal tile of a symmetric product also provides its mirror image; the addend is
    // read at the mirrored position, so an addend that is not exactly symmetric is honoured
    const bool mirror = args.symmetric != 0 && tile_n != tile_m;
    const bool vec_ok = (ldc & 3) == 0 && is_aligned16(C) &&
                        (EPI != kNewton || ((args.ldt & 3) == 0 && is_aligned16(T))) &&
                        (EPI != kAxpbyDense || ((args.lde & 3) == 0 && is_aligned16(E)));
    const bool mirror_vec = vec_ok && (args.M & 3) == 0;
    const bool direct_vec = vec_ok && (args.N & 3) == 0;
    if constexpr (kRequant) {
        // beta * deq(E) + alpha * acc goes straight back into E's codes, maxima and exact diagonal: the fp32
        // statistic never reaches memory.  A wave's 64 x 64 quadrant holds whole segments (blocksize 64) of 64
        // rows -- and, mirrored, of 64 rows of the transposed tile -- so it encodes them alone: 32 rows at a
        // time go through its staging area, 16 lanes take one row (four consecutive elements each), and the
        // maximum, the division and the table search are those of the flat quantizer.  Each element of E is
        // read and rewritten by the same wave, all reads of a row before its writes.
        float *stage = s_mem + wave * (32 * REQUANT_LD);
        uint8_t *o_codes = const_cast<uint8_t *>(e_codes);
        float *o_absmax = const_cast<float *>(e_absmax), *o_diag = const_cast<float *>(e_diag);
        const bool fast_ok = (tab.flags & kFlagLut) != 0, ascending = (tab.flags & kFlagAscending) != 0;
        const int order = args.Eq.order, per_row = order >> 6;
        auto encode_rows = [&](int row_base, int col_base) {
            if (col_base >= order) return;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int rl = q * 4 + (lane >> 4), c4 = (lane & 15) * 4;
                const float4 a4 = *reinterpret_cast<const float4 *>(stage + rl * REQUANT_LD + c4);
                const float a[4] = {a4.x, a4.y, a4.z, a4.w};
                const int row = row_base + rl, col = col_base + c4;
                if (row >= order) continue;                      // the 16 lanes of a segment share the row
                float e[4], y[4];
                dequant_four<EBITS>(e_codes, e_absmax, s_code, order, 6, row, col, e);
                const bool on_diag = o_diag != nullptr && (unsigned)(row - col) < 4u;
                if (on_diag) {
                    const float d = gload(o_diag + row);
#pragma unroll
                    for (int k = 0; k < 4; ++k) if (row == col + k) e[k] = d;
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) y[k] = __builtin_fmaf(args.alpha, a[k], args.beta * e[k]);
                if (on_diag) {
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if (row == col + k) { gstore(o_diag + row, y[k]); y[k] = 0.0f; }
                }
                uint32_t idx[4];
                const uint32_t m = encode_four<RCODE, 16>(y, tab, fast_ok, ascending, idx);
                if ((lane & 15) == 0) gstore(o_absmax + (long long)row * per_row + (col >> 6), __uint_as_float(m));
                const long long k0 = (long long)row * order + col;
                if (EBITS == 4)
                    *(QT_GLOBAL uint16_t *)(o_codes + (k0 >> 1)) = (uint16_t)(((idx[0] << 4) | idx[1]) | (((idx[2] << 4) | idx[3]) << 8));
                else
                    *(QT_GLOBAL uint32_t *)(o_codes + k0) = idx[0] | (idx[1] << 8) | (idx[2] << 16) | (idx[3] << 24);
            }
        };
#pragma unroll
        for (int i = 0; i < MI; ++i) {
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    stage[(8 * (r / 4) + 4 * (lane >> 5) + r % 4) * REQUANT_LD + j * 32 + (lane & 31)] = acc[i][j][r];
            wave_lds_sync();
            encode_rows(m0 + wm + i * 32, n0 + wn);
            wave_lds_sync();
        }
        if (mirror) {
#pragma unroll
            for (int j = 0; j < NI; ++j) {
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        stage[(lane & 31) * REQUANT_LD + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4] = acc[i][j][r];
                wave_lds_sync();
                encode_rows(n0 + wn + j * 32, m0 + wm);
                wave_lds_sync();
            }
        }
        return;
    }
    float local_err = 0.0f;
    // Each wave passes its accumulator blocks (32 x 32) through a staging square of its own in LDS, so that a
    // lane ends up with four consecutive elements of one output row: 16-byte stores, eight lanes per 128-byte
    // line, and one packed load per four elements of a quantized addend.
    float *stage = s_mem + wave * (32 * STAGE_LD);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            if (direct_vec) {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    stage[(8 * (r / 4) + 4 * (lane >> 5) + r % 4) * STAGE_LD + (lane & 31)] = acc[i][j][r];
                wave_lds_sync();
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const int ml = p * 8 + (lane >> 3), nl = (lane & 7) * 4;
                    const float4 a4 = *reinterpret_cast<const float4 *>(stage + ml * STAGE_LD + nl);
                    float y[4] = {a4.x, a4.y, a4.z, a4.w};
                    const int row = m0 + wm + i * 32 + ml, col4 = n0 + wn + j * 32 + nl;
                    if (row >= args.M || col4 >= args.N) continue;           // N % 4 == 0: col4 + 3 < N
                    if (EPI == kAxpbyDense) {
                        const float4 x = gload4(E + (long long)row * args.lde + col4);
                        const float e[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) y[q] = args.beta * e[q] + args.alpha * y[q];
                    } else if (kQuantAddend) {
                        float e[4];
                        dequant_four<EBITS>(e_codes, e_absmax, s_code, args.Eq.order, args.Eq.bs_shift, row, col4, e);
                        if (e_diag != nullptr && (unsigned)(row - col4) < 4u) {
                            const float d = gload(e_diag + row);
#pragma unroll
                            for (int q = 0; q < 4; ++q) if (row == col4 + q) e[q] = d;
                        }
                        // same two roundings as tensor.mul_(beta).add_(S, alpha=1-beta)
#pragma unroll
                        for (int q = 0; q < 4; ++q) y[q] = __builtin_fmaf(args.alpha, y[q], args.beta * e[q]);
                    } else if (EPI == kNewton) {
                        float t[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float eye = row == col4 + q ? 1.0f : 0.0f;
                            local_err = fmaxf(local_err, fabsf(y[q] - eye));
                            t[q] = (1.0f - args.newton_w) * eye + args.newton_w * y[q];
                        }
                        gstore4(T + (long long)row * args.ldt + col4, t);
                    }
                    gstore4(C + (long long)row * ldc + col4, y);
                }
                wave_lds_sync();
            } else {
                // accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the block
                const int col = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4;
                    if (row >= args.M || col >= args.N) continue;
                    float y = acc[i][j][r];
                    if (EPI == kAxpbyDense) {
                        y = args.beta * gload(E + (long long)row * args.lde + col) + args.alpha * y;
                    } else if (kQuantAddend) {
                        const float e = dequant_element<EBITS>(e_codes, e_absmax, e_diag, s_code, args.Eq.order,
                                                               args.Eq.bs_shift, row, col);
                        y = __builtin_fmaf(args.alpha, y, args.beta * e);
                    } else if (EPI == kNewton) {
                        const float eye = row == col ? 1.0f : 0.0f;
                        local_err = fmaxf(local_err, fabsf(y - eye));
                        gstore(T + (long long)row * args.ldt + col, (1.0f - args.newton_w) * eye + args.newton_w * y);
                    }
                    gstore(C + (long long)row * ldc + col, y);
                }
            }
            if (!mirror) continue;
            // The mirror image of the block: staged as [column][row], read back as 16 bytes along the row
            // index, stored as 128-byte runs of the mirrored rows.
#pragma unroll
            for (int r = 0; r < 16; ++r)
                stage[(lane & 31) * STAGE_LD + 8 * (r / 4) + 4 * (lane >> 5) + r % 4] = acc[i][j][r];
            wave_lds_sync();
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int nl = p * 8 + (lane >> 3), ml = (lane & 7) * 4;
                const float4 a4 = *reinterpret_cast<const float4 *>(stage + nl * STAGE_LD + ml);
                const float a[4] = {a4.x, a4.y, a4.z, a4.w};
                const int mrow = n0 + wn + j * 32 + nl;         // row of the mirrored elements (a column of the tile)
                const int mcol = m0 + wm + i * 32 + ml;         // their first column (a row of the tile)
                if (mrow >= args.N || mcol >= args.M) continue;
                // elements (mrow, mcol .. mcol+3), never on the diagonal
                float y[4], e[4] = {0.f, 0.f, 0.f, 0.f};
                const bool whole = mirror_vec;                  // M % 4 == 0: mcol + 3 < M
                if (EPI == kAxpbyDense) {
                    if (whole) { const float4 x = gload4(E + (long long)mrow * args.lde + mcol); e[0] = x.x; e[1] = x.y; e[2] = x.z; e[3] = x.w; }
                    else
#pragma unroll
                        for (int q = 0; q < 4; ++q) if (mcol + q < args.M) e[q] = gload(E + (long long)mrow * args.lde + mcol + q);
                } else if (kQuantAddend) {
                    // flat quantized layout: the order is a multiple of 64, so the four codes share a segment
                    dequant_four<EBITS>(e_codes, e_absmax, s_code, args.Eq.order, args.Eq.bs_shift, mrow, mcol, e);
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (EPI == kAxpbyDense) y[q] = args.beta * e[q] + args.alpha * a[q];
                    else if (kQuantAddend) y[q] = __builtin_fmaf(args.alpha, a[q], args.beta * e[q]);
                    else y[q] = a[q];
                }
                float *cm = C + (long long)mrow * ldc + mcol;
                if (whole) gstore4(cm, y);
                else
#pragma unroll
                    for (int q = 0; q < 4; ++q) if (mcol + q < args.M) gstore(cm + q, y[q]);
                if (EPI == kNewton) {
                    float t[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) t[q] = args.newton_w * y[q];
                    float *tm = T + (long long)mrow * args.ldt + mcol;
                    if (whole) gstore4(tm, t);
                    else
#pragma unroll
                        for (int q = 0; q < 4; ++q) if (mcol + q < args.M) gstore(tm + q, t[q]);
                }
            }
            wave_lds_sync();
        }
    if (EPI == kNewton) {
        uint32_t e = group_max_u32<64>(__float_as_uint(local_err));   // non-negative floats order like their bits
        if (lane == 0) atomicMax(reinterpret_cast<unsigned int *>(args.err) + b, e);
    }
    if (!streamed) return;
    run_at += seg_tiles;
    if (run_at >= run_end) return;
    __syncthreads();                               // the staging squares of the epilogue overlap the operand tiles
  }
}

// What the matrix pipes sustain with nothing else going on: every wave multiplies register operands of pseudo-random
// bits (the power a pipe draws, and with it the clock it holds, depends on how many bits toggle) into four accumulator
// blocks, 24 bf16 instructions (32x32x16) or 32 fp32 instructions (32x32x2) per round.  A yardstick for the rates of the
// product kernels beside the published peaks.
template <int PIPE>
__global__ __launch_bounds__(256) void mfma_rate_kernel(float *sink, int rounds) {
    f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    auto noise = [&](uint32_t q) {                          // in (-0.5, 0.5), different per lane, register and block
        uint32_t h = (threadIdx.x * 2654435761u) ^ (q * 40503u + blockIdx.x * 7919u);
        h ^= h >> 13; h *= 0x5bd1e995u; h ^= h >> 15;
        return (float)(int)(h & 0xffffu) / 65536.0f - 0.5f;
    };
    if constexpr (PIPE == kPipeSplit) {
        qt_bf16x8 a[6], b[6];
#pragma unroll
        for (int q = 0; q < 6; ++q)
#pragma unroll
            for (int e = 0; e < 8; ++e) { a[q][e] = (__bf16)noise(16 * q + e); b[q][e] = (__bf16)noise(16 * q + 8 + e); }
        for (int it = 0; it < rounds; ++it)
#pragma unroll
            for (int q = 0; q < 6; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[q], b[(q + i) % 6], acc[i], 0, 0, 0);
    } else {
        float a[8], b[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) { a[q] = noise(2 * q); b[q] = noise(2 * q + 1); }
        for (int it = 0; it < rounds; ++it)
#pragma unroll
            for (int q = 0; q < 8; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q], b[(q + i) % 8], acc[i], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    if (s == 12345.678f) sink[0] = s;                       // keeps the products alive; practically never taken
}

// Streamed products: out tile = sum of its pieces in the workspace, in the order of their k ranges.  A tile that
// one workgroup did as a whole is already in place.  Grid (tiles, 4 row bands of the tile).
__global__ __launch_bounds__(256) void reduce_pieces_kernel(const float *workspace, BatchPtr C, int ldc, int M, int N, int bm, int bn,
                                                            int tiles_m, int tiles_n, int k_tiles, int stream_per, int stream_lcm) {
    uint32_t t = blockIdx.x;
    const long long first = (long long)t * k_tiles, next = first + k_tiles;
    const long long s0 = first / stream_per + first / k_tiles - first / stream_lcm;
    const long long s1 = next / stream_per + next / k_tiles - next / stream_lcm;
    if (s1 - s0 <= 1) return;
    const int tile_n = t % tiles_n;
    t /= tiles_n;
    const int tile_m = t % tiles_m, b = t / tiles_m;
    float *out = const_cast<float *>(batch_ptr<float>(C, b));
    const int m0 = tile_m * bm, n0 = tile_n * bn, plane = bm * bn, quads_per_row = bn >> 2;
    const bool vec = (ldc & 3) == 0 && is_aligned16(out) && (N & 3) == 0;
    const int rows = bm / 4;                           // this block's band of rows
    for (int q = threadIdx.x; q < rows * quads_per_row; q += 256) {
        const int r = blockIdx.y * rows + q / quads_per_row, c = (q % quads_per_row) << 2;
        const int row = m0 + r, col = n0 + c;
        if (row >= M || col >= N) continue;
        const float *w = workspace + s0 * plane + r * bn + c;
        float4 sum = gload4(w);
        for (long long k = 1; k < s1 - s0; ++k) {
            const float4 x = gload4(w + k * plane);
            sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
        }
        float *o = out + (long long)row * ldc + col;
        if (vec) { const float y[4] = {sum.x, sum.y, sum.z, sum.w}; gstore4(o, y); }
        else {
            gstore(o, sum.x);
            if (col + 1 < N) gstore(o + 1, sum.y);
            if (col + 2 < N) gstore(o + 2, sum.z);
            if (col + 3 < N) gstore(o + 3, sum.w);
        }
    }
}


// out[b][m][n] = sum over slices of workspace[b][slice][m][n], slices added in order
__global__ __launch_bounds__(256) void reduce_slices_kernel(const float *workspace, int slices, BatchPtr C, int ldc, int M, int N) {
    const int b = blockIdx.y;
    const long long plane = (long long)M * N;
    const float *w = workspace + (long long)b * slices * plane;
    float *out = const_cast<float *>(batch_ptr<float>(C, b));
    const bool vec = (N & 3) == 0 && (ldc & 3) == 0 && is_aligned16(out) && is_aligned16(w);
    if (vec) {
        const long long quads = plane >> 2;
        for (long long q = blockIdx.x * 256ll + threadIdx.x; q < quads; q += (long long)gridDim.x * 256) {
            const long long e = q << 2;
            float4 sum = gload4(w + e);
            for (int s = 1; s < slices; ++s) {
                const float4 x = gload4(w + s * plane + e);
                sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
            }
            const int m = (int)(e / N), n = (int)(e % N);
            float *o = out + (long long)m * ldc + n;
            gstore(o, sum.x); gstore(o + 1, sum.y); gstore(o + 2, sum.z); gstore(o + 3, sum.w);
        }
    } else {
        for (long long e = blockIdx.x * 256ll + threadIdx.x; e < plane; e += (long long)gridDim.x * 256) {
            float sum = gload(w + e);
            for (int s = 1; s < slices; ++s) sum += gload(w + s * plane + e);
            gstore(out + (e / N) * ldc + e % N, sum);
        }
    }
}

template <int BM, int BN, int KA, int KB, int EPI, int PREC = kPipeF32>
void launch_gemm(const GemmArgs &a, int batch, hipStream_t stream) {
    const long long tn = (a.N + BN - 1) / BN, tm = (a.M + BM - 1) / BM;
    if (a.symmetric && BM != BN) { set_error(kBadArgument, "gemm: symmetric products need square tiles"); return; }
    long long blocks = (a.symmetric ? tn * (tn + 1) / 2 : tn * tm) * batch * (EPI == kStore ? a.split_k : 1);
    if (EPI == kStore && a.stream_per > 0) {
        const long long runs = tn * tm * batch * (a.K / BK);
        blocks = (runs + a.stream_per - 1) / a.stream_per;
    }
    if (blocks > 0x7fffffffLL) { set_error(kBadArgument, "gemm: too many tiles (%lld)", blocks); return; }
    hipLaunchKernelGGL((gemm_kernel<BM, BN, KA, KB, EPI, PREC>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
    if (EPI == kStore && a.stream_per > 0) {
        hipLaunchKernelGGL(reduce_pieces_kernel, dim3((unsigned)(tn * tm * batch), 4), dim3(256), 0, stream, a.workspace, a.C, a.ldc,
                           a.M, a.N, BM, BN, (int)tm, (int)tn, a.K / BK, a.stream_per, a.stream_lcm);
        return;
    }
    if (EPI == kStore && a.split_k > 1) {
        const long long quads = ((long long)a.M * a.N + 1023) / 1024;
        const unsigned grid = (unsigned)(quads < 4096 ? quads : 4096);
        hipLaunchKernelGGL(reduce_slices_kernel, dim3(grid, batch), dim3(256), 0, stream, a.workspace, a.split_k, a.C, a.ldc, a.M, a.N);
    }
}

bool valid_quant(const QuantRef &q, int bits, const char *what) {
    const int bs = 1 << q.bs_shift;
    if (q.bs_shift < 6 || q.bs_shift > 11 || q.order < bs || q.order % bs != 0) {
        set_error(kBadArgument, "gemm: %s: quantized matrices need blocksize in 64..2048 dividing the order (order %d, blocksize %d)",
                  what, q.order, bs);
        return false;
    }
    if (!has_host_ptr(q.codes) || !has_host_ptr(q.absmax)) {
        set_error(kNullPointer, "gemm: %s: null codes/absmax pointer", what);
        return false;
    }
    if ((long long)q.order * q.order > 0x7fffffffLL) {
        set_error(kBadArgument, "gemm: %s: order * order must stay below 2^31 (order %d)", what, q.order);
        return false;
    }
    (void)bits;
    return true;
}

}  // namespace
}  // namespace qt

// Flat C description of one batched product (see include/qtensor_hip.h for the field meanings).
struct qtensor_gemm_desc {
    int M, N, K, batch;
    int kind_a, kind_b, epilogue;
    qt::GemmArgs args;
};

// Scratch that is part of the library image, for callers that cannot allocate (qtensor_hip_gemm_static):
// one copy per GPU, held until the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; kernels get the address that call returns.
#ifndef QTENSOR_STATIC_SCRATCH_FLOATS
#define QTENSOR_STATIC_SCRATCH_FLOATS (1 << 24)
#endif
static __device__ __align__(256) float scratch[QTENSOR_STATIC_SCRATCH_FLOATS];

namespace {
// Per GPU: the device address of `scratch` (looked up once, with that device current) and who used it last.
// All calls on a GPU share the one array, so a call on another stream than the last one is only let through when
// that last call's work has finished on the device (an event recorded behind it says so); calls on one stream are
// ordered by the stream.
struct StaticScratch {
    float *address = nullptr;
    hipEvent_t last_done = nullptr;       // recorded behind the last call's launches
    hipStream_t last_stream = nullptr;
    bool pending = false;                 // last_done has been recorded and not yet been seen complete
};
constexpr int kMaxDevices = 64;
std::mutex static_guard;
StaticScratch static_slots[kMaxDevices];

// The current device's slot, set up on first use (nullptr and the error slot on failure).  Caller holds static_guard.
StaticScratch *static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        qt::set_error(qt::kBadArgument, "gemm_static: no current device");
        return nullptr;
    }
    StaticScratch &slot = static_slots[dev];
    if (slot.address == nullptr) {
        void *p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            qt::set_error(qt::kLaunchFailed, "gemm_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        e = hipEventCreateWithFlags(&slot.last_done, hipEventDisableTiming);
        if (e != hipSuccess) {
            qt::set_error(qt::kLaunchFailed, "gemm_static: hipEventCreateWithFlags failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        slot.address = static_cast<float *>(p);
    }
    return &slot;
}

void gemm_dispatch(const qtensor_gemm_desc *d, hipStream_t stream, int tile_hint = -1);

// Process-wide choice of the matrix pipe (qtensor_hip_gemm_pipe); starts from the
// environment variable QT_GEMM_PIPE ("f32" or "split"), else the split pipe.
std::atomic<int> &pipe_mode_slot() {
    static std::atomic<int> mode{[] {
        const char *e = getenv("QT_GEMM_PIPE");
        return e != nullptr && (strcmp(e, "f32") == 0 || strcmp(e, "0") == 0) ? qt::kPipeF32 : qt::kPipeSplit;
    }()};
    return mode;
}
int gemm_pipe_mode() { return pipe_mode_slot().load(std::memory_order_relaxed); }
}  // namespace

extern "C" double qtensor_hip_mfma_rate_flop(int pipe, int rounds, int workgroups_per_unit, float *sink, void *stream_v) {
    using namespace qt;
    clear_error();
    if ((pipe != kPipeF32 && pipe != kPipeSplit) || rounds < 1 || workgroups_per_unit < 1 || workgroups_per_unit > 8 || sink == nullptr) {
        set_error(kBadArgument, "mfma_rate: pipe 0 or 1, rounds >= 1, 1..8 workgroups per unit, a device word to write to");
        return 0.0;
    }
    const unsigned grid = (unsigned)(compute_units() * workgroups_per_unit);
    if (pipe == kPipeSplit) hipLaunchKernelGGL(mfma_rate_kernel<kPipeSplit>, dim3(grid), dim3(256), 0, (hipStream_t)stream_v, sink, rounds);
    else hipLaunchKernelGGL(mfma_rate_kernel<kPipeF32>, dim3(grid), dim3(256), 0, (hipStream_t)stream_v, sink, rounds);
    // multiply-adds x 2 of one launch: 4 waves, per round 24 instructions of 32x32x16 or 32 of 32x32x2
    return (double)grid * 4.0 * rounds * (pipe == kPipeSplit ? 24.0 * 32768.0 : 32.0 * 4096.0);
}

extern "C" int qtensor_hip_gemm_pipe(int mode) {
    qt::clear_error();
    if (mode < 0) return gemm_pipe_mode();
    if (mode != qt::kPipeF32 && mode != qt::kPipeSplit) {
        qt::set_error(qt::kBadArgument, "gemm_pipe: mode must be 0 (fp32 pipe), 1 (split bf16 pipe) or negative (query), got %d", mode);
        return gemm_pipe_mode();
    }
    return pipe_mode_slot().exchange(mode, std::memory_order_relaxed);
}

extern "C" void qtensor_hip_gemm(const qtensor_gemm_desc *d, void *stream_v) {
    qt::clear_error();
    gemm_dispatch(d, (hipStream_t)stream_v);
}

extern "C" void qtensor_hip_gemm_static(const qtensor_gemm_desc *d, void *stream_v) {
    using namespace qt;
    clear_error();
    if (!d) { set_error(kNullPointer, "gemm_static: null descriptor"); return; }
    if (d->M < 1 || d->N < 1 || d->K < 1 || d->batch < 1 || d->batch > 65535) {
        set_error(kBadArgument, "gemm_static: need M, N, K >= 1 and 1 <= batch <= 65535 (got %d %d %d, batch %d)", d->M, d->N, d->K, d->batch);
        return;
    }
    if (d->epilogue != kStore || d->args.symmetric != 0 || d->args.batch_inner > 1 || d->args.triangular != 0) {
        set_error(kBadArgument, "gemm_static: only plain-store products without the symmetric / triangular / two-level batch "
                                "options are cut along k; the others need no scratch: use qtensor_hip_gemm");
        return;
    }
    const long long need = 2LL * d->batch * d->M * d->N;       // two partial products: the least a cut needs
    if (need > QTENSOR_STATIC_SCRATCH_FLOATS) {
        set_error(kBadArgument, "gemm_static: 2 * batch * M * N = %lld floats exceed the static scratch of %d floats",
                  need, QTENSOR_STATIC_SCRATCH_FLOATS);
        return;
    }
    hipStream_t stream = (hipStream_t)stream_v;
    std::lock_guard<std::mutex> lock(static_guard);
    StaticScratch *slot = static_scratch();
    if (slot == nullptr) return;
    // A stream under graph capture launches nothing now: there is nothing to order against, and an event recorded
    // into a capture cannot be queried.  Such calls are the caller's to keep apart.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(stream, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
    if (!capturing && slot->pending && slot->last_stream != stream) {
        const hipError_t state = hipEventQuery(slot->last_done);
        if (state == hipErrorNotReady) {
            set_error(kBadArgument, "gemm_static: the static scratch of this GPU is still in use by a call on another stream; "
                                    "calls on different streams must not overlap (wait for the earlier one, or use one stream)");
            return;
        }
        if (state != hipSuccess) { set_error(kLaunchFailed, "gemm_static: hipEventQuery: %s", hipGetErrorString(state)); return; }
        slot->pending = false;
    }
    qtensor_gemm_desc with_scratch = *d;
    with_scratch.args.workspace = slot->address;
    with_scratch.args.workspace_floats = QTENSOR_STATIC_SCRATCH_FLOATS;
    gemm_dispatch(&with_scratch, stream);
    if (!capturing && error_code() == 0) {
        if (hipEventRecord(slot->last_done, stream) == hipSuccess) { slot->pending = true; slot->last_stream = stream; }
    }
}

// For callers inside the library that know their shapes better than the cost model below (the sweep's narrow
// projections): the product with the tile shape given, 0..3 = 128 x 128, 128 x 64, 64 x 128, 64 x 64.  The bits of a
// product do not depend on its tiles, only on whether k is cut, which is still decided for that shape.
namespace qt {
void gemm_with_tile(const qtensor_gemm_desc *d, hipStream_t stream, int tile);
}
void qt::gemm_with_tile(const qtensor_gemm_desc *d, hipStream_t stream, int tile) {
    qt::clear_error();
    gemm_dispatch(d, stream, tile);
}

namespace {
void gemm_dispatch(const qtensor_gemm_desc *d, hipStream_t stream, int tile_hint) {
    using namespace qt;
    if (!d) { set_error(kNullPointer, "gemm: null descriptor"); return; }
    GemmArgs a = d->args;
    a.M = d->M; a.N = d->N; a.K = d->K;
    if (d->M < 1 || d->N < 1 || d->K < 1 || d->batch < 1 || d->batch > 65535) {
        set_error(kBadArgument, "gemm: need M, N, K >= 1 and 1 <= batch <= 65535 (got %d %d %d, batch %d)", d->M, d->N, d->K, d->batch);
        return;
    }
    const int ka = d->kind_a, kb = d->kind_b, ep = d->epilogue;
    if (ka < kDense || ka > kQuant8 || kb < kDense || kb > kQuant8 || ep < kStore || ep > kRequant8) {
        set_error(kBadArgument, "gemm: unknown operand or epilogue kind (%d, %d, %d)", ka, kb, ep);
        return;
    }
    const bool requant = ep == kRequant4 || ep == kRequant8;        // no dense result: the addend is re-encoded in place
    if (!requant && (!has_host_ptr(a.C) || a.ldc < d->N)) { set_error(kBadArgument, "gemm: bad C (ldc %d < N %d or null)", a.ldc, d->N); return; }
    if (ka < kQuant4) {
        const int need = ka == kDense ? d->K : d->M;
        if (!has_host_ptr(a.A) || a.lda < need) { set_error(kBadArgument, "gemm: bad A (lda %d < %d or null)", a.lda, need); return; }
    } else {
        if (!valid_quant(a.Aq, ka == kQuant4 ? 4 : 8, "A")) return;
        if (a.Aq.order != d->M || d->K != d->M) { set_error(kBadArgument, "gemm: quantized A must be square with M == K == order"); return; }
    }
    if (kb < kQuant4) {
        const int need = kb == kDense ? d->N : d->K;
        if (!has_host_ptr(a.B) || a.ldb < need) { set_error(kBadArgument, "gemm: bad B (ldb %d < %d or null)", a.ldb, need); return; }
    } else {
        if (!valid_quant(a.Bq, kb == kQuant4 ? 4 : 8, "B")) return;
        if (a.Bq.order != d->N || d->K != d->N) { set_error(kBadArgument, "gemm: quantized B must be square with K == N == order"); return; }
    }
    if (ep == kAxpbyDense && (!has_host_ptr(a.E) || a.lde < d->N)) { set_error(kBadArgument, "gemm: bad dense addend"); return; }
    if (ep == kAxpbyQuant4 || ep == kAxpbyQuant8 || requant) {
        if (!valid_quant(a.Eq, ep == kAxpbyQuant4 || ep == kRequant4 ? 4 : 8, "addend")) return;
        if (a.Eq.order != d->M || d->M != d->N) { set_error(kBadArgument, "gemm: quantized addend must be M x N square of its order"); return; }
        if (requant && a.Eq.bs_shift != 6) { set_error(kBadArgument, "gemm: the requantizing epilogue needs blocksize 64"); return; }
    }
    if (ep == kNewton && (!has_host_ptr(a.T) || a.ldt < d->N || !a.err)) { set_error(kBadArgument, "gemm: Newton epilogue needs T and err"); return; }
    a.symmetric = a.symmetric != 0;
    a.batch_count = d->batch;
    a.stream_per = a.stream_lcm = 0;
    if (a.triangular != 0 && (ka >= kQuant4 || kb >= kQuant4 || a.symmetric || (a.triangular & ~3) != 0)) {
        set_error(kBadArgument, "gemm: triangular operands must be dense, in a product that is not marked symmetric");
        return;
    }
    if (a.batch_inner < 0) { set_error(kBadArgument, "gemm: negative inner batch count"); return; }
    if (a.symmetric && (d->M != d->N || ka >= kQuant4 || kb >= kQuant4)) {
        set_error(kBadArgument, "gemm: symmetric products need M == N and dense operands");
        return;
    }
    const bool need_code = ka >= kQuant4 || kb >= kQuant4 || ep == kAxpbyQuant4 || ep == kAxpbyQuant8 || requant;
    if (need_code && !a.code) { set_error(kNullPointer, "gemm: code table missing"); return; }

    // Tile shape: the one with the smallest estimated makespan.  Workgroups that share a compute unit
    // share its matrix pipes, so the time is (most tiles on one unit) x (tile area) / (efficiency of
    // that shape: smaller tiles read more LDS words per multiply).
    // (measured with thousands of tiles, 99 x 1024^3: 189 / 163 / 166 / 146 TFLOP/s on the split pipe -- a smaller tile splits
    // more operand elements per product -- and 126 / 119 / 123 / 117 on the fp32 pipe)
    struct Shape { int bm, bn; double eff, eff_split; };
    static const Shape shapes[4] = {{128, 128, 1.0, 1.0}, {128, 64, 0.95, 0.87}, {64, 128, 0.97, 0.88}, {64, 64, 0.93, 0.77}};
    // The split pipe: for whole k tiles, where the offsets of the dense operands' loads fit 31 bits -- whatever the tile
    // shape, so that the bits of a product do not depend on how it is tiled.
    bool split_pipe = false;
    if (a.pipe < 0 || a.pipe > 2) { set_error(kBadArgument, "gemm: pipe must be 0 (process default), 1 (fp32) or 2 (split bf16), got %d", a.pipe); return; }
    const int pipe_mode = a.pipe == 0 ? gemm_pipe_mode() : a.pipe == 1 ? kPipeF32 : kPipeSplit;
    if (pipe_mode == kPipeSplit && d->K % BK == 0 && d->K >= 2 * BK) {
        const long long reach_a = ka >= kQuant4 ? 0 : ka == kDense ? (long long)d->M * a.lda : (long long)BK * a.lda + d->M;
        const long long reach_b = kb >= kQuant4 ? 0 : kb == kDenseT ? (long long)d->N * a.ldb : (long long)BK * a.ldb + d->N;
        // (and a tile's rows, 128 at most, inside 32 bits of bytes from its first one)
        const bool near_a = ka >= kQuant4 || a.lda < (1 << 22), near_b = kb >= kQuant4 || a.ldb < (1 << 22);
        split_pipe = reach_a < 0x7fffffffLL && reach_b < 0x7fffffffLL && near_a && near_b;
    }
    int pick = 0;
    static const char *forced = QT_KNOB("QT_GEMM_TILE");
    if (forced != nullptr) {
        int fm = 0, fn = 0;
        if (sscanf(forced, "%dx%d", &fm, &fn) == 2)
            for (int i = 0; i < 4; ++i) if (shapes[i].bm == fm && shapes[i].bn == fn) pick = i;
    } else if (tile_hint >= 0 && tile_hint < 4) {
        pick = tile_hint;
    } else {
        const double units = compute_units();
        double best = 0.0;
        for (int i = 0; i < 4; ++i) {
            const Shape &sh = shapes[i];
            if (a.symmetric && sh.bm != sh.bn) continue;
            const long long tm = (d->M + sh.bm - 1) / sh.bm, tn = (d->N + sh.bn - 1) / sh.bn;
            const double tiles = (double)(a.symmetric ? tn * (tn + 1) / 2 : tm * tn) * d->batch;
            // a workgroup alone on its unit hides none of its load latencies, prologue and epilogue behind
            // another one's products: measured 0.56 of the rate reached with three per unit, 0.92 with two
            const double most = ceil(tiles / units);
            const double overlap = most <= 1.0 ? 0.56 : most <= 2.0 ? 0.92 : 1.0;
            const double cost = most * sh.bm * sh.bn / ((split_pipe ? sh.eff_split : sh.eff) * overlap);
            if (i == 0 || cost < best) { best = cost; pick = i; }
        }
    }
    if (a.symmetric && shapes[pick].bm != shapes[pick].bn) pick = 0;
    if (requant) pick = 0;          // a wave's quadrant must hold whole 64-element segments
    // Few tiles and a long k range: cut k into equal slices (whole k tiles each) that write partial products
    // to the caller's workspace and are summed in order afterwards.  Same cost model, with a fixed cost per
    // workgroup (prologue, epilogue, the extra pass over the output) worth about 64 k steps.
    a.split_k = 1;
    // (not with skip flags: the launch that adds the slices up would write the sum of slices nobody computed into the
    // results that are to be left alone)
    // (nor a quantized left factor with k up to 1024: measured on 36 to 144 output tiles, the product that is not cut
    // -- smaller tiles, three workgroups per unit -- takes 31-55 us where runs of k tiles and the launch that sums the
    // pieces take 35-57; from k = 1536 on the cut wins by a quarter and more, and so it does for a quantized right factor)
    const bool short_left = ka >= kQuant4 && d->K <= 1024;
    if (ep == kStore && !a.symmetric && a.batch_inner <= 1 && a.triangular == 0 && a.workspace != nullptr && d->K % 16 == 0 &&
        is_aligned(a.workspace, 16) && a.skip == nullptr && !short_left) {
        const Shape &sh = shapes[pick];
        const double units = compute_units();
        const long long tm = (d->M + sh.bm - 1) / sh.bm, tn = (d->N + sh.bn - 1) / sh.bn;
        const double tiles = (double)tm * tn * d->batch;
        const int k_tiles = d->K / 16;
        // Cost of a way to cut, in k steps of one workgroup that has its unit to itself: the workgroups of a launch run
        // three to a unit side by side, each at its own pace while the unit's matrix pipe has room (a lone workgroup
        // uses about half of it) -- so the time is the longer of (rounds of resident workgroups) x (k range + a fixed
        // cost per workgroup: prologue, epilogue) and (a unit's share of all k steps) x 0.5; a cut adds the launch that
        // sums the slices, worth about 200 k steps.
        const double fixed = 64.0, resident = 3.0, pipe_share = 0.5, sum_launch = 200.0;
        auto cost_of = [&](int sp) {
            const double groups = tiles * sp, range = (double)d->K / sp + fixed;
            const double rounds = ceil(groups / (units * resident)) * range;
            const double share = groups / units * range * pipe_share;
            return (rounds > share ? rounds : share) + (sp > 1 ? sum_launch : 0.0);
        };
        const double whole = cost_of(1);
        double best = whole;
        int best_split = 1;
        static const char *forced_split = QT_KNOB("QT_GEMM_SPLIT");
        for (int sp = 2; sp <= 8; ++sp) {
            if (k_tiles % sp != 0 || k_tiles / sp < 8) continue;
            if ((long long)sp * d->batch * d->M * d->N > a.workspace_floats) continue;
            const double cost = cost_of(sp);
            if (forced_split != nullptr) { if (sp == atoi(forced_split)) best_split = sp; }
            else if (cost < best) { best = cost; best_split = sp; }
        }
        if (forced_split != nullptr || best < 0.95 * whole) a.split_k = best_split;
        // The other way to cut k: lay the k tiles of all output tiles end to end and deal them out in equal
        // runs over a fixed number of workgroups per compute unit.  Every workgroup then has the same share of
        // the arithmetic whatever the number of output tiles, so the big, efficient tile shape can be kept
        // where it alone would leave half of the units idle (144 tiles of 128 x 128 on 256 units for a
        // 768 x 3072 result).  Taken when the output tiles of that shape would not fill the units twice over.
        static const int stream_wgs = QT_KNOB("QT_GEMM_STREAM_WGS") != nullptr ? atoi(QT_KNOB("QT_GEMM_STREAM_WGS")) : 2;
        const int big = d->M >= 96 && d->N >= 96 ? 0 : pick;
        const Shape &bs = shapes[big];
        const long long btm = (d->M + bs.bm - 1) / bs.bm, btn = (d->N + bs.bn - 1) / bs.bn;
        const long long big_tiles = btm * btn * d->batch, runs = big_tiles * k_tiles;
        if (stream_wgs > 0 && (ka >= kQuant4 || kb >= kQuant4) && a.skip == nullptr && k_tiles >= 16 && big_tiles < 2 * (long long)units) {
            long long groups = (long long)units * stream_wgs;
            static const int min_run = QT_KNOB("QT_GEMM_STREAM_MIN") != nullptr ? atoi(QT_KNOB("QT_GEMM_STREAM_MIN")) : 24;
            if (groups > runs / min_run) {                                // at least that many k tiles per workgroup,
                groups = runs / min_run;                                  // and no unit with one workgroup more than another
                if (groups > (long long)units) groups -= groups % (long long)units;
            }
            const long long per_group = groups > 0 ? (runs + groups - 1) / groups : 0;
            const long long used = per_group > 0 ? (runs + per_group - 1) / per_group : 0;
            if (per_group > 0 && per_group < 0x7fffffff && (used + big_tiles) * bs.bm * bs.bn <= a.workspace_floats) {
                long long x = per_group, y = k_tiles;
                while (y != 0) { const long long r = x % y; x = y; y = r; }
                const long long lcm = per_group / x * k_tiles;
                if (lcm < 0x7fffffff) {
                    a.stream_per = (int)per_group;
                    a.stream_lcm = (int)lcm;
                    a.split_k = 1;
                    pick = big;
                }
            }
        }
    }
    const int combo = ka * 100 + kb * 10 + ep;
#define QT_GEMM_CASE_DENSE(KA, KB, EP)                                                                       \
    case (KA) * 100 + (KB) * 10 + (EP):                                                                      \
        if (split_pipe) {                                                                                    \
            if (pick == 0) launch_gemm<128, 128, KA, KB, EP, kPipeSplit>(a, d->batch, stream);               \
            else if (pick == 1) launch_gemm<128, 64, KA, KB, EP, kPipeSplit>(a, d->batch, stream);           \
            else if (pick == 2) launch_gemm<64, 128, KA, KB, EP, kPipeSplit>(a, d->batch, stream);           \
            else launch_gemm<64, 64, KA, KB, EP, kPipeSplit>(a, d->batch, stream);                           \
        }                                                                                                    \
        else if (pick == 0) launch_gemm<128, 128, KA, KB, EP>(a, d->batch, stream);                          \
        else if (pick == 1) launch_gemm<128, 64, KA, KB, EP>(a, d->batch, stream);                           \
        else if (pick == 2) launch_gemm<64, 128, KA, KB, EP>(a, d->batch, stream);                           \
        else launch_gemm<64, 64, KA, KB, EP>(a, d->batch, stream);                                           \
        break;
#define QT_GEMM_CASE_REQUANT(KA, KB, EP)                                                                     \
    case (KA) * 100 + (KB) * 10 + (EP):                                                                      \
        if (split_pipe) launch_gemm<128, 128, KA, KB, EP, kPipeSplit>(a, d->batch, stream);                  \
        else launch_gemm<128, 128, KA, KB, EP>(a, d->batch, stream);                                         \
        break;
#define QT_GEMM_CASE_QUANT(KA, KB, EP)                                                                        \
    case (KA) * 100 + (KB) * 10 + (EP):                                                                      \
        if (split_pipe) {                                                                                    \
            if (pick == 0) launch_gemm<128, 128, KA, KB, EP, kPipeSplit>(a, d->batch, stream);               \
            else if (pick == 1) launch_gemm<128, 64, KA, KB, EP, kPipeSplit>(a, d->batch, stream);           \
            else if (pick == 2) launch_gemm<64, 128, KA, KB, EP, kPipeSplit>(a, d->batch, stream);           \
            else launch_gemm<64, 64, KA, KB, EP, kPipeSplit>(a, d->batch, stream);                           \
        }                                                                                                    \
        else if (pick == 0) launch_gemm<128, 128, KA, KB, EP>(a, d->batch, stream);                          \
        else if (pick == 1) launch_gemm<128, 64, KA, KB, EP>(a, d->batch, stream);                           \
        else if (pick == 2) launch_gemm<64, 128, KA, KB, EP>(a, d->batch, stream);                           \
        else launch_gemm<64, 64, KA, KB, EP>(a, d->batch, stream);                                           \
        break;
    switch (combo) {
        QT_GEMM_CASE_QUANT(kQuant4, kDense, kStore)
        QT_GEMM_CASE_QUANT(kQuant8, kDense, kStore)
        QT_GEMM_CASE_QUANT(kDense, kQuant4, kStore)
        QT_GEMM_CASE_QUANT(kDense, kQuant8, kStore)
        QT_GEMM_CASE_DENSE(kDense, kDenseT, kStore)
        QT_GEMM_CASE_DENSE(kDense, kDenseT, kAxpbyDense)
        QT_GEMM_CASE_DENSE(kDense, kDenseT, kAxpbyQuant4)
        QT_GEMM_CASE_DENSE(kDense, kDenseT, kAxpbyQuant8)
        QT_GEMM_CASE_REQUANT(kDense, kDenseT, kRequant4)
        QT_GEMM_CASE_REQUANT(kDense, kDenseT, kRequant8)
        QT_GEMM_CASE_REQUANT(kDenseT, kDense, kRequant4)
        QT_GEMM_CASE_REQUANT(kDenseT, kDense, kRequant8)
        QT_GEMM_CASE_DENSE(kDenseT, kDense, kStore)
        QT_GEMM_CASE_DENSE(kDenseT, kDense, kAxpbyDense)
        QT_GEMM_CASE_DENSE(kDenseT, kDense, kAxpbyQuant4)
        QT_GEMM_CASE_DENSE(kDenseT, kDense, kAxpbyQuant8)
        QT_GEMM_CASE_DENSE(kDense, kDense, kStore)
        QT_GEMM_CASE_DENSE(kDense, kDense, kAxpbyDense)
        QT_GEMM_CASE_DENSE(kDense, kDense, kNewton)
        default:
            set_error(kBadArgument, "gemm: combination A kind %d, B kind %d, epilogue %d is not built", ka, kb, ep);
            return;
    }
#undef QT_GEMM_CASE_DENSE
#undef QT_GEMM_CASE_REQUANT
#undef QT_GEMM_CASE_QUANT
    launch_ok("gemm");
}
}  // namespace
