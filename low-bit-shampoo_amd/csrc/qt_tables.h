// Device-side code-table preparation shared by the quantize kernels.
//
// The reference picks a table entry for v = x / absmax as follows (qtensor/functional.py:703-715):
// ins = #{entries <= v}; lo = max(ins-1,0); hi = min(ins,n-1); take hi iff
// |fl(v - code[lo])| > |fl(code[hi] - v)|, else lo.  Inside one gap [code[i], code[i+1]] both
// rounded distances are monotone in v, so the rule flips exactly once: there is a smallest
// fp32 value thr[i] from which entry i+1 is taken.  The chosen index is therefore
// #{i : !(v < thr[i])} -- which also gives 0 below the table, n-1 above it and n-1 for NaN,
// the values the reference's clamp + searchsorted produce.  thr[] is found per workgroup by
// bisection over fp32 bit patterns with the reference's own predicate, so it is exact for any
// table, not just the two shipped ones.
#pragma once

#include "qt_common.h"
#include "qt_divide.h"

namespace qt {

constexpr int kFlagAscending = 1;  // caller's table was already non-decreasing (perm = identity)
constexpr int kFlagLut = 2;        // bucket table usable (at most one threshold per bucket, none near 0)

// Bucket table geometry: buckets are (sign, exponent, top 6 mantissa bits) of v, for
// |v| from 2^-24 up to 1.0; anything smaller shares the innermost bucket of its sign.
constexpr int kLutShift = 17;
constexpr int kLutBinades = 24;
constexpr int kLutPerSign = kLutBinades * 64 + 1;
constexpr int kLutBias = (127 - kLutBinades) << 6;
constexpr int kLutEntries = 2 * kLutPerSign;

#if defined(__HIPCC__)

template <int NCODE>
struct alignas(16) CodeTables {
    float code[NCODE];     // ascending
    float thr[NCODE];      // thr[i], i < NCODE-1; last slot = +inf
    float raw[NCODE];      // caller's order
    uint16_t bucket[NCODE];
    uint8_t perm[NCODE];   // ascending position -> caller's index
    int flags;
};

__device__ __forceinline__ bool takes_upper(float v, float clo, float chi) {
    if (v >= chi) return true;
    float dlo = v - clo;   // compiled with -ffp-contract=off: two separate fp32 roundings
    float dhi = chi - v;
    return fabsf(dlo) > fabsf(dhi);
}

__device__ __forceinline__ int lut_bucket(float v) {
    uint32_t b = __float_as_uint(v);
    int fb = (int)((b & 0x7fffffffu) >> kLutShift) - kLutBias;
    fb = min(max(fb, 0), kLutPerSign - 1);
    int s = (int)b >> 31;
    return kLutPerSign + (fb ^ s);
}

// #{i < NCODE-1 : !(v < thr[i])}; thr ascending.  NaN counts everything -> NCODE-1.
template <int NCODE>
__device__ __forceinline__ int count_thresholds(float v, const float *thr) {
    if constexpr (NCODE == 16) {
        // two levels of four: the quarter from three fixed thresholds (reads that do not depend on v), then the
        // three thresholds inside it in one 16-byte read -- one dependent LDS access instead of four
        const int quarter = (int)!(v < thr[3]) + (int)!(v < thr[7]) + (int)!(v < thr[11]);
        const float4 t = *reinterpret_cast<const float4 *>(thr + 4 * quarter);
        return 4 * quarter + (int)!(v < t.x) + (int)!(v < t.y) + (int)!(v < t.z);
    } else {
        int pos = 0;
#pragma unroll
        for (int step = NCODE / 2; step >= 1; step >>= 1)
            if (!(v < thr[pos + step - 1])) pos += step;
        return pos;
    }
}

// All threads of the workgroup call this; ends with a barrier.  lut may be nullptr.
template <int NCODE>
__device__ void build_code_tables(const float *__restrict__ code, CodeTables<NCODE> &t, uint2 *lut) {
    const int tid = threadIdx.x, nt = blockDim.x;
    for (int i = tid; i < NCODE; i += nt) t.raw[i] = code[i];
    if (tid == 0) t.flags = kFlagAscending | kFlagLut;
    __syncthreads();
    // rank sort, ties by position
    for (int i = tid; i < NCODE; i += nt) {
        const float c = t.raw[i];
        int rank = 0;
        for (int j = 0; j < NCODE; ++j) {
            const float d = t.raw[j];
            rank += (d < c) || (d == c && j < i);
        }
        t.code[rank] = c;
        t.perm[rank] = (uint8_t)i;
        if (rank != i) atomicAnd(&t.flags, ~kFlagAscending);
    }
    __syncthreads();
    for (int i = tid; i < NCODE; i += nt) {
        float th = __uint_as_float(0x7f800000u);
        if (i < NCODE - 1) {
            const float clo = t.code[i], chi = t.code[i + 1];
            if (takes_upper(clo, clo, chi)) {
                th = clo;  // repeated entry
            } else {
                uint32_t lo = float_to_key(clo), hi = float_to_key(chi);
                for (int it = 0; it < 32; ++it) {
                    if (hi - lo <= 1u) break;
                    const uint32_t mid = lo + ((hi - lo) >> 1);
                    if (takes_upper(key_to_float(mid), clo, chi)) hi = mid; else lo = mid;
                }
                th = key_to_float(hi);
            }
            // The fast quotient is only exact for |v| >= 2^-40; below that the chosen index
            // must not depend on v, so no threshold may sit that close to zero.
            if ((__float_as_uint(th) & 0x7fffffffu) < 0x2c800000u) atomicAnd(&t.flags, ~kFlagLut);
            t.bucket[i] = (uint16_t)lut_bucket(th);
        }
        t.thr[i] = th;
    }
    __syncthreads();
    if (lut != nullptr) {
        for (int b = tid; b < kLutEntries; b += nt) {
            int base = 0;   // #{i : bucket[i] < b}
#pragma unroll
            for (int step = NCODE / 2; step >= 1; step >>= 1)
                if ((int)t.bucket[base + step - 1] < b) base += step;
            const bool one = base < NCODE - 1 && (int)t.bucket[base] == b;
            const bool two = base + 1 < NCODE - 1 && (int)t.bucket[base + 1] == b;
            if (two) atomicAnd(&t.flags, ~kFlagLut);
            lut[b] = make_uint2(one ? __float_as_uint(t.thr[base]) : 0x7f800000u, (uint32_t)base);
        }
        __syncthreads();
    }
}

// ---- from one value to its table index -------------------------------------------------------
__device__ __forceinline__ uint32_t abs_bits(float x) { return __float_as_uint(x) & 0x7fffffffu; }

// Index by the exact route: IEEE division, then the threshold count.  amax_bits == 0 -> 0.
template <int NCODE>
__device__ __forceinline__ uint32_t exact_index(float x, uint32_t amax_bits, const CodeTables<NCODE> &t) {
    if (amax_bits == 0u) return 0u;
    const float q = x / __uint_as_float(amax_bits);
    return t.perm[count_thresholds<NCODE>(q, t.thr)];
}

// Bucket of a quotient known to satisfy |q| <= 1 (no upper clamp needed).
__device__ __forceinline__ int lut_bucket_unit(float q) {
    const uint32_t b = __float_as_uint(q);
    int fb = (int)((b & 0x7fffffffu) >> kLutShift) - kLutBias;
    fb = max(fb, 0);
    return kLutPerSign + (fb ^ ((int)b >> 31));
}

template <int NCODE, bool USE_LUT>
__device__ __forceinline__ uint32_t fast_index(float x, float a, float r, const CodeTables<NCODE> &t, const uint2 *lut) {
    const float q = quotient(x, a, r);
    if (USE_LUT) {
        const uint2 e = lut[lut_bucket_unit(q)];
        return e.y + (uint32_t)!(q < __uint_as_float(e.x));
    }
    return (uint32_t)count_thresholds<NCODE>(q, t.thr);
}

// Four consecutive elements per lane, G lanes per segment: the segment maximum (as bits; a NaN
// becomes the canonical one) and the four table indices, by the arithmetic of the flat quantizer.
template <int NCODE, int G>
__device__ __forceinline__ uint32_t encode_four(const float x[4], const CodeTables<NCODE> &tab, bool fast_ok, bool ascending,
                                                uint32_t idx[4]) {
    uint32_t m = max(max(abs_bits(x[0]), abs_bits(x[1])), max(abs_bits(x[2]), abs_bits(x[3])));
    m = group_max_u32<G>(m);
    // 2^-60 <= maximum <= 2^60, else (zero, huge, tiny, inf, NaN) the exact route
    if (!fast_ok || (m - kFastDivLo) > (kFastDivHi - kFastDivLo)) {
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
    return m;
}

#endif  // __HIPCC__
}  // namespace qt
