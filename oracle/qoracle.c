/*
 * qoracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar, single-threaded plain-C restatement of the blockwise quantizer that the
 * reference runs on CPU tensors.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load this library; the shipped HIP path never does.
 *
 * Reference lines restated here (paths relative to the reference checkout):
 *   qtensor/functional.py:526-615   _quantize_blockwise_cpu      -> qo_quantize
 *   qtensor/functional.py:618-688   _dequantize_blockwise_cpu    -> qo_dequantize
 *   qtensor/functional.py:703-715   _nearest_code_indices        -> nearest_index
 *   qtensor/functional.py:718-746   _pack_indices/_unpack_indices-> pack / unpack below
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -shared -fPIC (see oracle/Makefile).
 * -ffp-contract=off matters: `v - code[lo]` must be rounded to fp32 before the compare.
 *
 * Parity pins (tests/test_oracle_*.py): known-answer vectors for ties / exact codes /
 * zero and NaN segments / nibble order, exact-rational brute force of the nearest rule,
 * cross-check against an independent numpy restatement (oracle/quant_np.py) and against
 * a per-segment torch loop (oracle/quant_loop_torch.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QO_OK 0
#define QO_EBITS 1
#define QO_EBLOCK 2
#define QO_ECODE 3
#define QO_ENOMEM 4

static float canonical_nan(void) {
    union { uint32_t u; float f; } c;
    c.u = 0x7fc00000u;
    return c.f;
}

/* fp32 <- bf16 (exact) and bf16 <- fp32 (round to nearest even; every NaN becomes 0x7FC0,
 * torch's scalar cast in functional.py:671 does the same; its vectorised cast yields another
 * NaN pattern, so comparisons treat all NaNs alike). */
float qo_bf16_to_f32(uint16_t h) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)h) << 16;
    return c.f;
}

uint16_t qo_f32_to_bf16(float x) {
    union { uint32_t u; float f; } c;
    c.f = x;
    if ((c.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)0x7fc0u;
    uint32_t lsb = (c.u >> 16) & 1u;
    c.u += 0x7fffu + lsb;
    return (uint16_t)(c.u >> 16);
}

void qo_bf16_to_f32_array(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = qo_bf16_to_f32(src[i]);
}

void qo_f32_to_bf16_array(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = qo_f32_to_bf16(src[i]);
}

/* Number of table entries <= v (searchsorted, right=True).  NaN compares false with
 * everything under torch's sort order it lands after the last entry: returns n. */
static int count_le(const float *code, int n, float v) {
    if (v != v) return n;
    int lo = 0, hi = n; /* first position whose entry is > v */
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (code[mid] <= v) lo = mid + 1; else hi = mid;
    }
    return lo;
}

/* functional.py:703-715.  Two neighbours around the insertion point; the upper one
 * wins only on a strictly smaller fp32-rounded distance. */
static int nearest_index(const float *code, int n, float v) {
    int ins = count_le(code, n, v);
    int lo = ins - 1 < 0 ? 0 : ins - 1;
    int hi = ins > n - 1 ? n - 1 : ins;
    volatile float dlo = v - code[lo];
    volatile float dhi = code[hi] - v;
    return (fabsf(dlo) > fabsf(dhi)) ? hi : lo;
}

struct sort_item { float v; int i; };

static int cmp_item(const void *a, const void *b) {
    const struct sort_item *x = (const struct sort_item *)a, *y = (const struct sort_item *)b;
    if (x->v < y->v) return -1;
    if (x->v > y->v) return 1;
    return (x->i > y->i) - (x->i < y->i);
}

/* functional.py:561-565: a table that is not ascending is sorted and the chosen
 * positions are mapped back to the caller's numbering. */
static int prepare_code(const float *code, int n, float *sorted, int *perm) {
    int ascending = 1;
    for (int i = 1; i < n; ++i) if (code[i] < code[i - 1]) ascending = 0;
    if (ascending) {
        memcpy(sorted, code, sizeof(float) * (size_t)n);
        for (int i = 0; i < n; ++i) perm[i] = i;
        return 0;
    }
    struct sort_item *it = (struct sort_item *)malloc(sizeof(struct sort_item) * (size_t)n);
    if (!it) return QO_ENOMEM;
    for (int i = 0; i < n; ++i) { it[i].v = code[i]; it[i].i = i; }
    qsort(it, (size_t)n, sizeof(struct sort_item), cmp_item);
    for (int i = 0; i < n; ++i) { sorted[i] = it[i].v; perm[i] = it[i].i; }
    free(it);
    return 0;
}

static float clampf_keep_nan(float v, float lo, float hi) {
    if (v != v) return v;
    if (v < lo) return lo;
    if (v > hi) return hi;
    return v;
}

/*
 * A: order*order fp32 row-major.  absmax: order*ceil(order/blocksize).  diag: order
 * entries (only touched when store_diag).  out: ceil(order*order*bits/8) bytes.
 */
int qo_quantize(const float *A, const float *code, int order, int blocksize, int bits,
                int store_diag, float *absmax, float *diag, uint8_t *out) {
    if (bits != 4 && bits != 8) return QO_EBITS;
    if (blocksize <= 0) return QO_EBLOCK;
    const int n = 1 << bits;
    float sorted[256];
    int perm[256];
    int rc = prepare_code(code, n, sorted, perm);
    if (rc) return rc;
    const float cmin = sorted[0], cmax = sorted[n - 1];
    const int nb = (order + blocksize - 1) / blocksize;
    const int64_t total = (int64_t)order * order;
    uint8_t *idx = (uint8_t *)malloc((size_t)(total > 0 ? total : 1));
    if (!idx) return QO_ENOMEM;

    for (int r = 0; r < order; ++r) {
        const float *row = A + (int64_t)r * order;
        if (store_diag) diag[r] = row[r];                     /* functional.py:574-576 */
        for (int b = 0; b < nb; ++b) {
            const int c0 = b * blocksize;
            const int c1 = c0 + blocksize < order ? c0 + blocksize : order;
            float amax = 0.0f;
            int saw_nan = 0;
            for (int c = c0; c < c1; ++c) {
                float x = (store_diag && c == r) ? 0.0f : row[c]; /* :577-578 */
                float a = fabsf(x);
                if (a != a) saw_nan = 1;
                else if (a > amax) amax = a;
            }
            if (saw_nan) amax = canonical_nan();             /* torch max propagates NaN */
            absmax[(int64_t)r * nb + b] = amax;               /* :597-598 */
            uint8_t *seg = idx + (int64_t)r * order;
            if (amax == 0.0f) {                               /* :600-602 */
                for (int c = c0; c < c1; ++c) seg[c] = 0;
                continue;
            }
            for (int c = c0; c < c1; ++c) {
                float x = (store_diag && c == r) ? 0.0f : row[c];
                volatile float q = x / amax;                  /* :604, true fp32 divide */
                float v = clampf_keep_nan(q, cmin, cmax);
                seg[c] = (uint8_t)perm[nearest_index(sorted, n, v)];
            }
        }
    }

    if (bits == 8) {
        memcpy(out, idx, (size_t)total);
    } else {                                                  /* :718-735, high nibble first */
        const int64_t nbytes = (total + 1) / 2;
        for (int64_t k = 0; k < nbytes; ++k) {
            uint8_t hi = idx[2 * k];
            uint8_t lo = (2 * k + 1 < total) ? idx[2 * k + 1] : 0;
            out[k] = (uint8_t)((hi << 4) + lo);
        }
    }
    free(idx);
    return QO_OK;
}

/*
 * q: packed codes.  out: order*order fp32.  diag may be NULL (plain form) or order
 * entries that overwrite the diagonal (functional.py:673-678).  The caller rounds
 * to bf16 afterwards when the target dtype is bf16 (functional.py:671 casts the whole
 * matrix first and the diagonal separately, which is the same thing elementwise).
 */
int qo_dequantize(const uint8_t *q, const float *code, int order, int blocksize, int bits,
                  const float *absmax, const float *diag, float *out) {
    if (bits != 4 && bits != 8) return QO_EBITS;
    if (blocksize <= 0) return QO_EBLOCK;
    const int nb = (order + blocksize - 1) / blocksize;
    for (int r = 0; r < order; ++r) {
        for (int c = 0; c < order; ++c) {
            const int64_t k = (int64_t)r * order + c;
            int id;
            if (bits == 8) id = q[k];
            else id = (k & 1) ? (q[k >> 1] & 15) : (q[k >> 1] >> 4);   /* :738-746 */
            const float amax = absmax[(int64_t)r * nb + c / blocksize];
            volatile float y = code[id] * amax;               /* :667 */
            out[k] = (amax == 0.0f) ? 0.0f : y;               /* :663-665, +0.0 */
        }
        if (diag) out[(int64_t)r * order + r] = diag[r];
    }
    return QO_OK;
}
