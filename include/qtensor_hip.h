/*
 * qtensor_hip.h -- C ABI of libqtensor_hip.so, the gfx950 replacement of the reference's
 * libqtensor_cuda{XY}.so.
 *
 * All pointers are DEVICE pointers on the caller's current HIP device (the code table
 * included).  The library never allocates, frees or retains caller memory, never
 * synchronises the device, and is re-entrant.  Matrices are order x order, row-major,
 * contiguous.  Quantisation segments are row pieces of `blocksize` consecutive elements
 * (the last piece of a row is shorter when blocksize does not divide order);
 * absmax[row * ceil(order/blocksize) + piece].  4-bit codes pack two per byte over the
 * FLAT element stream, first element in the HIGH nibble, an odd tail padded with 0.
 *
 * Arithmetic is that of the reference's CPU path (qtensor/functional.py:526-746), NOT of
 * its CUDA kernels: true fp32 division by the segment maximum, nearest table entry by two
 * fp32-rounded distances with ties to the lower index, index 0 for all-zero segments,
 * +0.0 when dequantizing a zero-maximum segment.
 *
 * The 16 unsuffixed entry points have exactly the names and argument order that the
 * reference binds with ctypes (cudaC_python/csrc/pythonInterface.cpp:27-52, bound at
 * qtensor/functional.py:17-60, called at :155, :211, :282, :343).  They launch on the
 * null stream, as the reference's `<<<grid, threads>>>` launches do
 * (cudaC_python/csrc/ops.cu:13).  Each has a `_stream` twin taking a hipStream_t as the
 * last argument.  blocksize must be one of 64,128,256,512,1024,2048 and order >= 1;
 * order*order must be below 2^31.  A violated precondition or a failed launch is
 * reported on stderr and through qtensor_hip_last_error(); nothing is launched then.
 * (The reference prints and calls exit(1), cudaC_python/csrc/ops.cuh:20-26.)
 */
#ifndef QTENSOR_HIP_H
#define QTENSOR_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *qtensor_stream_t; /* a hipStream_t; NULL = the null stream */
typedef uint16_t qtensor_bf16;  /* raw bfloat16 bits */

/* Library/version probe; returns 10000*major + 100*minor + patch. */
int qtensor_hip_version(void);
/* 0 if the last call on this host thread succeeded, else a nonzero code; the text is in
 * qtensor_hip_last_error_string().  Reading clears nothing; the next call resets it. */
int qtensor_hip_last_error(void);
const char *qtensor_hip_last_error_string(void);

/* Replaces pythonInterface.cpp:29-33 (called from functional.py:155). */
void cquantize_blockwise_8bit_fp32(float *A, float *code, int order, float *absmax, unsigned char *out, int blocksize);
void cquantize_blockwise_8bit_bf16(qtensor_bf16 *A, float *code, int order, float *absmax, unsigned char *out, int blocksize);
void cquantize_blockwise_4bit_fp32(float *A, float *code, int order, float *absmax, unsigned char *out, int blocksize);
void cquantize_blockwise_4bit_bf16(qtensor_bf16 *A, float *code, int order, float *absmax, unsigned char *out, int blocksize);

/* Replaces pythonInterface.cpp:35-39 (called from functional.py:211). */
void cdequantize_blockwise_8bit_fp32(unsigned char *A, float *code, int order, float *absmax, float *out, int blocksize);
void cdequantize_blockwise_8bit_bf16(unsigned char *A, float *code, int order, float *absmax, qtensor_bf16 *out, int blocksize);
void cdequantize_blockwise_4bit_fp32(unsigned char *A, float *code, int order, float *absmax, float *out, int blocksize);
void cdequantize_blockwise_4bit_bf16(unsigned char *A, float *code, int order, float *absmax, qtensor_bf16 *out, int blocksize);

/* Replaces pythonInterface.cpp:41-45 (called from functional.py:282).  diag[order] receives
 * the exact fp32 diagonal; the diagonal counts as 0 for the segment maxima and codes. */
void cquantize_blockwise_diagreal_8bit_fp32(float *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize);
void cquantize_blockwise_diagreal_8bit_bf16(qtensor_bf16 *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize);
void cquantize_blockwise_diagreal_4bit_fp32(float *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize);
void cquantize_blockwise_diagreal_4bit_bf16(qtensor_bf16 *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize);

/* Replaces pythonInterface.cpp:47-51 (called from functional.py:343).  out[i,i] = diag[i]. */
void cdequantize_blockwise_diagreal_8bit_fp32(unsigned char *A, float *code, int order, float *absmax, float *diag, float *out, int blocksize);
void cdequantize_blockwise_diagreal_8bit_bf16(unsigned char *A, float *code, int order, float *absmax, float *diag, qtensor_bf16 *out, int blocksize);
void cdequantize_blockwise_diagreal_4bit_fp32(unsigned char *A, float *code, int order, float *absmax, float *diag, float *out, int blocksize);
void cdequantize_blockwise_diagreal_4bit_bf16(unsigned char *A, float *code, int order, float *absmax, float *diag, qtensor_bf16 *out, int blocksize);

/* The same sixteen with an explicit stream (no counterpart in the reference, whose launches
 * are pinned to the null stream; these let the host mirror follow torch's current stream). */
void cquantize_blockwise_8bit_fp32_stream(float *A, float *code, int order, float *absmax, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_8bit_bf16_stream(qtensor_bf16 *A, float *code, int order, float *absmax, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_4bit_fp32_stream(float *A, float *code, int order, float *absmax, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_4bit_bf16_stream(qtensor_bf16 *A, float *code, int order, float *absmax, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_8bit_fp32_stream(unsigned char *A, float *code, int order, float *absmax, float *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_8bit_bf16_stream(unsigned char *A, float *code, int order, float *absmax, qtensor_bf16 *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_4bit_fp32_stream(unsigned char *A, float *code, int order, float *absmax, float *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_4bit_bf16_stream(unsigned char *A, float *code, int order, float *absmax, qtensor_bf16 *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_diagreal_8bit_fp32_stream(float *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_diagreal_8bit_bf16_stream(qtensor_bf16 *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_diagreal_4bit_fp32_stream(float *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cquantize_blockwise_diagreal_4bit_bf16_stream(qtensor_bf16 *A, float *code, int order, float *absmax, float *diag, unsigned char *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_diagreal_8bit_fp32_stream(unsigned char *A, float *code, int order, float *absmax, float *diag, float *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_diagreal_8bit_bf16_stream(unsigned char *A, float *code, int order, float *absmax, float *diag, qtensor_bf16 *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_diagreal_4bit_fp32_stream(unsigned char *A, float *code, int order, float *absmax, float *diag, float *out, int blocksize, qtensor_stream_t stream);
void cdequantize_blockwise_diagreal_4bit_bf16_stream(unsigned char *A, float *code, int order, float *absmax, float *diag, qtensor_bf16 *out, int blocksize, qtensor_stream_t stream);

/* ---- stacks of equally sized matrices in one launch (no counterpart in the reference, which
 * loops over matrices in Python: optimizers/shampoo2.py:184-200, 249-269) --------------------
 * A is batch x order x order, contiguous; absmax, diag and out are the per-matrix buffers of
 * the single-matrix entry points laid end to end (order * ceil(order / blocksize) maxima, order
 * diagonal entries, ceil(order * order * bits / 8) code bytes per matrix: the codes of an odd order are
 * padded to a whole byte per matrix).  batch*order*order < 2^31.  With blocksize dividing order and
 * 16-byte aligned A/out the whole stack is one stream of segments (the fast path); any other order goes
 * through the general path, one matrix per grid row, at most 65535 matrices per launch.  diag == NULL
 * selects the plain form. */
void qtensor_hip_quantize_batched(const void *A, int a_is_bf16, const float *code, int bits, int order, int batch,
                                  float *absmax, float *diag, unsigned char *out, int blocksize, qtensor_stream_t stream);
void qtensor_hip_dequantize_batched(const unsigned char *q, const float *code, int bits, int order, int batch,
                                    const float *absmax, const float *diag, void *out, int out_is_bf16, int blocksize,
                                    qtensor_stream_t stream);
/* Plain (no diagonal) quantizer applied to the transpose of every matrix of an fp32 stack, without
 * writing the transpose out: entry b equals cquantize_blockwise_*bit_fp32 of A[b]^T.  Replaces
 * `V.T.contiguous()` followed by the quantizer at qtensor/utils.py:169-170 of the reference.
 * Needs blocksize in {64, 128, 256} dividing order, order a multiple of 64, 16-byte aligned A. */
void qtensor_hip_quantize_transposed_batched(const float *A, const float *code, int bits, int order, int batch,
                                             float *absmax, unsigned char *out, int blocksize, qtensor_stream_t stream);

/* ---- self check and calibration (no counterpart in the reference) ------------------------
 * The flat-path quantizer replaces IEEE division by the segment maximum a with r = rcp(a) refined
 * by one Newton step and q = fma(fma(-x*r, a, x), r, x*r).  This entry point compares both
 * with IEEE division on the device for every divisor bit pattern lo_bits, lo_bits+stride, ...
 * <= hi_bits (0x21800000 = 2^-60 <= lo <= hi <= 0x5d800000 = 2^60), x_per_a pseudo-random
 * numerators each.  counts (device, 3 x uint64, zeroed by the caller) receives
 * {reciprocal mismatches, quotient mismatches, pairs tried}. */
void qtensor_hip_check_fast_division(uint32_t lo_bits, uint32_t hi_bits, uint32_t stride, int x_per_a,
                                     unsigned long long *counts, qtensor_stream_t stream);
/* Plain device copy of n floats (n divisible by 4, 16-byte aligned): a kernel of exactly known
 * HBM traffic (4n bytes read, 4n written) against which profiler byte counters are scaled. */
void qtensor_hip_copy_f32(const float *src, float *dst, unsigned long long n, qtensor_stream_t stream);

/* ---- batched fp32 products on the matrix cores with fused (de)quantization --------------------
 * Replaces, for a whole batch of equally shaped problems in one launch, what the reference
 * does as separate torch calls per matrix:
 *   P = dequantize(Pq); P @ G and G @ P        optimizers/shampoo2.py:255-268, shampoo1.py:224-237
 *   G @ G.T, G.T @ G, L.mul_(b).add_(S, alpha=1-b) on the dequantized statistic
 *                                              optimizers/shampoo1.py:164-178, shampoo2.py:185-199
 *   the matmuls and max|M - I| of the coupled Newton inverse root
 *                                              optimizers/matrix_functions.py:127-140
 * C[b] = epilogue(opA(A[b]) * opB(B[b])), b = 0..batch-1, all matrices row-major fp32 unless
 * quantized.  A quantized operand is a square matrix in the layout of cquantize_blockwise_*
 * with blocksize dividing its order (diag optional); 4-bit codes need 4-byte, 8-bit codes
 * 8-byte alignment. */
typedef struct {
    const void *base;           /* entry b lives at base + b * stride elements ...            */
    const void *const *list;    /* ... unless list != NULL: then at list[b] (device array)    */
    long long stride;
} qtensor_batch_ptr;

typedef struct {
    qtensor_batch_ptr codes;    /* uint8                                                      */
    qtensor_batch_ptr absmax;   /* float                                                      */
    qtensor_batch_ptr diag;     /* float; both pointers NULL = plain form without diagonal    */
    int order;
    int bs_shift;               /* log2(blocksize), 6..11                                     */
} qtensor_quant_ref;

enum { QTENSOR_DENSE = 0, QTENSOR_DENSE_T = 1, QTENSOR_QUANT4 = 2, QTENSOR_QUANT8 = 3 };
enum { QTENSOR_EPI_STORE = 0, QTENSOR_EPI_AXPBY_DENSE = 1, QTENSOR_EPI_AXPBY_QUANT4 = 2,
       QTENSOR_EPI_AXPBY_QUANT8 = 3, QTENSOR_EPI_NEWTON = 4,
       /* beta * deq(Eq) + alpha * (A B) re-encoded IN PLACE into Eq's codes, maxima and exact diagonal (C is
        * not used): the statistics update L <- beta L + (1 - beta) G G^T of optimizers/shampoo1.py:164-178
        * (dequantize, update, quantize) in one launch.  Blocksize 64; bit-identical to AXPBY_QUANT* followed
        * by the stack quantizer. */
       QTENSOR_EPI_REQUANT4 = 5, QTENSOR_EPI_REQUANT8 = 6 };

typedef struct {
    int M, N, K, batch;
    int kind_a;                 /* DENSE: A is M x K (lda); DENSE_T: stored K x M (lda); QUANT*: Aq, M == K   */
    int kind_b;                 /* DENSE: B is K x N (ldb); DENSE_T: stored N x K (ldb); QUANT*: Bq, K == N   */
    int epilogue;
    struct {
        int M_, N_, K_;         /* ignored (overwritten from the fields above)                 */
        qtensor_batch_ptr A; int lda;
        qtensor_batch_ptr B; int ldb;
        qtensor_quant_ref Aq, Bq;
        qtensor_batch_ptr C; int ldc;
        float alpha, beta;      /* AXPBY: C = beta * E + alpha * (A B)                          */
        qtensor_batch_ptr E; int lde;
        qtensor_quant_ref Eq;   /* AXPBY_QUANT*: E is this quantized M x M matrix               */
        qtensor_batch_ptr T; int ldt;   /* NEWTON: T = (1 - w) I + w (A B), besides C = A B     */
        float newton_w;
        float *err;             /* NEWTON: err[b] = max(err[b], max |A B - I|); caller zeroes   */
        const int *skip;        /* optional device array: skip[b] != 0 leaves entry b untouched */
        const float *code;      /* code table of the quantized operands / addend               */
        int symmetric;          /* != 0: A B is known to be symmetric (M == N, dense operands): only the tiles
                                 * on and above the diagonal are multiplied out and every off-diagonal
                                 * tile is also stored mirrored; an addend is read at the mirrored place   */
        float *workspace;       /* optional scratch (16-byte aligned) of workspace_floats floats: a plain-store
                                 * product with few output tiles and a long k range is then cut along k (equal
                                 * slices per output tile, or equal runs over the k tiles of all output tiles);
                                 * the partial products land here and are summed in a fixed order             */
        long long workspace_floats;
        int split_k_;           /* ignored (set by the library)                                             */
        int batch_count_, stream_per_, stream_lcm_;   /* ignored (set by the library)                        */
        int batch_inner;        /* > 1: two-level batch for the strided dense operands A, B, C, E (blocks inside the
                                 * matrices of a stack): entry b lives at base + (b / batch_inner) * stride +
                                 * (b % batch_inner) * inner_x elements; 0 or 1: plain batch                    */
        long long inner_a, inner_b, inner_c, inner_e;
        int triangular;         /* bit 0: A is upper triangular (A[m][k] = 0 for k < m), bit 1: B is upper triangular
                                 * (B[k][n] = 0 for k > n), square in their k index: the zero part of the k range is
                                 * skipped (dense operands only, not with `symmetric`)                           */
        int pipe;               /* which matrix pipe multiplies this product: 0 = the process-wide choice
                                 * (qtensor_hip_gemm_pipe), 1 = the fp32 pipe, 2 = the split bf16 pipe (where its
                                 * conditions hold, see qtensor_hip_gemm_pipe; the fp32 pipe otherwise)          */
    } args;
} qtensor_gemm_desc;

/* Combinations built: (QUANT*, DENSE, STORE), (DENSE, QUANT*, STORE), (DENSE, DENSE_T, STORE|AXPBY_*),
 * (DENSE_T, DENSE, STORE|AXPBY_*), (DENSE, DENSE, STORE|AXPBY_DENSE|NEWTON), and REQUANT* with
 * (DENSE, DENSE_T) or (DENSE_T, DENSE); anything else is an error. */
void qtensor_hip_gemm(const qtensor_gemm_desc *desc, qtensor_stream_t stream);

/* qtensor_hip_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc); it has no counterpart in the reference.  The partial
 * products of a product that is cut along k go to a static device array of the library image,
 * QTENSOR_STATIC_SCRATCH_FLOATS floats (64 MiB) per GPU, held until the process ends; desc->args.workspace
 * is ignored and nothing is allocated or freed, here or in any routine it calls.  Takes the plain-store
 * epilogue without the symmetric / triangular / two-level batch options (the only products that are ever cut);
 * anything else, and any product with 2 * batch * M * N > QTENSOR_STATIC_SCRATCH_FLOATS, is refused with an
 * error and nothing is launched.  Results are bit-identical to qtensor_hip_gemm with a caller workspace of
 * that size.  All calls on one GPU share the array, so calls that overlap in time on one GPU would race: calls on
 * one stream are ordered by the stream; a call on another stream than the last one is refused with an error
 * (nothing launched) while the last call's work is still running on the GPU -- wait for it first.  A stream under
 * graph capture is not checked (nothing runs at capture time): keeping replays of such graphs apart is the
 * caller's business.  Nothing in the array needs clearing between calls (every partial product is written in
 * full before it is read).  The first call on a GPU looks the array's address up (hipGetSymbolAddress) and makes
 * the event that the check uses: make it before a graph capture begins. */
#define QTENSOR_STATIC_SCRATCH_FLOATS (1 << 24)
void qtensor_hip_gemm_static(const qtensor_gemm_desc *desc, qtensor_stream_t stream);

/* Which matrix pipe multiplies, for the whole process (no counterpart in the
 * reference, whose products are torch's fp32 matmul).
 *   0: the fp32 pipe (v_mfma_f32_32x32x2_f32) on the operands as they are;
 *   1: the bf16 pipe on split operands: every fp32 element x is written as h + m + l, three bf16 numbers, each the
 *      round-to-nearest of what the ones before leave over (|x - h - m - l| <= 2^-24 |x|), and a b is taken as
 *      a_h b_h + a_h b_m + a_m b_h + a_h b_l + a_l b_h + a_m b_m -- six bf16 products, each exact in fp32, summed
 *      in fp32 by v_mfma_f32_32x32x16_bf16.  What is left out is below 2^-24 |a b| per product, so a dot product
 *      carries the error of fp32 arithmetic (tests/test_gpu_gemm.py measures both pipes against float64), while the
 *      bf16 pipe does sixteen multiply-adds per cycle for every one of the fp32 pipe.  Differences: an infinite
 *      operand element gives NaN where the fp32 pipe gives infinity, and so does a finite one of magnitude
 *      >= 0x7f7f8000 as bits (about 3.3962e38, the top 2^-9 of the fp32 range), whose leading piece rounds to the
 *      bf16 infinity; elements below 2^-110 lose their low pieces.
 *      Taken for K a multiple of 16 and at least 32 (dense operands within 31-bit offsets; quantized operands are
 *      expanded to fp32 and split the same way), under every tile shape, so that the bits of a product do not
 *      depend on how it is tiled; every other product runs on the fp32 pipe whatever the mode.  In a symmetric
 *      product every element below the diagonal takes the value of its partner above (a b and b a add their
 *      pieces in different orders): the result is exactly symmetric.
 * mode < 0 only queries.  Returns the mode in force before the call.  The initial mode is 1 unless the environment
 * variable QT_GEMM_PIPE is "f32".  Every product that leaves args.pipe at 0 reads the mode when it is launched,
 * including the products inside the Cholesky / Gram-Schmidt entry points below: change it only while no other
 * host thread is launching products (before an optimizer's first step, say), or choose per product with args.pipe.
 * (QT_GEMM_PIPE is the only environment variable a release build reads; builds made with -DQT_TUNING_KNOBS also
 * read QT_GEMM_TILE, QT_GEMM_SPLIT, QT_GEMM_STREAM_WGS, QT_GEMM_STREAM_MIN, QT_BGS_PANEL and QT_SOLVE_PANEL, which
 * force tile shapes, k cuts and panel widths for experiments and thereby change summation orders.) */
int qtensor_hip_gemm_pipe(int mode);

/* Yardstick for the product kernels (no counterpart in the reference): one launch in which every wave of
 * workgroups_per_unit workgroups per compute unit does nothing but matrix instructions on register operands of
 * pseudo-random bits -- per round 24 x v_mfma_f32_32x32x16_bf16 (pipe 1) or 32 x v_mfma_f32_32x32x2_f32 (pipe 0).
 * Returns the floating-point operations of the launch (0 and the error slot on bad arguments); time it with
 * events: the rate is what the pipe sustains at the clock it holds under that load.  `sink`: a device word. */
double qtensor_hip_mfma_rate_flop(int pipe, int rounds, int workgroups_per_unit, float *sink, qtensor_stream_t stream);

/* ---- batched Cholesky factorisation and triangular solve (Cholesky QR) ---------------------------
 * Replace, for a whole stack of statistics at once, the QR factorisation the reference calls per
 * matrix in QTensorSVDFast.quantize (torch.linalg.qr, qtensor/utils.py:157): one round of
 *   G = Q^T Q (qtensor_hip_gemm, symmetric);  U = chol(G);  Q <- Q U^-1
 * keeps span(Q[:, :k]) for every k, so repeating it until Q is orthonormal yields the Q factor.
 * Stacks are contiguous [batch, n, n] fp32 with n a multiple of 64; everything runs on `stream`.
 *
 * cholesky_upper: gram (upper triangle read, contents destroyed) = U^T U.  u receives the block
 *   rows of U on and above the diagonal (of the part below the diagonal blocks only the 64 x 64 block under
 *   each diagonal block is written: scratch); the
 *   64 x 64 diagonal blocks of x [batch, n, n] receive the inverses of U's diagonal blocks (nothing
 *   else of x is touched).  info[b] (zeroed by the caller) gets bit 0 set when matrix b has a
 *   non-positive or NaN pivot (its factor is then meaningless).
 * cholesky_upper_floor: the same with a floor under the pivots (the squared lengths of what is left of a
 *   column after the columns before it are taken out): a pivot that is not above pivot_floor -- a column that
 *   depends on the earlier ones up to the rounding noise of the Gram matrix -- is taken out of the factorisation
 *   (pivot = the floor, rest of its row of U zero) and bit 1 of info[b] is set; q U^-1 then leaves that column
 *   lifted by 1 / sqrt(pivot_floor) instead of failing, and a repeated round completes the basis.  Bit 0 is
 *   then only set by a NaN.  pivot_floor = 0 is cholesky_upper.
 * solve_upper_right: out = q U^-1 for q, out [batch, rows, n] with u, x from cholesky_upper.  x must
 *   be zero below its diagonal blocks (zero it once before the first factorisation; no call writes
 *   there).  Its inverted diagonal blocks are doubled level by level (two launches per level for all
 *   blocks of all matrices) up to 256 x 256; then the column panels of that width are solved in turn,
 *   out_j = (q_j - out_<j U_<j,j) x_jj.  work is scratch of batch * max(rows, n) * n floats (gram may
 *   be passed when rows <= n).  out must not alias q. */
void qtensor_hip_cholesky_upper_batched(float *gram, float *u, float *x, int *info, int n, int batch, qtensor_stream_t stream);
void qtensor_hip_cholesky_upper_floor_batched(float *gram, float *u, float *x, int *info, int n, int batch, float pivot_floor,
                                              qtensor_stream_t stream);
/* Block Gram-Schmidt with reorthogonalisation, in place: the columns of every q[b] (n x n, unit columns on entry) are
 * made orthonormal left to right in panels -- a panel has the finished columns taken out of it (W = Q_<^T Y_p,
 * Y_p -= Q_< W), is orthonormalised inside, and all of that once more; on the outer level a panel is
 * qtensor_hip_block_gram_schmidt_width() columns wide and "inside" is the same scheme over its 64-column panels,
 * where "inside" is one Cholesky QR round in three launches: the Gram matrix of the panel as it is, its factorisation
 * scaled to a unit diagonal (pivot_floor as in cholesky_upper_floor), and the panel times D^-1 U^-1.  Keeps
 * span(q[:, :k]) for every k like the Cholesky QR rounds above, but loses orthogonality only in proportion to fp32
 * rounding, not to the squared condition number, so one sweep replaces their repetition; it replaces torch.linalg.qr
 * of qtensor/utils.py:157 for a whole stack.  fill (optional, [n, n], unit columns): a column that the projections of
 * the first pass leave shorter than sqrt(null_norm2) -- rounding noise: it depends on the columns before it -- leaves
 * that pass as a zero column and enters the second one as the same column of fill (bit 2 of info[b]); the last
 * 4 * batch floats of w then hold which columns those are.  w: scratch [batch, n, width]; gram, x: scratch
 * [batch, 64, 64] each; u: not used any more (kept in the signature); info as in cholesky_upper_floor (zeroed by the
 * caller), where bit 1 also stands for a column that the last pass over its panel found shortened to less than half and
 * lifted back to unit length: such a matrix can be off by the rounding error over what was left and wants a test. */
int qtensor_hip_block_gram_schmidt_width(void);
void qtensor_hip_block_gram_schmidt_batched(float *q, float *w, float *gram, float *u, float *x, const float *fill, int *info,
                                            int n, int batch, float pivot_floor, float null_norm2, qtensor_stream_t stream);
/* The same sweep; with replace_dependent != 0 (needs fill and pivot_floor > 0) a column that the first pass finds
 * dependent on the columns before it inside its 64-column panel (pivot at or below the floor) is replaced by its
 * stand-in column from fill before the second pass as well (bit 2 of info[b]), instead of being handed to the second pass
 * as it is (bit 1 if it is dependent there again).  For matrices of low numerical rank, where what a first pass leaves
 * of such a column is rounding noise: the plain sweep ends with columns that are not orthogonal there.  (No
 * counterpart in the reference: Householder QR completes a rank-deficient basis by construction.) */
void qtensor_hip_block_gram_schmidt_replacing_batched(float *q, float *w, float *gram, float *u, float *x, const float *fill,
                                                      int *info, int n, int batch, float pivot_floor, float null_norm2,
                                                      int replace_dependent, qtensor_stream_t stream);
/* The test that ends the rounds: out[2 b] = max |G_b - I|, out[2 b + 1] = ||G_b - I||_F^2 for the stack
 * gram [batch, n, n], one pass, fixed summation order, NaN if G_b holds one.  partial: scratch of
 * batch * 64 floats.  (No counterpart in the reference: Householder QR needs no such test.) */
void qtensor_hip_gram_deviation_batched(const float *gram, float *partial, float *out, int n, int batch, qtensor_stream_t stream);
/* out[b * n + j] = sum_i a[b][i][j] * b[b][i][j] for two stacks [batch, n, n] (n a multiple of 64): the diagonal of
 * a^T b in one pass over both stacks and a fixed summation order -- the Rayleigh quotients diag(Q^T (L Q)) after a
 * subspace iteration step, which the reference takes from the full product V^T L V (qtensor/utils.py:158). */
void qtensor_hip_column_dots_batched(const float *a, const float *b, float *out, int n, int batch, qtensor_stream_t stream);
/* dst[b] = src[b] (n x n fp32 each) for every b with flags[b] != 0; the other matrices of dst are left
 * alone.  Puts the previous iterate back where a factorisation failed, without a pass over the whole
 * stack and without the host knowing which ones failed.  (No counterpart in the reference.) */
void qtensor_hip_copy_flagged_batched(float *dst, const float *src, const int *flags, int n, int batch, qtensor_stream_t stream);
void qtensor_hip_solve_upper_right_batched(const float *q, const float *u, float *x, float *work, float *out,
                                           int rows, int n, int batch, qtensor_stream_t stream);

/* out[b] = a[b] v[b] for a stack a [batch, n, n] of fp32 matrices and vectors v, out [batch, n], in one launch and a
 * fixed summation order: the matrix-vector product of the power iteration that scales the ridge term of the inverse
 * roots (torch.mv per matrix and round in the reference: optimizers/matrix_functions.py:42). */
void qtensor_hip_matvec_batched(const float *a, const float *v, float *out, int n, int batch, qtensor_stream_t stream);

/* ---- the elementwise end of an optimizer step for all parameters at once -------------------------
 * Replaces the per-parameter torch calls of the reference's step():
 *   grafting   direction.mul_(grad.norm() / (direction.norm() + 1e-12))   optimizers/shampoo1.py:421, shampoo2.py:453
 *   AdamW      p.mul_(1 - lr*wd); exp_avg / exp_avg_sq update; p.addcdiv_  optimizers/shampoo1.py:405-427, shampoo2.py:446-468
 *   SGD        weight decay, momentum buffer, (Nesterov) update             optimizers/shampoo1.py:310-331, shampoo2.py:346-367
 * table: device array with one row per tensor; chunk_tensor: device array, row index of the tensor
 * that owns chunk c; a tensor of n elements owns ceil(n / qtensor_hip_tail_chunk()) consecutive
 * chunks starting at first_chunk.  partial: device scratch of 2 * n_chunks floats (only used when
 * graft != 0).  Rows with flags bit 0 set get dir rescaled to the norm of grad (dir itself is not
 * written); the others use dir as it is.  All tensors fp32. */
typedef struct {
    float *param;
    const float *dir;           /* preconditioned gradient, or the gradient itself            */
    const float *grad;          /* read only for grafted rows                                 */
    float *m;                   /* AdamW: exp_avg; SGD: momentum buffer                       */
    float *v;                   /* AdamW: exp_avg_sq; SGD: unused                             */
    long long n;
    long long first_chunk;
    long long flags;            /* bit 0: graft                                               */
} qtensor_tail_tensor;
int qtensor_hip_tail_chunk(void);
void qtensor_hip_adamw_tail(const qtensor_tail_tensor *table, const int *chunk_tensor, int n_chunks, float *partial, int graft,
                            double lr, double beta1, double beta2, double eps, double weight_decay, long long step,
                            qtensor_stream_t stream);
/* qtensor_hip_adamw_tail for parameters whose step counts differ (the reference counts steps per parameter,
 * optimizers/shampoo2.py:335-342, and skips a parameter without a gradient, :415): row_corrections (device,
 * 2 floats per table row) holds {sqrt(1 - beta2^t), -lr / (1 - beta1^t)} for that row's own step count t. */
void qtensor_hip_adamw_tail_rows(const qtensor_tail_tensor *table, const int *chunk_tensor, int n_chunks, float *partial,
                                 int graft, double lr, double beta1, double beta2, double eps, double weight_decay,
                                 const float *row_corrections, qtensor_stream_t stream);
void qtensor_hip_sgd_tail(const qtensor_tail_tensor *table, const int *chunk_tensor, int n_chunks, float *partial, int graft,
                          double lr, double momentum, double weight_decay, int nesterov, qtensor_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* QTENSOR_HIP_H */
