/*
 * libbi8 -- blockwise int8 linear hot path for AMD MI355X (gfx950), C ABI.
 *
 * The reference (LiuTaowen-Tony/blockwise_int8_linear) has no FFI: its operator boundary is three
 * Python launchers in triton_functions.py that allocate their outputs with torch.empty and start a
 * Triton kernel on the current stream.  Each entry point below replaces the device work of one of
 * those launchers; the Python side (blockwise_int8_linear_amd/ops.py) keeps the launchers' names,
 * signatures and output layouts and only allocates and forwards pointers.
 *
 * Conventions
 *   - plain pointers to DEVICE memory, element counts as int64_t, leading dimensions in ELEMENTS;
 *   - the library never allocates, frees or synchronizes; every call only enqueues kernels on
 *     `stream` (a hipStream_t passed as void*, NULL = the default stream) and returns;
 *   - re-entrant, no global mutable state, callable from any host thread;
 *   - return value 0 = success, BI8_ERR_* for rejected arguments (nothing was launched),
 *     BI8_ERR_HIP_BASE + hipError_t when the launch itself failed;
 *   - `block` is the quantization group size along the contraction dimension
 *     (block_linear_config.GROUP_SIZE, block_linear_config.py:3): any size from 1 to 2^20 is accepted;
 *     the fast kernels take powers of two (quantizers 8..512, GEMM 32, 64 and 128 with K a multiple of
 *     128 and 16-byte aligned rows), every other case runs slower general kernels with the same results;
 *   - scales use the reference's layout: fp32 [ceil(K/block), rows], block-major / row-minor
 *     (triton_functions.py:214-216, :227), and hold the block ABSMAX (not absmax/127).
 */
#ifndef BI8_H
#define BI8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of the floating-point operands (block_linear_config.INPUT_OUTPUT_TORCH_TYPE) */
#define BI8_F32 0
#define BI8_BF16 1
#define BI8_F16 2

#define BI8_OK 0
#define BI8_ERR_NULL_POINTER 1
#define BI8_ERR_BAD_DTYPE 2
#define BI8_ERR_BAD_BLOCK 3
#define BI8_ERR_BAD_SHAPE 4   /* negative size, or a leading dimension smaller than the row length */
#define BI8_ERR_TOO_LARGE 5   /* a dimension exceeds what one launch can index */
#define BI8_ERR_UNSUPPORTED 6 /* valid arguments outside what this entry point covers; nothing was launched */
#define BI8_ERR_SCRATCH_TOO_SMALL 7 /* the problem wants more scratch memory than the library's static buffer holds */
#define BI8_ERR_HIP_BASE 1000 /* BI8_ERR_HIP_BASE + hipError_t */

/* ABI version of this header (bumped on any signature change). */
int bi8_version(void);

/* Static, NUL-terminated description of a return code. */
const char *bi8_strerror(int code);

/*
 * Block quantize along rows.  Replaces quantize_block_rowwise / _quantize_block_rowwise
 * (triton_functions.py:221-233 / :193-216).
 *   x       [M,K] of x_dtype, row-major, leading dimension ldx
 *   q       int8 [M,K], leading dimension ldq:   rint_even(127 * (x / absmax)), two fp32 roundings
 *   scales  fp32 [ceil(K/block), M]:             absmax of each (row, block)
 * An all-zero block gets scale 0 and codes 0; NaN elements are ignored by the maximum and get code 0.
 */
int bi8_quantize_rowwise(const void *x, int x_dtype, int8_t *q, float *scales,
                         int64_t M, int64_t K, int64_t ldx, int64_t ldq, int block, void *stream);

/*
 * Block quantize of the TRANSPOSE, without materializing it.  Replaces the pair
 * `t = x.t().contiguous(); quantize_block_rowwise(t)` of the backward pass (block_linear.py:93-94,
 * :100-103).
 *   x        [R,C] of x_dtype, row-major, leading dimension ldx
 *   qT       int8 [C,R], leading dimension ldq;  blocks run down the columns of x
 *   scalesT  fp32 [ceil(R/block), C]
 */
int bi8_quantize_transposed(const void *x, int x_dtype, int8_t *qT, float *scalesT,
                            int64_t R, int64_t C, int64_t ldx, int64_t ldq, int block, void *stream);

/*
 * Both of the above from ONE pass over x: q / scales as bi8_quantize_rowwise writes them, qT / scalesT as
 * bi8_quantize_transposed writes them (bit for bit).  A training step of the reference quantizes each of X, W and
 * G once per direction (block_linear.py:77-78 forward, :92-94 and :100-103 backward); this entry point serves both
 * uses of a tensor with one read of it.
 *   x [R,C] leading dimension ldx;  q int8 [R,C] ld ldq, scales fp32 [ceil(C/block), R];
 *   qT int8 [C,R] ld ldqt, scalesT fp32 [ceil(R/block), C]
 * One kernel for block 32 / 64 / 128 with 16-byte aligned rows (ldq a multiple of 8, ldqt of 16); every other case
 * runs the two single-direction kernels one after the other.
 */
int bi8_quantize_dual(const void *x, int x_dtype, int8_t *q, float *scales, int8_t *qT, float *scalesT,
                      int64_t R, int64_t C, int64_t ldx, int64_t ldq, int64_t ldqt, int block, void *stream);

/*
 * bi8_quantize_dual that also returns the column sums of x: colsum[c] = cast(sum over r of x[r,c]), in x's type.
 * With x = the output gradient G this is the backward pass's bias gradient, `grad_bias = G.sum(dim=0)`
 * (block_linear.py:110), taken from the same read of G that quantizes it for the two gradient GEMMs (:92, :101-103).
 * fp32 sums in a fixed order (rows top to bottom in groups, groups and 128-row tiles ascending): deterministic, and
 * equal to torch's sum up to fp32 summation order.  `workspace`: bi8_colsum_workspace_bytes(R, C) bytes of scratch
 * memory (ceil(R/128) * C floats), 4-byte aligned, used only by the kernels of this call.
 */
int64_t bi8_colsum_workspace_bytes(int64_t R, int64_t C);
int bi8_quantize_dual_colsum(const void *x, int x_dtype, int8_t *q, float *scales, int8_t *qT, float *scalesT,
                             void *colsum, void *workspace, int64_t workspace_bytes,
                             int64_t R, int64_t C, int64_t ldx, int64_t ldq, int64_t ldqt, int block, void *stream);

/*
 * Block dequantize.  Replaces dequantize_block_rowwise / _dequantize_block_rowwise
 * (triton_functions.py:492-500 / :468-490):  out = (scale * float(q)) * fp32(1/127), cast to out_dtype.
 */
int bi8_dequantize_rowwise(const int8_t *q, const float *scales, void *out, int out_dtype,
                           int64_t M, int64_t K, int64_t ldq, int64_t ldo, int block, void *stream);

/*
 * int8 GEMM with the per-K-block dequantize fused into the K loop.  Replaces
 * int8_matmul_block64_rowwise_dequantize / _int8_matmul_block64_rowwise_dequantize
 * (triton_functions.py:142-168 / :70-139), SPLIT_K = 1 semantics.
 *   A   int8 [M,K], leading dimension lda      (quantized activations)
 *   W   int8 [N,K], leading dimension ldw      (the reference passes the view W.t(): both operands
 *                                               are contiguous along K, block_linear.py:80)
 *   sA  fp32 [ceil(K/block), M],  sW  fp32 [ceil(K/block), N]
 *   C[m,n] = cast( sum_j sW[j,n] * sA[j,m] * P_j[m,n] / 127^2 ),  P_j = int32 dot over K-block j;
 *   then, if bias != NULL (bias [N] of bias_dtype):  C = C + cast(bias), evaluated in c_dtype
 *   (triton_functions.py:127-131).  fp32 accumulation order over j is ascending; the products inside
 *   one term may be associated differently from the reference (results agree to ~1e-6 relative).
 */
int bi8_gemm_nt_dequant(const int8_t *A, const int8_t *W, const float *sA, const float *sW,
                        const void *bias, int bias_dtype, void *C, int c_dtype,
                        int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                        int block, void *stream);

/*
 * bi8_gemm_nt_dequant with a caller-provided scratch buffer.  On problems with fewer output tiles than the chip has
 * compute units (a few hundred rows of activations, or the grad-weight GEMM of a narrow layer) the contraction is
 * split: the (tile, 128-byte stage of K) pairs are dealt to the workgroups in equal runs, which need not end where a
 * tile ends, each workgroup writes fp32 partial sums of the tiles it touches to the workspace, and a second kernel adds
 * a tile's partial sums in a fixed order, casts and adds the bias.  (The reference's kernel has the same idea as SPLIT_K with atomic adds, triton_functions.py:121-139; its
 * launcher always passes SPLIT_K = 1.)  Results agree with bi8_gemm_nt_dequant to fp32 rounding of the sum over
 * K-blocks.  bi8_gemm_workspace_bytes tells how many bytes the split of a given problem wants (0: it would not
 * split); a NULL, misaligned (16 bytes) or smaller workspace makes the call identical to bi8_gemm_nt_dequant.
 * The workspace is only used by the kernels of this call, in stream order.
 */
int64_t bi8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int block);
int bi8_gemm_nt_dequant_ws(const int8_t *A, const int8_t *W, const float *sA, const float *sW,
                           const void *bias, int bias_dtype, void *C, int c_dtype,
                           int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                           int block, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * bi8_gemm_nt_dequant_ws WITHOUT a workspace argument and without any allocation: the fp32 slabs of a split of K go
 * to a static array in device memory that belongs to the library (bi8_static_scratch_bytes() = 32 MiB on every GPU
 * the library runs on, held until the process ends).  No counterpart in the reference: it is for callers that
 * cannot allocate -- code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The call
 * makes no hipMalloc / hipFree and no allocating library call; the first call on a device looks up the array's
 * address there (hipGetSymbolAddress), so make one call on each device outside any capture.
 * Same kernels, same results (bit for bit) as bi8_gemm_nt_dequant_ws given bi8_gemm_workspace_bytes() of workspace.
 * A problem whose split wants more than the array holds returns BI8_ERR_SCRATCH_TOO_SMALL and launches nothing (with
 * the present split rule -- fewer than 512 slabs of 128 x 128 fp32 -- no problem does).
 * All calls on one GPU share the array, which keeps the last call's contents (every call overwrites what it reads,
 * nothing has to start at zero): calls that overlap on one GPU -- two streams, two host threads -- race on it.
 * Serialize them on one stream, or give the overlapping ones their own workspace through bi8_gemm_nt_dequant_ws.
 */
int64_t bi8_static_scratch_bytes(void);
int bi8_gemm_nt_dequant_static(const int8_t *A, const int8_t *W, const float *sA, const float *sW,
                               const void *bias, int bias_dtype, void *C, int c_dtype,
                               int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t ldc,
                               int block, void *stream);

/*
 * Name of the kernel family that bi8_gemm_nt_dequant_ws runs on a problem with 16-byte aligned operands and
 * `workspace_bytes` of scratch memory ("gemm_wide", "gemm_wide_256x128", "gemm_wide_256x128_splitk", "gemm_tile_256x128",
 * "gemm_tile_128x128", "gemm_tile_64x128", "gemm_tile_128x128_splitk", "gemm_tile_64x128_splitk", "gemm_panel", "gemm_panel_splitk", "gemv_rows",
 * "gemv_staged", "gemm_skinny", "gemm_generic"; "gemm_wide+<tile kernel>" for a problem that runs as two launches, the 256x256 kernel on the leading
 * rows or columns that fill whole rounds of workgroups and a tile kernel on the rest; "none" for an empty problem).
 * Static string.  The reference picks its kernel configuration with Triton's autotuner
 * (triton_functions.py:41-65) and offers no way to ask which one ran; tests and benchmarks use this to say so.
 */
const char *bi8_gemm_kernel_name(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int block,
                                 int64_t workspace_bytes);

/*
 * The int32 block partial products of the same kernel, before any scaling (what tl.dot yields at
 * triton_functions.py:115):  P int32 [ceil(K/block), M, N], contiguous.  Parity/debug entry point.
 */
int bi8_gemm_nt_partials(const int8_t *A, const int8_t *W, int32_t *P,
                         int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw,
                         int block, void *stream);

/*
 * Quantize + GEMM of the eval path in ONE launch for one or two rows (single-token decode).  Replaces the pair
 * `quantize_block_rowwise(X)` + `int8_matmul_block64_rowwise_dequantize(X_int8, W_int8.t(), state_X, state_W, bias)`
 * of BlockInt8Linear.infer (block_linear.py:141-144) when X has 1 or 2 rows.
 *   x     [M,K] of `dtype`, leading dimension ldx   (activations, not yet quantized)
 *   W     int8 [N,K], leading dimension ldw;  sW fp32 [K/block, N]   (the cached weights, block_linear.py:127-128)
 *   C     [M,N] of the same `dtype`, leading dimension ldc;  bias [N] of bias_dtype or NULL
 * The result is bit for bit that of bi8_quantize_rowwise followed by bi8_gemm_nt_dequant on the same operands.
 * Covers 1 <= M <= 2, block 64 or 128, K a positive multiple of 128 with
 * 80 * roundup16((ceil(K/1024) + 1) * (1024/block)) + M*K*(1 + sizeof(elem)) + 1024 <= 65536 (x, its codes and the
 * scales sit in LDS), x and W
 * 16-byte aligned with ldx*sizeof(elem) and ldw multiples of 16; anything else
 * returns BI8_ERR_UNSUPPORTED and the caller uses the two separate entry points.
 */
int bi8_linear_few_rows(const void *x, int dtype, const int8_t *W, const float *sW,
                        const void *bias, int bias_dtype, void *C,
                        int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldc,
                        int block, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BI8_H */
