/* mdy_fp8.h - C ABI of libmdyfp8.so: DeepSeek-V3-style block-wise FP8 linear path
 * for AMD MI355X (gfx950).
 *
 * Every entry point
 *   - takes raw device pointers, sizes/strides in ELEMENTS and a HIP stream
 *     (passed as void*; NULL = the null stream),
 *   - enqueues its kernels on that stream and returns without synchronising,
 *   - allocates nothing, keeps no mutable global state and is re-entrant,
 *   - returns 0 on success, a negative MDY_E_* code for a rejected argument
 *     (nothing was launched) or a positive hipError_t if the launch failed.
 *     mdy_fp8_last_error() returns a thread-local message for the last non-zero
 *     return on the calling thread.
 *
 * Sizes: every row / column count up to 2^30 (MDY_E_SHAPE beyond); operands may exceed 2^32 bytes (all
 * addressing is 64-bit).  A launch whose block count does not fit the grid limits (more than 33 million columns)
 * returns hipErrorInvalidConfiguration.
 *
 * Reference interfaces are cited as file:line under the reference tree
 * (triton_kernels/deepseekv3/offical_kernel.py = "offical_kernel.py",
 *  triton_kernels/dpsk_fp8linear/fp8.py        = "fp8.py").
 */
#ifndef MDY_FP8_H_
#define MDY_FP8_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MDY_FP8_ABI_VERSION 15

/* error codes (negative = argument rejected before any launch) */
#define MDY_OK 0
#define MDY_E_NULL (-1)      /* a required pointer is NULL */
#define MDY_E_SHAPE (-2)     /* a size/stride violates the documented precondition */
#define MDY_E_ALIGN (-3)     /* a pointer or stride is not aligned as documented */
#define MDY_E_DTYPE (-4)     /* unknown dtype / mode selector */
#define MDY_E_DEVICE (-5)    /* the current device is not a gfx950 GPU */

/* output dtype selectors */
#define MDY_DT_BF16 0
#define MDY_DT_F32 1

/* quantizer dialects */
#define MDY_QUANT_OFFICIAL 0 /* s = amax / 448                      offical_kernel.py:14 */
#define MDY_QUANT_DEEPLINEAR 1 /* s = (min(amax,1e4) + 1e-8) / 448, saturating cast  fp8.py:109-111 */
#define MDY_QUANT_OFFICIAL_E5M2 2 /* s = amax / 57344, e5m2 bytes: the default fp8 dtype of triton_kernels/deepseekv3/
                                   * fp8_kernel.py (:62, :124, :303); accepted by mdy_act_quant_typed, mdy_weight_quant(_typed)
                                   * and mdy_act_quant_transpose */

/* operand byte formats of mdy_fp8_gemm_nt_rowscaled */
#define MDY_FMT_E4M3 0
#define MDY_FMT_E5M2 1

int mdy_fp8_abi_version(void);
const char* mdy_fp8_last_error(void);

/* Per-token 1x128 activation quantizer.
 * Replaces act_quant (offical_kernel.py:21-28, kernel :9-18) with
 * mode = MDY_QUANT_OFFICIAL, PM = M, PK = K, and quant_input(only_forward=True)
 * (fp8.py:122-161, kernel :87-120) with mode = MDY_QUANT_DEEPLINEAR and the
 * padded sizes that launcher computes.
 *
 *   x  bf16 [M, K], element (m, k) at x[m * x_row_stride + k]   (unit column stride; x_row_stride >= K, or 0 for
 *      a row broadcast M times)
 *   y  e4m3fn [PM, PK] row-major; PM >= M, PK >= K, PK % 128 == 0; padding reads as 0
 *   s  fp32, scale of row m, K-block kb at s[m * s_row_stride + kb * s_col_stride]
 *      for m < PM, kb < PK / 128
 * Vector path needs x 16-byte aligned with x_row_stride % 8 == 0 and K % 8 == 0;
 * anything else takes an element-wise path inside the same kernel.
 * y must be 8-byte aligned.  M == 0 is a no-op.
 */
int mdy_act_quant(const void* x, void* y, float* s, int64_t M, int64_t K, int64_t x_row_stride,
                  int64_t PM, int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode,
                  void* stream);

/* The general form of mdy_act_quant: inputs that are not bf16 and group widths other than 128.  The reference kernels
 * load with .to(tl.float32) and so also take fp16 and fp32 tensors (offical_kernel.py:12, fp8.py:108), and act_quant
 * takes any block_size (offical_kernel.py:21-27); every input type is quantized from its exact fp32 value.
 * x_dtype = MDY_XT_BF16 with block_size = 128 is mdy_act_quant itself (the tuned kernel); everything else runs a kernel
 * whose quotient is an IEEE division per element (same results as the reference's arithmetic, slower).
 * block_size: a power of two from 8 to 512; PK % block_size == 0; the scale of row m, group g is at
 * s[m * s_row_stride + g * s_col_stride].  Strides of x in elements of x_dtype. */
#define MDY_XT_BF16 0
#define MDY_XT_F16 1
#define MDY_XT_F32 2
int mdy_act_quant_typed(const void* x, int x_dtype, int block_size, void* y, float* s, int64_t M, int64_t K,
                        int64_t x_row_stride, int64_t PM, int64_t PK, int64_t s_row_stride, int64_t s_col_stride, int mode,
                        void* stream);

/* 128x128 block weight quantizer.
 * Replaces quant_weight(only_forward=True/False) (fp8.py:206-247, kernel :171-203)
 * with mode = MDY_QUANT_DEEPLINEAR, and weight_quant_block
 * (triton_kernels/deepseekv3/fp8_kernel.py:124-138, kernel :88-122) with
 * mode = MDY_QUANT_OFFICIAL.
 *
 *   w   bf16 [N, K], element (n, k) at w[n * w_row_stride + k * w_col_stride]
 *   y   e4m3fn [PN, PK] row-major, PN % 128 == 0, PK % 128 == 0, padding reads as 0; or NULL when only the
 *       transposed copy is wanted (per_block_cast_to_fp8(output_normal=False), megatron_patchs/fp8_matmul.py:334-392)
 *   s   fp32 [PN/128, PK/128] row-major or NULL (must be given iff y is)
 *   y_t e4m3fn [PK, PN] row-major (transposed copy) or NULL
 *   s_t fp32 [PK/128, PN/128] row-major or NULL (must be given iff y_t is); at least one of y / y_t
 */
int mdy_weight_quant(const void* w, void* y, float* s, void* y_t, float* s_t, int64_t N, int64_t K,
                     int64_t w_row_stride, int64_t w_col_stride, int64_t PN, int64_t PK, int mode,
                     void* stream);
/* The same for a weight of type w_dtype (MDY_XT_BF16 / MDY_XT_F16 / MDY_XT_F32; strides in its elements): the reference
 * kernels load with .to(tl.float32) (fp8.py:193), so an fp32 master weight is quantized from its exact values. */
int mdy_weight_quant_typed(const void* w, int w_dtype, void* y, float* s, void* y_t, float* s_t, int64_t N, int64_t K,
                           int64_t w_row_stride, int64_t w_col_stride, int64_t PN, int64_t PK, int mode, void* stream);

/* Training-time quantizer: row-wise 1x128 quantization of x AND the quantized transpose,
 * one read of x.  DeepLinear dialect only (clamp 1e4 + eps 1e-8, saturating cast).
 * Replaces quant_grad_output (fp8.py:46-77, kernel :13-44) with t_mode = MDY_T_COLUMN and
 * quant_input(only_forward=False) (fp8.py:122-161, kernel branch :115-120) with
 * t_mode = MDY_T_BLOCK.
 *
 *   x    bf16 [M, K], element (m, k) at x[m * x_row_stride + k * x_col_stride]
 *   y    e4m3fn [PM, PK] row-major, PM % 128 == 0, PK % 128 == 0, padding reads as 0
 *   s    fp32, scale of row m, K-group kb at s[kb * s_kb_stride + m]; s_kb_stride >= PM (= PM for the
 *        [PK/128, PM] buffer of quant_input / quant_grad_output; the total row count when the rows are one
 *        expert group of a larger matrix, group_per_token_cast_to_fp8 at megatron_patchs/fp8_matmul.py:218-247)
 *   y_t  e4m3fn [PK, PM] row-major: y_t[k, m] = x[m, k] / scale_t
 *   s_t  MDY_T_COLUMN: one scale per column k and 128-row group a, at s_t[a * PK + k]
 *                      ([PM/128, PK] row-major; the reference returns its transpose view)
 *        MDY_T_BLOCK:  one scale per 128x128 tile, at s_t[(k/128) * (PM/128) + m/128]
 *                      ([PK/128, PM/128] row-major)
 */
#define MDY_T_COLUMN 0
#define MDY_T_BLOCK 1
int mdy_quant_transpose(const void* x, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                        int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride,
                        int t_mode, void* stream);
/* The same for an input of type x_dtype (MDY_XT_BF16 / MDY_XT_F16 / MDY_XT_F32; strides in its elements). */
int mdy_quant_transpose_typed(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                        int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int64_t s_kb_stride,
                        int t_mode, void* stream);

/* Official-dialect training quantizer (mode MDY_QUANT_OFFICIAL: s = amax / 448, e4m3fn; MDY_QUANT_OFFICIAL_E5M2:
 * s = amax / 57344, e5m2; no clamp, no eps): the row-wise 1x128 quantization of x and
 * the quantized transpose with one scale per column and 128 rows, one read of x.  Replaces the pair
 * act_quant_block(x) / act_quant_block(x, transpose=True) (triton_kernels/deepseekv3/fp8_kernel.py:62-87, kernel
 * :14-60) that the reference's Fp8Linear runs on x and on dy (:286-301).
 *
 *   x    [M, K] of x_dtype (MDY_XT_BF16 / MDY_XT_F16 / MDY_XT_F32), element (m, k) at x[m * x_row_stride + k * x_col_stride]
 *   y    e4m3fn [PM, PK] row-major or NULL (then s must be NULL too: only the transposed copy is produced)
 *   s    fp32 [PM, PK/128] row-major
 *   y_t  e4m3fn [PK, PM] row-major: y_t[k, m] = x[m, k] / s_t[k, m / 128]
 *   s_t  fp32 [PK, PM/128] row-major
 * PM >= M and PK >= K are multiples of 128; padding reads as 0 (an all-zero group has scale 0 and NaN bytes, as in the
 * reference).  y / y_t 8-byte aligned.
 */
int mdy_act_quant_transpose(const void* x, int x_dtype, void* y, float* s, void* y_t, float* s_t, int64_t M, int64_t K,
                            int64_t x_row_stride, int64_t x_col_stride, int64_t PM, int64_t PK, int mode, void* stream);

/* Block-scaled FP8 GEMM, NT layout, with 1x128 scales on both operands:
 *   c[m, n] = sum_kb (sum_{k in kb} a[m,k] * b[n,k]) * a_s[m, kb] * b_s[n, kb]
 * Replaces fp8_matmul(..., have_w=False) (triton_kernels/deepseekv3/fp8_kernel.py:214-252, kernel branch :190-205),
 * the weight-gradient GEMM of the reference's Fp8Linear (fp8_matmul_bwd, :254-257).
 *
 *   a   e4m3fn [M, K] row-major, 16-byte aligned     a_s fp32, element (m, kb) at a_s[m * as_row_stride + kb * as_col_stride]
 *   b   e4m3fn [N, K] row-major, 16-byte aligned     b_s fp32, element (n, kb) at b_s[n * bs_row_stride + kb * bs_col_stride]
 *   c   [M, N] row-major of out_dtype
 * fmt: byte format of BOTH operands, MDY_FMT_E4M3 or MDY_FMT_E5M2.  A weight with 128x128 block scales runs here too
 * with its scales expanded to one per row (bs_row_stride of the expanded tensor): the Python wrappers do that for e5m2
 * operands, which the block-scaled kernels of mdy_fp8_gemm_nt (e4m3fn only) do not take.
 * K % 128 == 0, K <= 2^20; scale strides non-negative, each scale tensor spanning less than 2^31 bytes.
 */
int mdy_fp8_gemm_nt_rowscaled(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                              const void* b, const float* b_s, int64_t bs_row_stride, int64_t bs_col_stride, void* c,
                              int64_t M, int64_t N, int64_t K, int fmt, int out_dtype, void* stream);

/* SwiGLU, alone or fused with the 1x128 activation quantizer that feeds the next GEMM.
 *   act[m, n] = bf16( silu(gate[m, n]) * up[m, n] ), silu(g) = g / (1 + exp(-g)) in fp32;
 *   (y, s)    = 1x128 quantization of act (the bf16-rounded value) as mdy_act_quant would produce it.
 * Replaces silu_fwd (triton_kernels/deepseekv3/fp8_kernel.py:384-402, kernel :315-344; the same kernel
 * is triton_kernels/megatron_patchs/swiglu.py:6-36) and the silu_fwd + act_quant pair of the FP8 MLP
 * (fp8_kernel.py:447-450, 500-515) in one pass.
 *
 *   x    bf16 [M, 2N], row m at x + m * x_row_stride; gate_first = 0: columns [0,N) are `up` and [N,2N)
 *        `gate` (the reference's order 'up-gate'); gate_first = 1: the other way round ('gate-up')
 *   act  bf16 [M, N] row-major or NULL
 *   y    e4m3fn [PM, PN] row-major or NULL (then s, PM, PN, strides and mode are ignored);
 *        PM >= M, PN >= N, PN % 128 == 0, padding quantizes as 0
 *   s    fp32, scale of (row m, group kb) at s[m * s_row_stride + kb * s_col_stride]
 *   mode MDY_QUANT_OFFICIAL or MDY_QUANT_DEEPLINEAR
 * At least one of act, y must be given.
 */
int mdy_swiglu(const void* x, void* act, void* y, float* s, int64_t M, int64_t N, int64_t x_row_stride,
               int gate_first, int64_t PM, int64_t PN, int64_t s_row_stride, int64_t s_col_stride, int mode,
               void* stream);

/* Backward of SwiGLU: dx[m, up] = silu(gate) * dy, dx[m, gate] = (sig + silu * (1 - sig)) * up * dy.
 * Replaces silu_bwd (fp8_kernel.py:404-421, kernel :346-382).
 *   x bf16 [M, 2N] (row stride x_row_stride), dy bf16 [M, N] row-major, dx bf16 [M, 2N] row-major.
 */
int mdy_swiglu_bwd(const void* x, const void* dy, void* dx, int64_t M, int64_t N, int64_t x_row_stride,
                   int gate_first, void* stream);

/* 128x128 block weight dequantizer: y[n,k] = fp32(x[n,k]) * s[n/128, k/128].
 * Replaces weight_dequant (offical_kernel.py:46-53, kernel :31-43).
 *   x e4m3fn [N, K] row-major; s fp32 [ceil(N/128), ceil(K/128)] row-major;
 *   y [N, K] row-major of out_dtype (MDY_DT_BF16 or MDY_DT_F32).
 */
int mdy_weight_dequant(const void* x, const float* s, void* y, int64_t N, int64_t K, int out_dtype,
                       void* stream);
/* The same with square scale blocks of block_size x block_size (a power of two >= 8; s is
 * [ceil(N/block_size), ceil(K/block_size)]): the reference's weight_dequant takes any block_size (offical_kernel.py:46). */
int mdy_weight_dequant_block(const void* x, const float* s, void* y, int64_t N, int64_t K, int block_size, int out_dtype,
                             void* stream);

/* Block-scaled FP8 GEMM, NT layout:
 *   c[m,n] = sum_kb (sum_{k in kb} a[m,k] * b[n,k]) * a_s[m,kb] * b_s[n/128,kb]  (+ bias[n])
 * Replaces fp8_gemm (offical_kernel.py:100-109, kernel :61-97) with
 * as_row_stride = ceil(K/128), as_col_stride = 1, and fp8_matmul (fp8.py:307-311,
 * i.e. deep_gemm.gemm_fp8_fp8_bf16_nt) with the column-major scale strides
 * (1, PM) that quant_input returns; bias folds add_bias (fp8.py:297-305) into
 * the epilogue.
 *
 *   a    e4m3fn [M, K] row-major         a_s fp32, (m,kb) at a_s[m*as_row_stride + kb*as_col_stride]
 *   b    e4m3fn [N, K] row-major         b_s fp32 [ceil(N/128), ceil(K/128)] row-major
 *   c    [M, N] row-major of out_dtype   bias bf16 [N] or NULL (added in fp32 before the cast)
 * Any M, N, K >= 1 is accepted (M == 0 or N == 0 is a no-op); K % 128 == 0 with
 * 16-byte aligned a and b takes the MFMA kernels, anything else a scalar kernel.
 */
int mdy_fp8_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                    const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                    int64_t K, int out_dtype, void* stream);

/* mdy_fp8_gemm_nt on float8_e5m2 operands (the default fp8 dtype of triton_kernels/deepseekv3/fp8_kernel.py:62,124,234):
 * the MFMA kernels with the instruction's operand format set to bf8 - the tile kernels for more than 64 rows, the
 * weight-streaming and strip kernels (or 128x128 / 64x64 tiles against a wide weight) for up to 64.  Same arguments and
 * formula as mdy_fp8_gemm_nt; any M >= 1, but only K % 128 == 0, K <= 65536, 16-byte aligned a / b and activation scales
 * that span less than 2^31 bytes (MDY_E_SHAPE otherwise: run those through mdy_fp8_gemm_nt_rowscaled with the weight's
 * block scales expanded to one per row, as the Python wrapper does). */
int mdy_fp8_gemm_nt_e5m2(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride, const void* b,
                         const float* b_s, void* c, const void* bias, int64_t M, int64_t N, int64_t K, int out_dtype,
                         void* stream);

/* The same GEMM with a caller-provided scratch buffer.  Shapes whose output tiles do not fill the GPU
 * (roughly 32 < M <= 1024 against a long K: small-batch prefill, large-batch decode) are cut along K as
 * well; the fp32 partial sums of the K slices go through `workspace` and are added in a fixed order, so the
 * result is deterministic, but it may differ in the last bit from mdy_fp8_gemm_nt (another summation order).
 * Large shapes with row-major activation scales (as_col_stride == 1) use the buffer for a [K/128, M] copy of
 * the scales, which the tile kernels fetch with 32x fewer cache-line requests (about 3 % faster; same bits).
 * No counterpart in the reference (its Triton kernel / DeepGEMM never split K); the Python wrappers fp8_gemm
 * and fp8_matmul call it with a torch-allocated buffer.
 *
 *   mdy_fp8_gemm_workspace_bytes(M, N, K)  bytes of workspace this shape can use (0: none)
 *   workspace        device memory, 16-byte aligned, workspace_bytes long; may be NULL / too small: the call
 *                    then is mdy_fp8_gemm_nt.  Calls that overlap in time need separate workspaces.
 */
int64_t mdy_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mdy_fp8_gemm_nt_ws(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                       const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                       int64_t K, int out_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* Which kernel family mdy_fp8_gemm_nt (with_workspace = 0) or mdy_fp8_gemm_nt_ws with a sufficient workspace
 * (with_workspace = 1) runs for these operands; launches nothing, needs no GPU.  No counterpart in the reference
 * (its Triton kernel has one code path); the Python wrappers use it to warn when a large shape would take the
 * scalar kernel, which exists for K % 128 != 0 and unaligned operands and is ~100x slower than the MFMA kernels
 * (aligned shapes reach it only with K > 65536, or activation scales spanning 2^31 bytes or more, and M > 64).
 * a and b are only inspected for 16-byte alignment (NULL counts as aligned).
 */
#define MDY_PATH_SCALAR 0
#define MDY_PATH_SMALL_M 1
#define MDY_PATH_STRIP 2
#define MDY_PATH_TILES 3
#define MDY_PATH_TILES_SPLIT_K 4 /* K cut into slabs of the workspace: MFMA tiles, or the small-M kernel for up to 64 rows */
int mdy_fp8_gemm_path(const void* a, const void* b, int64_t as_row_stride, int64_t as_col_stride, int64_t M,
                      int64_t N, int64_t K, int with_workspace);

/* mdy_fp8_gemm_nt_ws for callers that cannot allocate device memory and so cannot bring a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * Same arguments, kernels and results as mdy_fp8_gemm_nt_ws minus the workspace pair: the scratch memory is a
 * static device array of mdy_fp8_gemm_static_workspace_bytes() (32 MiB) inside the library, which every GPU the
 * library has run this call on holds until the process ends.  The call allocates nothing and frees nothing
 * (no hipMalloc / hipFree, no allocating library routine).
 *
 *   - a shape whose mdy_fp8_gemm_workspace_bytes(M, N, K) exceeds the static buffer is rejected with MDY_E_SHAPE
 *     (nothing launched): use mdy_fp8_gemm_nt_ws or mdy_fp8_gemm_nt for it;
 *   - every call on a GPU shares that GPU's buffer and leaves its partial sums in it: calls that overlap in time
 *     on one GPU (two streams, two threads) race - serialise them, or give the others their own workspace
 *     through mdy_fp8_gemm_nt_ws.  Nothing in the buffer has to be cleared between calls;
 *   - the buffer's device address is looked up on the first call on each device (one symbol query, no
 *     allocation); mdy_fp8_gemm_static_workspace_init() does that lookup for the current device ahead of time,
 *     e.g. before a stream capture begins.
 */
int64_t mdy_fp8_gemm_static_workspace_bytes(void);
int mdy_fp8_gemm_static_workspace_init(void);
int mdy_fp8_gemm_nt_static_ws(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                              const void* b, const float* b_s, void* c, const void* bias, int64_t M, int64_t N,
                              int64_t K, int out_dtype, void* stream);

/* Grouped (mixture-of-experts) block-scaled FP8 GEMM, NT layout: the rows of a are split into G
 * consecutive groups of m_splits[g] rows and group g is multiplied with its own weight,
 *   c[m, n] = sum_kb (sum_{k in kb} a[m,k] * b[g,n,k]) * a_s[m,kb] * b_s[g, n/128, kb]  (+ bias[g, n])
 * for the rows m of group g.  Replaces fp8_grouped_matmul
 * (triton_kernels/megatron_patchs/fp8_matmul.py:400-413, i.e.
 * deep_gemm.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous with the per-row group index built from m_splits).
 * Group sizes need no alignment (the reference pads them to 256 rows; zero-sized groups are allowed).
 *
 *   a        e4m3fn [M, K] row-major, M = sum of m_splits      a_s as in mdy_fp8_gemm_nt
 *   b        e4m3fn [G, N, K] row-major                        b_s fp32 [G, ceil(N/128), ceil(K/128)]
 *   c        [M, N] row-major of out_dtype                     bias bf16 [G, N] or NULL
 *   m_splits HOST pointer to G non-negative row counts (read before the call returns); G <= 256 for
 *            the single-launch MFMA path, larger G or K % 128 != 0 / unaligned operands run one launch
 *            per group.
 */
int mdy_fp8_grouped_gemm_nt(const void* a, const float* a_s, int64_t as_row_stride, int64_t as_col_stride,
                            const void* b, const float* b_s, void* c, const void* bias,
                            const int64_t* m_splits, int64_t G, int64_t N, int64_t K, int out_dtype,
                            void* stream);

/* Row padding (unpad = 0) / unpadding (unpad != 0) of grouped activations: the rows of the unpadded matrix are G
 * consecutive groups of m_splits[g] rows; in the padded matrix group g owns a slot of ceil(m_splits[g] / multiple) *
 * multiple rows whose rows beyond m_splits[g] are zero.  Replaces Fp8Padding / Fp8Unpadding
 * (triton_kernels/megatron_patchs/dpsk_grouped_linear.py:690-902: TransformerEngine's multi_padding_fused with
 * multiple = 256, and torch.split + torch.cat for the way back).
 *
 *   x         source, row-major, row_bytes bytes per row (any element type): [sum m, row_bytes] when padding,
 *             [sum pad(m), row_bytes] when unpadding
 *   y         destination of the other layout; every byte of it is written
 *   m_splits  HOST pointer to G non-negative row counts (read before the call returns)
 * 16-byte aligned pointers and row_bytes % 16 == 0 take the vector path; anything else is copied in 2- or 1-byte pieces.
 */
int mdy_group_pad_rows(const void* x, void* y, const int64_t* m_splits, int64_t G, int64_t row_bytes, int64_t multiple,
                       int unpad, void* stream);

/* In-place x[m, :] = bf16(fp32(x[m, :]) + fp32(b)) on bf16 x [M, N] row-major, bf16 b [N].
 * Replaces add_bias (fp8.py:297-305, kernel :283-295). */
int mdy_add_bias(void* x, const void* b, int64_t M, int64_t N, void* stream);
/* The same with a bias of type b_dtype (MDY_XT_BF16 / MDY_XT_F16 / MDY_XT_F32): the reference loads the bias with
 * .to(tl.float32) (fp8.py:291), so an fp32 bias is added at full precision. */
int mdy_add_bias_typed(void* x, const void* b, int b_dtype, int64_t M, int64_t N, void* stream);

/* In-place gradient accumulation over n elements: x[i] = T(fp32(x[i]) + fp32(y[i])), x of x_dtype, y of y_dtype
 * (MDY_DT_BF16 / MDY_DT_F32 each).  Replaces add_grad (triton_kernels/megatron_patchs/add_kernel.py:55-62, kernel
 * :41-52), the Megatron patch's accumulation of a weight gradient into main_grad. */
int mdy_add_grad(void* x, const void* y, int64_t n, int x_dtype, int y_dtype, void* stream);

/* Diagnostic: element-wise fp32 -> e4m3fn with the same device conversion the
 * quantizers use (saturate != 0 clamps finite values to +-448 first).  No
 * counterpart in the reference (the cast is implicit in tl.store, fp8.py:112);
 * exists so that the cast can be checked against the format definition. */
int mdy_cast_f32_to_e4m3(const float* x, void* y, int64_t n, int saturate, void* stream);
/* The same for the e5m2 conversion (round to nearest even, overflow to infinity), used by MDY_QUANT_OFFICIAL_E5M2. */
int mdy_cast_f32_to_e5m2(const float* x, void* y, int64_t n, void* stream);

/* Diagnostic: returns in out[0..3] the number of (amax, x) bf16 pairs, of fp32
 * quotient mismatches and of e4m3fn byte mismatches between the quantizers'
 * reciprocal+2-FMA quotient and IEEE division, over every finite bf16 amax in
 * [amax_lo, amax_hi) (bit patterns) and every bf16 x with |x| <= amax, for the
 * given dialect.  out is device memory, 4 x uint64, zeroed by the call. */
int mdy_quotient_selfcheck(uint64_t* out, int amax_lo, int amax_hi, int mode, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MDY_FP8_H_ */
