/*
 * fouroversix_hip.h -- C ABI of the gfx950 (MI355X) quantize / FP4-matmul library.
 *
 * Plain pointers and sizes only; every pointer except the error strings is DEVICE memory.
 * All entry points are asynchronous on the given HIP stream and never synchronise.  Apart
 * from fos_quantize_static (which says so below) they keep no mutable state between calls,
 * so they are safe to call from several host threads on different streams.  Return value: 0 on success, a negative FOS_E_* code otherwise
 * (nothing is launched when an argument check fails).
 *
 * Each function names the interface of the reference (mit-han-lab/fouroversix, paths
 * relative to its tree) that it stands in for.
 */
#ifndef FOUROVERSIX_HIP_H
#define FOUROVERSIX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *fos_stream_t; /* a hipStream_t; NULL = the default stream */

enum {
    FOS_OK = 0,
    FOS_E_BAD_SHAPE = -1,     /* negative / zero-size / unsupported dimension */
    FOS_E_BAD_ALIGNMENT = -2, /* pointer or leading dimension not aligned as documented */
    FOS_E_UNSUPPORTED = -3,   /* format / rule / rounding combination without a kernel */
    FOS_E_NULL_POINTER = -4,
    FOS_E_WORKSPACE = -5, /* workspace missing or too small */
    FOS_E_LAUNCH = -6     /* hipGetLastError() reported a launch failure */
};

/* formats, mirroring DataType members of src/fouroversix/utils.py:13-41 */
enum { FOS_DTYPE_NVFP4 = 0, FOS_DTYPE_IF4 = 1, FOS_DTYPE_MXFP4 = 2 };
/* scale rules with the ids of ScaleRule.cuda_id, src/fouroversix/utils.py:271-280 and
 * csrc/quantize/fp4_quant.cu:111-119 */
enum { FOS_RULE_STATIC_6 = 0, FOS_RULE_STATIC_4 = 1, FOS_RULE_MAE = 2, FOS_RULE_MSE = 3, FOS_RULE_ABS_MAX = 4 };
/* RoundStyle, src/fouroversix/utils.py:223-247 */
enum { FOS_ROUND_NEAREST = 0, FOS_ROUND_STOCHASTIC = 1, FOS_ROUND_STOCHASTIC_UNBIASED = 2 };
/* block-scale layout: row-major [rows, cols/16], or the 128x4-tile layout of
 * to_blocked(), src/fouroversix/quantize/utils.py:88-96 */
enum { FOS_SF_LINEAR = 0, FOS_SF_TILED_128X4 = 1 };
/* input / output element types */
enum { FOS_T_BF16 = 0, FOS_T_F16 = 1, FOS_T_F32 = 2 };

/* Library version (major * 10000 + minor * 100 + patch). */
int fos_version(void);

/* Human-readable text for a return code (host pointer, static storage). */
const char *fos_error_string(int code);

/* Kernel-choice overrides for tuning runs and tests (FOS_GEMM_TILE, FOS_GEMM_SPLITK,
 * FOS_MX_TILE, FOS_QUANT_GRID, FOS_AMAX_GRID) are read from the environment once, at the
 * first call that needs them; this reads them again.  No counterpart in the reference. */
void fos_tuning_reload(void);

/* Rows / columns of the padded outputs: rows up to a multiple of 128, columns up to a
 * multiple of 64 (QuantizedTensor, src/fouroversix/quantize/quantized_tensor.py:65-78). */
int64_t fos_padded_rows(int64_t rows);
int64_t fos_padded_cols(int64_t cols);
/* Same for a given format: FOS_DTYPE_MXFP4 (blocks of 32) pads columns to a multiple of 128. */
int64_t fos_padded_cols_for(int dtype, int64_t cols);

/* Bytes of device workspace fos_quantize needs for an [rows, cols] input (never 0). */
size_t fos_quantize_workspace_bytes(int64_t rows, int64_t cols);

/*
 * amax[0] = max |x| over a row-major matrix of x_type (FOS_T_BF16, FOS_T_F16 or FOS_T_F32)
 * elements (pass 1 of fos_quantize on its own).  Stands in for `x.abs().max().float()` of the reference quantizer
 * (src/fouroversix/quantize/pytorch/reference.py:573-578; the prologue kernel of the
 * native op, src/fouroversix/csrc/include/fp4_quant_kernel.h:195-215).  Same workspace
 * as fos_quantize.
 */
int fos_amax(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, float *amax,
             void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * Quantize a row-major matrix x[rows, cols] (leading dimension ld elements)
 * to packed 4-bit codes with one E4M3 scale per 1x16 block and one FP32 tensor scale.
 * Stands in for torch.ops.fouroversix.quantize (src/fouroversix/csrc/bindings.cpp:28,
 * csrc/quantize/fp4_quant.cu:99-239) with the semantics of the reference's PyTorch
 * backend (src/fouroversix/quantize/pytorch/backend.py:39-121,
 * quantize/pytorch/reference.py:555-679): the input is zero-padded to
 * (fos_padded_rows, fos_padded_cols) and every padded output element is written.
 *
 *   x_type      FOS_T_BF16; FOS_T_F16 and FOS_T_F32 (the reference converts its input with
 *               `.float()`, reference.py:577,593,596; its native op takes bf16 and fp16,
 *               csrc/quantize/fp4_quant.cu:134-136) give the same results; aligned fp16 rows
 *               with NVFP4 (1x16 blocks, round to nearest) or MXFP4 run at the bf16 kernels'
 *               speed, the other cases on element-wise kernels below it
 *   dtype       FOS_DTYPE_*; rule FOS_RULE_* (IF4 takes only the adaptive rules)
 *   round_style FOS_ROUND_*; seed/offset key the Philox dither of the stochastic styles
 *   block2d     non-zero: one scale and one decision per 16x16 tile
 *   sf_layout   FOS_SF_* layout of `sf`
 *   codes       u8 [rows_p, cols_p / 2], low nibble = even column
 *   sf          u8 [rows_p * cols_p / 16] E4M3 bytes (IF4: bit 7 marks integer blocks)
 *   amax        f32[1]; written with max|x| unless amax_is_input, in which case it is read
 *   workspace   >= fos_quantize_workspace_bytes(rows, cols) bytes, 256-byte aligned
 *
 * FOS_DTYPE_MXFP4 (src/fouroversix/quantize/pytorch/reference.py:149-181): E2M1 codes with
 * one E8M0 scale per 1x32 block, static rules and FOS_ROUND_NEAREST only, 1x32 blocks only;
 * columns are padded to a multiple of 128 (fos_padded_cols_for), `sf` holds
 * rows_p * cols_p / 32 bytes, amax is written with 1 (the format has no tensor scale) and
 * the workspace is not used.
 */
int fos_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                 int dtype, int rule, int round_style, int block2d,
                 uint64_t seed, uint64_t offset, int sf_layout,
                 uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                 void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * fos_quantize without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The pass-1 partial maxima go to an 8 KiB array that the
 * library holds in every GPU's memory for the life of the process; the call allocates and
 * frees nothing.  The array's address is looked up on the first call on each device (with
 * that device current), so make that first call outside a stream capture.  Every shape
 * fos_quantize accepts fits (its workspace never exceeds the array); a shape that would
 * not returns FOS_E_WORKSPACE.  All calls on one GPU share the array: calls that overlap
 * in time on one GPU (different streams, concurrently replayed graphs) race on it and must
 * be serialised by the caller.  Results are those of fos_quantize.
 */
int fos_quantize_static(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                        int dtype, int rule, int round_style, int block2d,
                        uint64_t seed, uint64_t offset, int sf_layout,
                        uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                        fos_stream_t stream);

/*
 * Pre-transform of the training-side quantize options: y = x^T (transpose != 0) and / or
 * the 16-point random Hadamard transform of every group of 16 consecutive row elements
 * (rht != 0; fixed sign vector), written as a row-major matrix y of x's type (x_type
 * FOS_T_BF16, FOS_T_F16 or FOS_T_F32; [cols, rows] when transposed, else [rows, cols]; leading dimension
 * ldy), and amax[0] = max |y|.  Stands in
 * for the `x.T` / `x.reshape(-1, 16) @ had` / `abs().max()` steps of the reference
 * quantizer (src/fouroversix/quantize/pytorch/reference.py:567-578,
 * quantize/utils.py:19-85; CUDA: csrc/include/hadamard_transform.h:16-37).  Follow it with
 * fos_quantize(y, ..., amax, amax_is_input = 1).  y is written in whole groups of 16: it is
 * 16-byte aligned and ldy a multiple of 8 that holds the output width rounded up to 16; a
 * group that reaches past the input's last row / column is completed with zeros (the
 * reference's zero padding, src/fouroversix/quantize/pytorch/backend.py:57-79), so with rht
 * the last group of a ragged width carries values in all 16 places.  x is read with 128-bit
 * loads when it is 16-byte aligned and ld a multiple of 8, element by element otherwise.
 * FOS_T_F32 (ldy a multiple of 4): the reference's fp32 product with the Hadamard matrix is a library matmul
 * whose summation order is not fixed; y equals the exact product to within four fp32 roundings of the
 * largest partial sum of a group.
 * Same workspace as fos_quantize.
 */
int fos_transform(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                  int transpose, int rht, void *y, int64_t ldy, float *amax,
                  void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * fos_transform followed by fos_quantize of its result, without the small kernel that reduces the
 * transform's per-workgroup maxima to one number in between: the quantizer's second pass reduces them
 * itself, as it does behind its own first pass.  y [out_rows, ldy] receives the transformed tensor (the
 * caller may discard it); codes / sf / amax are those of fos_quantize(y, ...) -- rows = cols of x when
 * transposing, width rounded up to 16 with rht -- byte for byte.  One workspace serves both steps.
 * FOS_DTYPE_NVFP4 and FOS_DTYPE_IF4.  Stands in for the transpose / rht options of
 * quantize_to_fp4 (src/fouroversix/quantize/pytorch/reference.py:567-578) in one call.
 */
int fos_transform_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                           int transpose, int rht, void *y, int64_t ldy,
                           int dtype, int rule, int round_style, int block2d,
                           uint64_t seed, uint64_t offset, int sf_layout,
                           uint8_t *codes, uint8_t *sf, float *amax,
                           void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * fos_quantize with the dither key of the stochastic styles read by the kernels from device memory:
 * key[0] = seed, key[1] = offset (8-byte aligned, read when the kernels run).  For launches recorded into a
 * HIP graph, whose scalar arguments are frozen at capture: the caller advances key[1] between replays (a
 * small kernel of its own, recorded with the rest) and every replay rounds with fresh bits.  Same results
 * as fos_quantize called with the values the key holds.  No counterpart in the reference, whose kernels take
 * their random bits as launch arguments (src/fouroversix/csrc/quantize/fp4_quant.cu:134-136).
 */
int fos_quantize_devkey(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                        int dtype, int rule, int round_style, int block2d,
                        const uint64_t *key, int sf_layout,
                        uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                        void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * Fused quantize -> dequantize round trip: out[rows, cols] (bf16, leading dimension ldo) =
 * the values fos_dequantize would return for fos_quantize's result, without materialising
 * codes or scales.  Stands in for QuantizeBackendBase.pseudo_quantize
 * (src/fouroversix/quantize/backend.py:213-234; fused Triton kernel
 * src/fouroversix/kernels/triton/ops.py:212-374).  Arguments as fos_quantize; out has x's element
 * type.  Fused kernels exist for the combinations fos_pseudo_quantize_is_fused names, with x and out
 * 16-byte aligned, ld and ldo multiples of 8 and cols a multiple of 16; anything else returns
 * FOS_E_UNSUPPORTED (compose fos_quantize and fos_dequantize instead).
 */
int fos_pseudo_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                        int dtype, int rule, int round_style, int block2d,
                        void *out, int64_t ldo, float *amax, int amax_is_input,
                        void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * fos_pseudo_quantize with the dither key of the stochastic rounding styles (seed, offset as in
 * fos_quantize; fos_pseudo_quantize uses 0, 0): the output is bit for bit what fos_dequantize returns for
 * fos_quantize's result under the same key.  The reference's fused kernel draws its random bits inside
 * the kernel (src/fouroversix/kernels/triton/ops.py:212-374); here the caller holds the key.
 */
int fos_pseudo_quantize_keyed(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                              int dtype, int rule, int round_style, int block2d, uint64_t seed, uint64_t offset,
                              void *out, int64_t ldo, float *amax, int amax_is_input,
                              void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * 1 when a fused kernel exists for this element type (FOS_T_*), format, selection rule, rounding style and
 * block shape (alignment aside), else 0: FOS_DTYPE_NVFP4 with FOS_ROUND_NEAREST on bf16 (either block
 * shape) and fp16 (1x16 blocks); FOS_DTYPE_NVFP4 with FOS_ROUND_STOCHASTIC on bf16, either block shape (the
 * unbiased style with the MSE and static rules); FOS_DTYPE_IF4 with FOS_RULE_MSE on bf16, round to nearest,
 * 1x16 blocks.  Pure host function.
 */
int fos_pseudo_quantize_is_fused(int x_type, int dtype, int rule, int round_style, int block2d);

/*
 * D[M, N] = alpha * sum_k (A[m,k] * sfA[m,k/16]) * (B[n,k] * sfB[n,k/16]), FP32
 * accumulation, written as out_type (FOS_T_BF16 or FOS_T_F16) with leading dimension ldd.
 * Stands in for torch.ops.fouroversix.gemm_nvfp4nvfp4_accum_fp32_out_{bf16,fp16}_tnt
 * (src/fouroversix/csrc/bindings.cpp:31-33, csrc/fp4_gemm.cu:40-154).
 *   A  u8 [M, K/2], B u8 [N, K/2]: packed E2M1, low nibble = even k
 *   sfA, sfB  E4M3 bytes in the FOS_SF_TILED_128X4 layout of [M, K/16] / [N, K/16]
 *   alpha f32[1] on the device
 * N must be a multiple of 128 and K of 64, and M a multiple of 128 (the padded shapes that
 * fos_quantize produces); D 16-byte aligned and ldd a multiple of 8 (8-byte aligned and a
 * multiple of 4 suffice for M <= 128).  M < 128 is also accepted when K is a multiple of 256: A then
 * holds M rows, sfA the full 128-row band of the tiled layout, and only M rows of D are
 * written (decode-sized batches skip the work on the padding rows).
 *   workspace  optional (may be NULL): fos_gemm_workspace_bytes(M, N, K) bytes, 16-byte
 *              aligned.  With it, shapes with few output tiles (small M) split the K
 *              dimension over several workgroups and reduce FP32 partial tiles in a fixed
 *              order (deterministic); without it they run unsplit, only slower.
 */
int fos_gemm_nvfp4(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                   const float *alpha, int64_t M, int64_t N, int64_t K,
                   void *D, int out_type, int64_t ldd,
                   void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * fos_gemm_nvfp4 with the output scale formed inside the kernel from the operands' tensor
 * maxima: alpha = (amax_a[0] * amax_b[0]) * f32(1 / denominator), the value fos_gemm_alpha
 * writes (src/fouroversix/matmul/cutlass/backend.py:86-98), without that launch.
 * amax_a / amax_b are device f32[1], e.g. the `amax` outputs of fos_quantize.
 */
int fos_gemm_nvfp4_amax(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                        const float *amax_a, const float *amax_b, double denominator,
                        int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd,
                        void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * fos_gemm_nvfp4_amax that also folds max|D| -- of the values as stored, in the output type --
 * into d_amax[0] (device f32[1]): every wavefront does an unsigned atomic max on the value's
 * bits, so the caller sets d_amax[0] to 0 before the call (or leaves an earlier maximum there to
 * extend it).  A NaN among the outputs is recorded as NaN (its bits lie above every number's), as the
 * reference's `x.abs().max()` would report it.  The next layer's activation quantization can then take d_amax as its
 * `amax` input (amax_is_input = 1) and skip its own pass over D.  No counterpart in the
 * reference, whose quantize op always reduces its input
 * (src/fouroversix/quantize/pytorch/reference.py:573-600).
 */
int fos_gemm_nvfp4_amax_out(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                            const float *amax_a, const float *amax_b, double denominator,
                            int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd, float *d_amax,
                            void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * The product of a linear layer in one launch: fos_gemm_nvfp4_amax_out with an optional bias (N values of
 * the output type, 8-byte aligned, or NULL) and an optional d_amax (NULL: not recorded).  With a bias,
 * D = RN(RN(alpha * acc) + bias[n]): the product rounded to the output type, then the sum rounded again --
 * the two roundings of `out = quantized_matmul(...); out = out + bias` in the reference's layer
 * (src/fouroversix/model/modules/linear.py:83-92) -- and d_amax receives max|D| of that sum, so that a layer
 * with a bias hands its output maximum on like one without.
 */
int fos_gemm_nvfp4_linear(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                          const float *amax_a, const float *amax_b, double denominator,
                          int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd, const void *bias,
                          float *d_amax, void *workspace, size_t workspace_bytes, fos_stream_t stream);

/*
 * alpha[0] = (amax_a[0] * amax_b[0]) * f32(1 / denominator), in fp32 on the device: the
 * GEMM's output scale as src/fouroversix/matmul/cutlass/backend.py:86-98 forms it on a GPU
 * (torch divides a tensor by a host scalar through the reciprocal, taken in double and
 * rounded to fp32; denominator = the product of both operands' qmax * smax * rounding
 * adjustment), in one launch.
 */
int fos_gemm_alpha(const float *amax_a, const float *amax_b, double denominator, float *alpha,
                   fos_stream_t stream);

/* Bytes of workspace with which fos_gemm_nvfp4 runs this shape fastest (0 = none needed).
 * The reference's op runs CUTLASS without a workspace
 * (src/fouroversix/csrc/fp4_gemm.cu:148-151), so this has no counterpart there. */
size_t fos_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * MXFP4 counterpart of fos_gemm_nvfp4: D = alpha * sum_k (A 2^(sfA-127)) (B 2^(sfB-127)) on
 * the native scaled FP4 matrix instruction.  Stands in for
 * torch.ops.fouroversix.gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt
 * (src/fouroversix/csrc/bindings.cpp:26-35, src/fouroversix/matmul/cutlass/backend.py:79-110).
 *   A u8 [M, K/2], B u8 [N, K/2]; sfA, sfB E8M0 bytes in the FOS_SF_TILED_128X4 layout of
 *   [M, K/32] / [N, K/32]; M, N, K multiples of 128 (the padded shapes fos_quantize produces).
 *   D bf16 / fp16 [M, ldd], 16-byte aligned, ldd a multiple of 8 (rows are stored 16 bytes per lane).
 */
int fos_gemm_mxfp4(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                   const float *alpha, int64_t M, int64_t N, int64_t K,
                   void *D, int out_type, int64_t ldd, fos_stream_t stream);

/*
 * out[rows, cols] = dequantized values of a quantized tensor, cropped to (rows, cols).
 * Stands in for QuantizeBackendBase.dequantize (src/fouroversix/quantize/backend.py:89-160).
 *   codes u8 [rows_p, cols_p/2], sf in sf_layout over [rows_p, cols_p/16], amax f32[1]
 *   divisor = qmax * smax * adjustment of the tensor's scale rule and rounding style
 *   out_type FOS_T_BF16 / FOS_T_F16 / FOS_T_F32, leading dimension ldo
 *   intermediate_type FOS_T_F16 (the reference's default) or FOS_T_F32: the type in which
 *   value and block scale are multiplied (`intermediate_dtype`); it matters for IF4's
 *   integer blocks (factor 6/7) and for MXFP4 scales outside fp16's range
 * FOS_DTYPE_MXFP4: blocks of 32, E8M0 scales, amax and divisor are ignored (amax may be NULL).
 */
int fos_dequantize(const uint8_t *codes, const uint8_t *sf, const float *amax,
                   int dtype, int sf_layout, double divisor,
                   int64_t rows, int64_t cols, int64_t rows_p, int64_t cols_p,
                   void *out, int out_type, int64_t ldo, int intermediate_type, fos_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FOUROVERSIX_HIP_H */
