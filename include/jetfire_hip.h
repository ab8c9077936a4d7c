/*
 * jetfire_hip.h -- C ABI of libjetfire_hip.so: the gfx950 (MI355X) implementation of the
 * Jetfire per-block INT8 data-flow path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; nothing here allocates, frees,
 *     synchronises or copies to the host.  Work is enqueued on `stream` (a hipStream_t passed
 *     as void*; NULL = the default stream).
 *   - return value: 0 on success, a negative JF_ERR_* for a rejected argument, a positive
 *     hipError_t if the launch failed.  jf_error_string() names either.
 *   - a "block tensor" is (q: int8 [R,C] row-major, s: scale [R/32, C/32] row-major), x ~= q*s.
 *     All of R, C, M, N, K must be positive multiples of 32.  Data pointers must be 16-byte aligned, scale pointers
 *     aligned to their element type (2 or 4 bytes); exactly the elements of a scale array are read, nothing beyond.
 *   - `scale_dtype` selects the element type of EVERY scale pointer of the call
 *     (JF_SCALE_F16 = IEEE binary16, what the reference stores; JF_SCALE_F32 = binary32).
 *   - GEMM scale operands are K-major (JF_SCALES_KMAJOR): sa[kb*(M/32)+mb], sb[kb*(N/32)+nb], or, per operand, the
 *     block tensor's own row-major scale array (JF_SCALES_ROWMAJOR): sa[mb*(K/32)+kb]; output scales are
 *     sc[mb*(N/32)+nb]  (reference: …/igemm/igemm_BlockSquare32OutputIntQuantizeBiasRowCol.cu:110-111,
 *     187-188, 297-304; paths below are relative to JetfireGEMMKernel/BlockQuantize/cpp_extension/).
 *   - stochastic rounding draws Philox4x32 noise keyed by (seed, offset + flat output index / 8), 16 bits per
 *     element, so results do not depend on the launch geometry.  The round count is a build-time choice
 *     (JF_PHILOX_ROUNDS: 7 by default, 10 = the count of the reference's generators); jf_philox_rounds() reports it.
 */
#ifndef JETFIRE_HIP_H
#define JETFIRE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JF_OK                 0
#define JF_ERR_NULL          -1   /* a required pointer is NULL                      */
#define JF_ERR_SHAPE         -2   /* a dimension is not a positive multiple of 32    */
#define JF_ERR_ENUM          -3   /* unknown layout / dtype / rounding / approx code */
#define JF_ERR_ALIGN         -4   /* pointer or leading dimension not 16-byte aligned */
#define JF_ERR_WORKSPACE     -5   /* workspace missing or smaller than required      */
#define JF_ERR_DEVICE        -6   /* the current device is not gfx950                */
#define JF_ERR_UNSUPPORTED   -7   /* valid codes, but this combination of layouts is not implemented */
#define JF_ERR_SCRATCH_LIMIT -8   /* jf_igemm_block_fp_noalloc: the K split needs more than JF_NOALLOC_SCRATCH_BYTES */

/* A operand layout of jf_igemm_block_fp (every other GEMM entry point takes A as [M,K]) */
#define JF_A_MK 0                 /* A is [M,K] row-major                                                          */
#define JF_A_KM 1                 /* A is [K,M] row-major: the un-transposed gradient [tokens, C_out] of a weight
                                     gradient; implemented together with JF_B_KN (else JF_ERR_UNSUPPORTED)         */

/* B operand layout of the GEMMs */
#define JF_B_NK 0                 /* B is [N,K] row-major ("row x col", forward)      */
#define JF_B_KN 1                 /* B is [K,N] row-major ("row x row", dgrad, wgrad) */

#define JF_SCALE_F16 0
#define JF_SCALE_F32 1

/* Where the scale of block (row block r, K block kb) of a GEMM operand lives */
#define JF_SCALES_KMAJOR   0      /* s[kb*(rows/32) + r]: what the reference kernels take (callers transpose)        */
#define JF_SCALES_ROWMAJOR 1      /* s[r*(K/32) + kb]: the block tensor's own scale array, no transposed copy needed */

#define JF_FP_F16  0
#define JF_FP_F32  1
#define JF_FP_BF16 2

#define JF_ROUND_NEAREST    0     /* ties-to-even                                    */
#define JF_ROUND_STOCHASTIC 1
#define JF_ROUND_TRUNC      2     /* toward zero (the add kernels of the reference)   */
#define JF_ROUND_STOCHASTIC_TRUNC 3

#define JF_GELU_ERF  0
#define JF_GELU_TANH 1

typedef void *jf_stream_t;

const char *jf_error_string(int code);

/* Rounds of the Philox4x32 generator this library was built with (reference: curandStatePhilox4_32_10 at
 * igemm/igemm_BlockSquare32OutputIntQuantizeStochastic.cu:311, 10 rounds). */
int jf_philox_rounds(void);

/* Bytes of device scratch the GEMM entry points need for this problem: 0 for both layouts (a JF_B_KN operand is
 * staged as it lies in memory and transposed by the LDS read).  The workspace arguments of jf_igemm_s32,
 * jf_igemm_block_acc and jf_igemm_block_q are kept for callers written against an implementation that re-lays B out
 * first; they are ignored and may be NULL / 0. */
size_t jf_igemm_workspace_bytes(int M, int N, int K, int b_layout);

/* C_s32[M,N] = A[M,K] * B.   Replaces igemm_basic_int8_gemm (include/igemm.h:3-12,
 * igemm/igemm_BasicInt8Gemm.cu:113-140). */
int jf_igemm_s32(const int8_t *A, const int8_t *B, int32_t *C, int M, int N, int K, int b_layout,
                 void *workspace, size_t workspace_bytes, jf_stream_t stream);

/* acc[kb][M][N] (int32) = A[:, 32kb:32kb+32] * B[32kb:32kb+32, :] for every K block: the per-block
 * INT32 accumulators (frag_intc at …BiasRowCol.cu:209-211) made observable for parity tests. */
int jf_igemm_block_acc(const int8_t *A, const int8_t *B, int32_t *acc, int M, int N, int K, int b_layout,
                       void *workspace, size_t workspace_bytes, jf_stream_t stream);

/* C_fp[M,N] = sum_kb sa*sb*(A_kb*B_kb), fp32 accumulate in ascending kb, stored as out_dtype.
 * Replaces igemm_output_fp_no_quantize (include/igemm.h:14-25, igemm/igemm_BlockSquare32OutputFp.cu:340-382).
 * With a_layout = JF_A_KM the weight gradient dW = dY^T X is computed from dY [tokens, C_out] as it lies in memory:
 * the reference's callers materialise dY^T first (Linear/linear_bwd.py:21, Nonlinear/transpose.py:69-97).
 *
 * splitk: 1 = one accumulation chain over all of K per output (the reference's arithmetic, bit for bit).
 * n > 1 = K is cut into up to n parts of whole multiples of 4 K blocks (at least 16 K blocks each); every part is
 * accumulated as above into an fp32 partial result, and the partial results are added in ascending order before the
 * conversion to out_dtype: the result differs from splitk = 1 only in the rounding of those last additions.  For
 * weight gradients with few output tiles and a deep K (GPT-2 small: 768 x 768 outputs over 12288 tokens = 36 tiles
 * for 256 CUs; the reference runs the same under-filled grid, igemm_BlockSquare32OutputFp.cu:346-352) it fills the
 * GPU.  0 = the library picks n from the tile count.  jf_igemm_splitk_plan reports the parts actually used (so a
 * checker can reproduce the arithmetic), jf_igemm_block_fp_workspace_bytes the scratch needed (0 for one part). */
int jf_igemm_splitk_plan(int M, int N, int K, int splitk, int *splits, int *kb_per_split);
size_t jf_igemm_block_fp_workspace_bytes(int M, int N, int K, int b_layout, int splitk);
int jf_igemm_block_fp(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C,
                      int M, int N, int K, int a_layout, int b_layout, int scale_dtype, int sa_layout, int sb_layout,
                      int out_dtype, int splitk, void *workspace, size_t workspace_bytes, jf_stream_t stream);

/* jf_igemm_block_fp for callers that cannot allocate or pass device scratch: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same arithmetic and the
 * same bits as jf_igemm_block_fp with the same splitk request, minus the workspace: the fp32 partial results of the K
 * split live in a buffer built into the library (JF_NOALLOC_SCRATCH_BYTES per GPU the library runs on, held until the
 * process ends).  Calls nothing that allocates or frees -- with one proviso: the HIP runtime loads a library's device
 * code (and with it this buffer) on the first call into the library on a device, so make one warm-up call of any
 * entry point on that device before a capture or an allocation-free region begins.  A problem whose K split needs more scratch
 * (parts * M * N * 4 bytes, see jf_igemm_splitk_plan) is refused with JF_ERR_SCRATCH_LIMIT; splitk = 1 never needs any.
 * All calls on one GPU share that GPU's buffer: two calls that may overlap on one GPU (different streams, or threads
 * without ordering between them) race on it and must be serialised by the caller. */
#define JF_NOALLOC_SCRATCH_BYTES (64u << 20)
int jf_igemm_block_fp_noalloc(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C,
                              int M, int N, int K, int a_layout, int b_layout, int scale_dtype, int sa_layout,
                              int sb_layout, int out_dtype, int splitk, jf_stream_t stream);

/* (C_s8[M,N], sc[M/32,N/32]) = per-32x32-block requantisation of the same accumulation.
 *   rounding JF_ROUND_NEAREST : q = clamp(rn(127*(acc+bias[n]) / (amax+biasmax)), +-127)
 *       replaces igemm_output_int_quantize_bias_rowcol / _rowrow / igemm_output_int_quantize
 *       (include/igemm.h:40-51,53-77; igemm/…BiasRowCol.cu:386-434; …IntQuantize.cu)
 *   rounding JF_ROUND_STOCHASTIC : q = clamp(rn(127*acc/amax + noise), +-127)
 *       replaces igemm_output_int_quantize_stochastic (include/igemm.h:79-90; …Stochastic.cu:372-419)
 * bias ([N] fp32) and biasmax ([1] fp32, device) may be NULL (= zeros). */
int jf_igemm_block_q(const int8_t *A, const int8_t *B, const void *sa, const void *sb,
                     const float *bias, const float *biasmax, int8_t *C, void *sc,
                     int M, int N, int K, int b_layout, int scale_dtype, int sa_layout, int sb_layout, int rounding,
                     uint64_t seed, uint64_t offset,
                     void *workspace, size_t workspace_bytes, jf_stream_t stream);

/* The forward GEMM (A [M,K], B [N,K], round-to-nearest) with the GELU forward fused into its epilogue: (C, sc) is what
 * jf_igemm_block_q writes, (C_gelu, sc_gelu) is what jf_gelu_fwd would make of it (bit for bit, including the scale
 * as stored in scale_dtype), without the second pass over HBM.  Replaces the pair igemm_output_int_quantize_bias_rowcol
 * (include/igemm.h:66-77) + int8_gelu_forward (Jetfire/Nonlinear/gelu_fwd.py:128-162) of the recipe's MLP
 * (INT8_GPT2/qmodel.py:210-214), which needs both tensors: the first for the backward pass, the second as the input
 * of the next layer. */
int jf_igemm_block_q_gelu(const int8_t *A, const int8_t *B, const void *sa, const void *sb, const float *bias,
                          const float *biasmax, int8_t *C, void *sc, int8_t *C_gelu, void *sc_gelu, int M, int N, int K,
                          int scale_dtype, int sa_layout, int sb_layout, int gelu_approx, float gelu_amax_eps,
                          jf_stream_t stream);

/* The activation-gradient GEMM (A = dY [M,K], B = W [K,N], stochastic rounding with (seed, offset)) with the GELU
 * backward fused into its epilogue: (C, sc) is what jf_gelu_bwd(Xq, Xs, <the GEMM's requantised output>, ...,
 * gelu_rounding, gelu_seed, gelu_offset) would return, bit for bit (the intermediate gradient is requantised to INT8
 * with its scale rounded to scale_dtype exactly as jf_igemm_block_q stores it, but never written).  (Xq, Xs): the
 * GELU's forward input, an [M,N] block tensor.  Replaces the pair igemm_output_int_quantize_stochastic
 * (include/igemm.h:79-90) + int8_gelu_backward (Jetfire/Nonlinear/gelu_bwd.py:173-215) of the recipe's MLP backward
 * (INT8_GPT2/qmodel.py:249-253), whose intermediate gradient has no other reader. */
int jf_igemm_block_q_gelu_bwd(const int8_t *A, const int8_t *B, const void *sa, const void *sb, const int8_t *Xq,
                              const void *Xs, int8_t *C, void *sc, int M, int N, int K, int scale_dtype, int sa_layout,
                              int sb_layout, int gelu_approx, uint64_t seed, uint64_t offset, int gelu_rounding,
                              uint64_t gelu_seed, uint64_t gelu_offset, jf_stream_t stream);

/* jf_igemm_block_q with the dequantisation of its result fused into the epilogue: out[M,N] (out_dtype: JF_FP_*) =
 * codes x scales of the block tensor jf_igemm_block_q would have stored (scales rounded to scale_dtype as it stores
 * them), i.e. what jf_dequantize of that result returns, bit for bit; the INT8 tensor itself is never written.
 * Replaces the reference's unquantised-output path, which runs the quantising GEMM and multiplies codes by scales in a
 * second pass: int8_linear_forward(..., output_quantized=False) (Jetfire/Linear/linear_fwd.py:22-32; the QKV projection,
 * INT8_GPT2/qmodel.py:103) and int8_linear_backward(..., dgrad_quantize=False) (Jetfire/Linear/linear_bwd.py:17-29; the
 * activation gradient of the attention output projection, INT8_GPT2/qmodel.py:168). */
int jf_igemm_block_q_dequant(const int8_t *A, const int8_t *B, const void *sa, const void *sb, const float *bias,
                             const float *biasmax, void *out, int M, int N, int K, int b_layout, int scale_dtype,
                             int sa_layout, int sb_layout, int out_dtype, int rounding, uint64_t seed, uint64_t offset,
                             jf_stream_t stream);

/* Block quantise x[R,C] (x_dtype: JF_FP_*) -> (q, s); optionally also qT[C,R] = q transposed.
 * Replaces int8_quantize (Jetfire/Nonlinear/quantize.py:128-164) and, with qT != NULL,
 * int8_quantize_transpose (Jetfire/Nonlinear/quantize_transpose.py:131-171). */
int jf_quantize(const void *x, int x_dtype, int R, int C, int8_t *q, void *s, int8_t *qT,
                int scale_dtype, int rounding, uint64_t seed, uint64_t offset, float amax_eps,
                jf_stream_t stream);

/* jf_quantize of a tensor that exists only as column slabs lying side by side: slab k is x[k], [R, widths[k]] with rows
 * ldx[k] elements apart (nslabs <= 4; x, ldx, widths are HOST arrays); (q, s) is the block tensor of the concatenation,
 * [R, sum of widths].  Rounding noise is drawn by position in the result, so the codes are those jf_quantize gives for
 * the concatenated tensor.  No counterpart in the reference, which quantises the concatenated gradient of the attention
 * kernel's three inputs (INT8_GPT2/qmodel.py:112-120 behind autograd's cat); here the three gradients are read where
 * they lie and the 78 MB concatenation is never made. */
int jf_quantize_slabs(const void *const *x, const int *ldx, const int *widths, int nslabs, int x_dtype, int R,
                      int8_t *q, void *s, int scale_dtype, int rounding, uint64_t seed, uint64_t offset, float amax_eps,
                      jf_stream_t stream);

/* out[R,C] = q*s, the fp32 product rounded to `out_dtype` (JF_FP_F32 / JF_FP_F16 / JF_FP_BF16; for binary16 scales and
 * output this equals the reference's binary16 multiplication).  Replaces int8_dequantize
 * (Jetfire/Nonlinear/dequantize.py:86-116) and the dequantisation int8_linear_forward does on its unquantised-output
 * path (Jetfire/Linear/linear_fwd.py:29-31). */
int jf_dequantize(const int8_t *q, const void *s, int R, int C, int scale_dtype, void *out, int out_dtype,
                  jf_stream_t stream);

/* out[C,R] = in[R,C].  Replaces int8_transpose (Jetfire/Nonlinear/transpose.py:69-97). */
int jf_transpose_s8(const int8_t *in, int R, int C, int8_t *out, jf_stream_t stream);

/* Per-row mean and 1/sqrt(var+eps) of a block tensor (the statistics LayerNorm takes as inputs;
 * the reference gets them from add_mean_var.py:219-221 or qmodel.py:429-430). */
int jf_rowstats(const int8_t *q, const void *s, int R, int C, int scale_dtype, float eps,
                float *mean, float *rstd, jf_stream_t stream);

/* dequant -> (x-mean)*rstd*gamma + beta -> requant.  beta may be NULL.
 * Replaces int8_layernorm_forward (Jetfire/Nonlinear/layernorm.py:430-465). */
int jf_layernorm_fwd(const int8_t *q, const void *s, const float *gamma, const float *beta,
                     const float *mean, const float *rstd, int R, int C, int scale_dtype,
                     int8_t *qy, void *sy, jf_stream_t stream);

/* Bytes of scratch for jf_layernorm_bwd. */
size_t jf_layernorm_bwd_workspace_bytes(int R, int C);

/* LayerNorm backward over full rows: (qdx, sdx) requantised dx, dgamma[C], dbeta[C] (either may be NULL).
 * Replaces int8_layernorm_backward (Jetfire/Nonlinear/layernorm.py:467-526). */
int jf_layernorm_bwd(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg,
                     const float *gamma, const float *mean, const float *rstd, int R, int C,
                     int scale_dtype, int rounding, uint64_t seed, uint64_t offset,
                     int8_t *qdx, void *sdx, float *dgamma, float *dbeta,
                     void *workspace, size_t workspace_bytes, jf_stream_t stream);

/* jf_layernorm_bwd followed by jf_add(x1, dx codes, dx scales) in one kernel, for rows of up to 2048 columns
 * (JF_ERR_SHAPE beyond: make the two calls): dx is requantised with (rounding, seed, offset) exactly as jf_layernorm_bwd
 * does, read back as codes x the stored scale, added to x1, and the sum (y1, in y1_dtype) and its block quantisation
 * (q, s; add_rounding, add_seed, add_offset) are what is written -- bit for bit what the two calls write, without dx's
 * round trip through memory.  dx itself is not stored.  Workspace as for jf_layernorm_bwd.
 * Replaces the pair int8_layernorm_backward + int8_add_Ifp_Ig16_Ofp_Og of the reference's recipe
 * (INT8_GPT2/qmodel.py:125-128 and :258-261; Jetfire/Nonlinear/layernorm.py:467-526, add.py:164-211). */
int jf_layernorm_bwd_add(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg,
                         const float *gamma, const float *mean, const float *rstd, int R, int C,
                         int scale_dtype, int rounding, uint64_t seed, uint64_t offset,
                         const void *x1, int x1_dtype, int add_rounding, uint64_t add_seed, uint64_t add_offset,
                         void *y1, int y1_dtype, int8_t *q, void *s, float *dgamma, float *dbeta,
                         void *workspace, size_t workspace_bytes, jf_stream_t stream);

/* dequant -> GELU -> requant (amax_eps is added to the block amax: 5e-5 in the reference).
 * Replaces int8_gelu_forward (Jetfire/Nonlinear/gelu_fwd.py:128-162). */
int jf_gelu_fwd(const int8_t *q, const void *s, int R, int C, int scale_dtype, int approx,
                float amax_eps, int8_t *qy, void *sy, jf_stream_t stream);

/* dequant(x), dequant(g) -> gelu'(x)*g -> requant.
 * Replaces int8_gelu_backward (Jetfire/Nonlinear/gelu_bwd.py:173-215). */
int jf_gelu_bwd(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg, int R, int C,
                int scale_dtype, int approx, int rounding, uint64_t seed, uint64_t offset,
                int8_t *qy, void *sy, jf_stream_t stream);

/* y = x1 + q2*s2 in fp32, (q, s) = block quantisation of y; optional per-row, per-32-column partial
 * sums of y and y^2 (rowsum, rowsq: [C/32, R] fp32 -- part-major, so that a block's 32 rows are one contiguous store;
 * may be NULL).  y1 receives y in y1_dtype (JF_FP_F32: as the reference's kernels write it; JF_FP_F16 / JF_FP_BF16: y
 * rounded to nearest even, i.e. the kernel followed by the cast the reference's recipe applies to it,
 * INT8_GPT2/qmodel.py:228, without the fp32 tensor in between).  The quantisation and the partial sums always use the
 * fp32 y.
 * Replaces int8_add_Ifp_Ig16_Ofp_Og (Jetfire/Nonlinear/add.py:164-211) and
 * int8_add_Ifp_Ig16_Ofp_Og_MeanVar (Jetfire/Nonlinear/add_mean_var.py:179-230). */
int jf_add(const void *x1, int x1_dtype, const int8_t *q2, const void *s2, int R, int C,
           int scale_dtype, int rounding, uint64_t seed, uint64_t offset,
           void *y1, int y1_dtype, int8_t *q, void *s, float *rowsum, float *rowsq, jf_stream_t stream);

/* out[c] = sum over all rows of q[r,c] * s[r/32,c/32] (fp32): the column sums of a block tensor, i.e. the bias gradient
 * of a linear layer from its quantised output gradient (sketched in the reference as G8.sum(0),
 * JetfireGEMMKernel/BlockQuantize/QBlockLinear.py:63-66).  Arithmetic, in a fixed order: per 32-row strip rb the term
 * float(exact integer sum of the strip's 32 codes of column c) * s[rb, c/32]; lane g of 32 adds the terms of strips
 * g, g+32, ... in ascending order starting from +0; the 32 partial sums are added in ascending g.
 * workspace: jf_block_colsum_workspace_bytes(R, C) bytes of device scratch (the strip terms). */
size_t jf_block_colsum_workspace_bytes(int R, int C);
int jf_block_colsum(const int8_t *q, const void *s, int R, int C, int scale_dtype, float *out, void *workspace,
                    size_t workspace_bytes, jf_stream_t stream);

/* mean[r] = (sum of rowsum[0..parts-1, r], ascending) / C;  rstd[r] = 1 / sqrt((sum of rowsq[:, r]) / C - mean[r]^2)
 * (no epsilon): the finishing step of int8_add_Ifp_Ig16_Ofp_Og_MeanVar (Jetfire/Nonlinear/add_mean_var.py:219-221), which
 * the reference computes with torch operators on the kernel's partial sums.  rowsum, rowsq: [parts, R] fp32 as written by
 * jf_add. */
int jf_rowstats_finish(const float *rowsum, const float *rowsq, int R, int parts, int C, float *mean, float *rstd,
                       jf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* JETFIRE_HIP_H */
