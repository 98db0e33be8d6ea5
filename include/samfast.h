/*
 * samfast - C ABI of the MI355X (gfx950) SAM image-encoder hot path.
 *
 * Two groups of entry points:
 *   attention with decomposed relative-position bias (global 64-wide grids and
 *   small windows), and dynamic symmetric int8 linears (row quantiser, int8
 *   GEMM with int32 accumulators, fused scale+bias epilogue).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless named host_*; the caller owns
 *     all buffers, nothing is retained after the call returns;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); calls
 *     only enqueue work, they never synchronise and never allocate;
 *   - strides are in ELEMENTS; the innermost (head_dim / K) axis is contiguous
 *     and every row start must be 16-byte aligned;
 *   - return value 0 = ok; negative = SAMFAST_E_*; the text of the last error
 *     on the calling thread is returned by samfast_last_error();
 *   - a call with no rows (M == 0) or no images (B == 0) is valid: the shape is
 *     checked, nothing is launched, 0 is returned, and the buffers that would
 *     hold those rows may be NULL (an empty tensor's data pointer).
 *
 * The reference interfaces each entry point stands in for are cited as
 * file:line under segment_anything_fast/ of pytorch-labs/segment-anything-fast.
 */
#ifndef SAMFAST_H
#define SAMFAST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SAMFAST_VERSION 1

/* element types (`dtype` arguments).  The attention entry points take both, as the reference's
 * operator does (flash_4.py:188,348); the int8 linears read and write bf16 only and return
 * SAMFAST_E_UNSUPPORTED for anything else. */
#define SAMFAST_BF16 0
#define SAMFAST_F16 1

#define SAMFAST_OK 0
#define SAMFAST_E_INVALID (-1)      /* bad shape / stride / alignment / null pointer */
#define SAMFAST_E_UNSUPPORTED (-2)  /* a shape or type no kernel here covers */
#define SAMFAST_E_LAUNCH (-3)       /* the HIP runtime refused the launch */

/*
 * Layouts of an int8 GEMM operand with R rows and K columns (activations xq: R = M; dense
 * weights wq: R = N):
 *   ROWMAJOR  (R, K), element (r, k) at r*K + k - what torch._int_mm takes;
 *   KB64      K-block major, (K/64, R, 64): element (r, k) at ((k/64)*R + r)*64 + k%64, so the
 *             64-byte k tile of consecutive rows is contiguous memory and the GEMM reads whole
 *             cache lines.  K % 64 == 0.  The quantisers can write it, the fused GEMMs read it.
 */
#define SAMFAST_LAYOUT_ROWMAJOR 0
#define SAMFAST_LAYOUT_KB64 1

int samfast_version(void);
/* "gfx950" - the only architecture the code objects are built for */
const char* samfast_arch(void);
const char* samfast_last_error(void);

/*
 * out = softmax(q k^T * sm_scale + rel_h[.., kh] + rel_w[.., kw]) v, the bias
 * computed inside the kernel from the two relative-position tables:
 *   rel_h[b,h,(y,x),j] = <q[b,h,(y,x),:], rel_pos_h[y - j + gh - 1, :]>
 *   rel_w[b,h,(y,x),j] = <q[b,h,(y,x),:], rel_pos_w[x - j + gw - 1, :]>
 * Replaces, in one launch: add_decomposed_rel_pos (modeling/image_encoder.py:338-372,
 * called at :234) + _attention_rel_h_rel_w (flash_4.py:335-370, called at
 * modeling/image_encoder.py:245), for both the global (gh=gw=64) and the windowed
 * (gh=gw=14) blocks.
 *
 * q,k,v,out: logical shape (B, nH, N=gh*gw, hd), addressed as
 *   ptr + b*s_b + h*s_h + n*s_n + d, so head-major (B,nH,N,hd) tensors and the
 *   token-major output of the qkv Linear ((B,N,3,nH,hd)) are both accepted
 *   without a copy.
 * rel_pos_h: (2*gh-1, hd) contiguous, rel_pos_w: (2*gw-1, hd) contiguous, same
 *   element type as q.
 * Supported: hd in {64, 80}; (gw == 64 and N % 128 == 0) or (gh <= 15 and
 *   gw <= 16 and N <= 208); dtype SAMFAST_BF16 or SAMFAST_F16 (q, k, v, out and the tables
 *   all of that type; accumulation, softmax and bias in fp32 either way).
 * Range of the bias in the window kernels: the two factors <q, rel_pos row> travel through the
 *   matrix cores as 16-bit values already divided by sm_scale, so they carry the element type's
 *   resolution and, for SAMFAST_F16, must satisfy |<q, rel_pos row>| < 65504 * sm_scale (about
 *   7300 at head_dim 80, where the reference's fp16 einsum itself overflows at 65504); padding
 *   keys are masked with a score of -60000 / sm_scale, so real scores have to stay well above that.
 *   The global kernels keep the factors in fp32 and have no such limit.
 */
int samfast_attn_relpos_fwd(
    const void* q, const void* k, const void* v,
    const void* rel_pos_h, const void* rel_pos_w, void* out,
    int B, int nH, int gh, int gw, int hd,
    int64_t q_sb, int64_t q_sh, int64_t q_sn,
    int64_t k_sb, int64_t k_sh, int64_t k_sn,
    int64_t v_sb, int64_t v_sh, int64_t v_sn,
    int64_t o_sb, int64_t o_sh, int64_t o_sn,
    int dtype, float sm_scale, void* stream);

/*
 * Windowed attention on image-ordered tokens: window_partition, the attention of every
 * window and window_unpartition (modeling/image_encoder.py:169-178, helpers :273-323) in one
 * launch, without materialising the padded windows.  q, k, v, out are (B, nH, img_h*img_w, hd)
 * views addressed like samfast_attn_relpos_fwd with n = y*img_w + x; the image is cut into
 * ceil(img_h/ws) x ceil(img_w/ws) windows of ws x ws tokens; positions outside the image are
 * the reference's zero-padded tokens: they take part as keys / values with the rows
 * pad_k / pad_v ((nH, hd) each, same element type - for SAM the bf16-rounded k and v bias of
 * the qkv Linear, which is what a zero input row produces) and produce no output.
 * rel_pos_h / rel_pos_w: (2*ws-1, hd).  Supported: hd in {64, 80}, ws <= 14 (ws*ws <= 208), bf16 or fp16.
 */
int samfast_attn_relpos_windowed_fwd(
    const void* q, const void* k, const void* v,
    const void* rel_pos_h, const void* rel_pos_w,
    const void* pad_k, const void* pad_v, void* out,
    int B, int nH, int img_h, int img_w, int ws, int hd,
    int64_t q_sb, int64_t q_sh, int64_t q_sn,
    int64_t k_sb, int64_t k_sh, int64_t k_sn,
    int64_t v_sb, int64_t v_sh, int64_t v_sn,
    int64_t o_sb, int64_t o_sh, int64_t o_sn,
    int dtype, float sm_scale, void* stream);

/*
 * Same attention with the two bias factors already computed by the caller:
 *   rel_h: (B, nH, N, gh) addressed ptr + b*rh_sb + h*rh_sh + n*rh_sn + j
 *   rel_w: (B, nH, N, gw) addressed ptr + b*rw_sb + h*rw_sh + n*rw_sn + j
 * This is the operand form of _attention_rel_h_rel_w(q,k,v,rel_h,rel_w)
 * (flash_4.py:335) and, with rel_h = base, rel_w = base + 64 and row stride 128,
 * of the operator customflash::custom_flash_aligned(q,k,v,rel_h_w,sm_scale)
 * (flash_4.py:268-329).  Same supported shapes as samfast_attn_relpos_fwd.
 */
int samfast_attn_relpos_bias_fwd(
    const void* q, const void* k, const void* v,
    const void* rel_h, const void* rel_w, void* out,
    int B, int nH, int gh, int gw, int hd,
    int64_t q_sb, int64_t q_sh, int64_t q_sn,
    int64_t k_sb, int64_t k_sh, int64_t k_sn,
    int64_t v_sb, int64_t v_sh, int64_t v_sn,
    int64_t o_sb, int64_t o_sh, int64_t o_sn,
    int64_t rh_sb, int64_t rh_sh, int64_t rh_sn,
    int64_t rw_sb, int64_t rw_sh, int64_t rw_sn,
    int dtype, float sm_scale, void* stream);

/*
 * Per-row symmetric int8 quantiser: for each of M rows of x (K values, row
 * stride ldx elements, type `dtype`):
 *   s = max(absmax(row), 1e-5) / 127;  xq = clamp(rint(row / s), -127, 127)
 * Writes xq (M, K) int8 contiguous and sx (M) fp32.  Stands for the per-token
 * activation quantiser torchao.apply_dynamic_quant installs in front of every
 * Linear (call site experiments/eval_combo.py:357-359).  K % 8 == 0, K <= 8192.
 * `layout` is the layout xq is written in (SAMFAST_LAYOUT_*).
 * A row that holds a NaN gets sx = NaN (its codes are unspecified), so the Linear that
 * consumes it returns NaN for that row and only that row; an infinite value makes the
 * scale infinite.  The same holds for samfast_layernorm_quant_i8.
 */
int samfast_quant_rowwise_i8(
    const void* x, int64_t ldx, int8_t* xq, float* sx,
    int64_t M, int K, int dtype, int layout, void* stream);

/*
 * acc[m, n] = sum_k xq[m, k] * wq[n, k], int32, exact.  xq (M, K) and wq (N, K)
 * int8 contiguous; acc (M, N) int32 contiguous.  The torch._int_mm step of the
 * quantised Linear (same call site), exposed so accumulators can be compared
 * bit for bit.  K % 64 == 0, N % 8 == 0.
 */
int samfast_gemm_i8_i32(
    const int8_t* xq, const int8_t* wq, int32_t* acc,
    int64_t M, int N, int K, void* stream);

/*
 * y[m, n] = (float(acc[m, n]) * sx[m]) * sw[n] + bias[n], rounded to `dtype`
 * (bf16), acc as in samfast_gemm_i8_i32 but never written to memory.  bias is
 * fp32 (N) or NULL; y has row stride ldy elements.  The whole quantised
 * nn.Linear.forward for qkv / proj (modeling/image_encoder.py:228,251) and
 * lin1 / lin2 (modeling/common.py:26) after samfast_quant_rowwise_i8.
 */
int samfast_gemm_i8_scale_bias(
    const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
    const float* bias, void* y, int64_t ldy,
    int64_t M, int N, int K, int dtype, void* stream);

/*
 * LayerNorm over each row followed by the per-row int8 quantiser, with an optional
 * row gather: output row r is computed from source row src_row[r] of x (src_row NULL =
 * identity); src_row[r] < 0 yields an all-zero row with scale 1e-5/127.
 *   y = (x - mean) / sqrt(var + eps) * gamma + beta   (fp32, biased variance, rounded
 *   to `dtype` as a separate LayerNorm would store it), then quantised as above.
 * One launch for norm1 + window_partition (zero padding to the window multiple) + the
 * qkv Linear's activation quantiser (modeling/image_encoder.py:169-173), or norm2 +
 * lin1's quantiser (:181).  gamma, beta: K values of type `dtype`.
 */
int samfast_layernorm_quant_i8(
    const void* x, int64_t ldx, const void* gamma, const void* beta, float eps,
    const int32_t* src_row, int8_t* xq, float* sx,
    int64_t M, int K, int dtype, int layout, void* stream);

/* epilogues of samfast_gemm_i8_fused */
#define SAMFAST_EPILOGUE_NONE 0      /* same as samfast_gemm_i8_scale_bias */
#define SAMFAST_EPILOGUE_GELU 1      /* y = gelu_erf(bf16(linear))                 */
#define SAMFAST_EPILOGUE_RESIDUAL 2  /* y[dst] = bf16(linear) + residual[dst]      */

/*
 * samfast_gemm_i8_scale_bias with a fused tail:
 *   GELU      exact-erf GELU of the bf16-rounded Linear output - lin1 followed by
 *             act() in MLPBlock.forward (modeling/common.py:26);
 *   RESIDUAL  adds `residual` (bf16, row stride ld_res) and scatters rows: GEMM row m
 *             is written to output row dst_row[m] (NULL = identity, < 0 = dropped) and
 *             the residual is read at that same output row.  With the inverse window
 *             map this is proj + window_unpartition + `shortcut + x`
 *             (modeling/image_encoder.py:176-180); with the identity map it is lin2 +
 *             `x + mlp(...)` (:181).  y and residual may be the same buffer.
 * `layout` names the layout of BOTH xq and wq (SAMFAST_LAYOUT_*).
 */
int samfast_gemm_i8_fused(
    const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
    const float* bias, void* y, int64_t ldy,
    int64_t M, int N, int K, int dtype, int epilogue,
    const void* residual, int64_t ld_res, const int32_t* dst_row, int layout, void* stream);

/*
 * samfast_gemm_i8_fused (epilogues NONE / GELU / RESIDUAL, no row scatter) that also hands the
 * NEXT Linear its quantised input: after y is written, each row of y - passed through LayerNorm
 * first when ln_gamma / ln_beta (N values of type `dtype`) are given - is quantised per row exactly
 * as samfast_quant_rowwise_i8 / samfast_layernorm_quant_i8 would quantise it, into yq (M, N) int8 in
 * `yq_layout` and sy (M) fp32; codes and scales are bit-equal to those two calls on y.  Stands for
 * what the compiler fuses around the reference's quantised Linears: lin1 + GELU + lin2's activation
 * quantiser (modeling/common.py:25-26), proj + residual + norm2 + lin1's quantiser and lin2 +
 * residual + the next block's norm1 + qkv's quantiser (modeling/image_encoder.py:167-183).
 * Where the shape allows (K >= 256; GELU with N in {3072, 4096, 5120}, or RESIDUAL + LayerNorm with
 * N in {768, 1024, 1280}) everything is ONE launch: the workgroup that completes a 128-row tile
 * quantises its rows (no workgroup ever waits for another); other shapes run as two launches.
 * `tile_counters`: device workspace of at least ceil(M / 128) int32, all zero on entry; the launch
 * leaves it all zero again, so one buffer serves every call on a stream.  Calls that share a counter
 * buffer must not overlap in time (use one buffer per stream).
 */
int samfast_gemm_i8_fused_quant(
    const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
    const float* bias, void* y, int64_t ldy,
    int64_t M, int N, int K, int dtype, int epilogue,
    const void* residual, int64_t ld_res, int layout,
    const void* ln_gamma, const void* ln_beta, float ln_eps,
    int8_t* yq, float* sy, int yq_layout, int32_t* tile_counters, void* stream);

/*
 * samfast_gemm_i8_fused_quant for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid it).  It has no counterpart in the reference.  Same
 * arguments and results, minus the `tile_counters` workspace: the counters live in a device array
 * inside the library (128 KiB per GPU, held until the process ends), whose entries the call clears
 * with a small kernel before it uses them.  M is limited to 4 194 304 rows (32768 row tiles of 128);
 * a larger M returns SAMFAST_E_INVALID.  All calls on one GPU share that array, so two such calls
 * must not overlap in time on one GPU (issue them on one stream, or order the streams).
 */
int samfast_gemm_i8_fused_quant_noalloc(
    const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
    const float* bias, void* y, int64_t ldy,
    int64_t M, int N, int K, int dtype, int epilogue,
    const void* residual, int64_t ld_res, int layout,
    const void* ln_gamma, const void* ln_beta, float ln_eps,
    int8_t* yq, float* sy, int yq_layout, void* stream);

/*
 * 2:4-sparse weights for the sparse int8 matrix cores (v_smfmac_i32_32x32x64_i8).
 *
 * samfast_prune24_pack_i8: from a dense int8 weight wq (N, K) keep, in every aligned group
 * of 4 consecutive k, the 2 entries of largest magnitude (ties: lowest k) and write them in
 * the packed form the GEMM below reads.  A matrix that already is 2:4 (at most 2 non-zeros
 * per group, e.g. quantised after magnitude pruning of the float weight) is packed without
 * loss.  K % 64 == 0.  Packed layout, K-block major (kb = k / 64):
 *   wc   (K/64, N, 32) int8:  byte 16*h + 2*g + e  (h in 0..1, g in 0..7, e in 0..1) holds
 *        wq[n, 64*kb + 32*(g/4) + 16*h + 4*(g%4) + p_e], p_0 < p_1 the kept positions;
 *   widx (K/64, N, 2) int32:  word h, bits 4g+1:4g = p_0, bits 4g+3:4g+2 = p_1.
 * Stands for the prune + compress steps of apply_sparse (sparse.py:6-32: WeightNormSparsifier
 * with sparse_block_shape (1,4), zeros_per_block 2, then to_sparse_semi_structured), applied
 * to int8 weights.
 */
int samfast_prune24_pack_i8(
    const int8_t* wq, int8_t* wc, int32_t* widx, int N, int K, void* stream);

/*
 * acc[m, n] = sum_k xq[m, k] * w[n, k] (int32, exact) with w given in the packed 2:4 form;
 * equals samfast_gemm_i8_i32 on the pruned dense matrix.  K % 128 == 0, K >= 256, N % 8 == 0.
 */
int samfast_gemm_i8_sparse24_i32(
    const int8_t* xq, const int8_t* wc, const int32_t* widx, int32_t* acc,
    int64_t M, int N, int K, void* stream);

/*
 * samfast_gemm_i8_fused (epilogues NONE / GELU / RESIDUAL, no row scatter) with the weight
 * in the packed 2:4 form: the semi-structured Linear the reference builds at sparse.py:28-32,
 * here for the int8 MLP linears lin1 (GELU) and lin2 (residual) (modeling/common.py:26).
 * y and residual rows must be 16-byte aligned (ldy, ld_res multiples of 8).  `layout` is the
 * layout of xq (the weight has its own packed form).
 */
int samfast_gemm_i8_sparse24_fused(
    const int8_t* xq, const float* sx, const int8_t* wc, const int32_t* widx,
    const float* sw, const float* bias, void* y, int64_t ldy,
    int64_t M, int N, int K, int dtype, int epilogue,
    const void* residual, int64_t ld_res, int layout, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SAMFAST_H */
