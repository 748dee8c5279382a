/*
 * mase_amd C ABI: gfx950 (MI355X) kernels for MASE's quantized-inference hot path.
 *
 * Every entry point
 *   - takes plain device pointers, sizes and format integers (no framework types),
 *   - enqueues its kernels on `stream` (a hipStream_t passed as void*) and returns immediately,
 *   - never allocates, frees or synchronises,
 *   - returns MASE_OK (0) or a negative MASE_ERR_* code; it never throws or aborts.
 * Tensors are dense and contiguous in the order stated for each call.  "dtype" is one of MASE_DT_*.
 *
 * Reference interfaces replaced (paths relative to the reference's src/chop/):
 *   mase_mxint_qdq          nn/quantizers/mxint/mxint.py:211-251  (mxint_quantizer, non-search branch :145-169;
 *                           arithmetic nn/quantizers/mxint/fake.py:11-80)
 *   mase_block_fp_qdq       nn/quantizers/block_fp.py:111-142     (block_fp_quantizer; arithmetic :7-82,
 *                           blocking nn/quantizers/utils.py:350-629)
 *   mase_integer_qdq        nn/quantizers/integer.py:97-122       (integer_quantizer / integer_floor_quantizer)
 *   mase_minifloat_qdq      nn/quantizers/minifloat.py:90-117, :200-225 (minifloat_denorm/ieee_quantizer)
 *   mase_minifloat_mx_qdq   nn/quantizers/_minifloat_mx/minifloat.py:12-33 (minifloat_quantizer_sim)
 *   mase_mxfp_qdq           nn/quantizers/mxfp/mxfp.py:187-230    (mxfp_quantizer, non-search branch)
 *   mase_mxint_clip_search  nn/quantizers/mxint/mxint.py:40-143 (quantile_search=True without calibration activations)
 *   mase_mxfp_clip_search   nn/quantizers/mxfp/mxfp.py:40-105   (quantile_search=True without calibration activations)
 *   mase_mxint_clip_candidates, mase_mxfp_clip_candidates   the candidates of the same searches, for the form scored
 *                           on calibration outputs (mxint.py:99-131, mxfp.py:65-93)
 *   mase_rope               nn/quantized/functional/rope.py:17-27 (_apply_rope)
 *   mase_rmsnorm_minifloat  nn/quantized/modules/llama/rms_norm.py:72-84 (LlamaRMSNormMinifloat.forward)
 *   mase_silu_mul_minifloat nn/quantized/modules/llama/mlp.py:60-62 (silu_minifloat(gate) * up)
 *   mase_rmsnorm_mxint, mase_silu_mul_mxint   the two above followed by the consumer LinearMXInt's activation
 *                           quantizer (nn/quantized/modules/linear.py:956-972) in the same pass
 *   mase_silu_mul_mxint_lut, mase_silu_table  mase_silu_mul_mxint for 16-bit tensors with silu read from a table
 *   mase_add_rmsnorm_mxint  models/llama/modeling_llama.py:901-905 (residual addition, then the norm as above)
 *   mase_attn_softmax_mx    nn/quantized/modules/llama/attention.py:363-392 (scores -> quantized probabilities)
 *   mase_attention_causal   models/llama/modeling_llama.py:362-480 (the attention core on unquantized q, k, v)
 *   mase_mx_unpack          nn/quantizers/mxint/fake.py:59-80, nn/quantizers/mxfp/fake.py:75-104 (compose_*)
 *   mase_mxfp_pack(_tiled), mase_mxfp_tile_codes, mase_gemm_mxfp_scaled, mase_gemm_mxfp4_scaled_tiled
 *                           nn/quantized/modules/linear.py:877-895 (LinearMXFP.forward on
 *                           formats the block-scaled matrix instruction supports)
 *   mase_gemm_mxfp4_skinny  nn/quantized/modules/linear.py:877-895 for at most 128 rows, MXFP4 weights
 *   mase_gemm_mxint8_skinny nn/quantized/modules/linear.py:972 for at most 128 rows, weights as int8 codes + scales
 *   mase_gemm_bf16_skinny   same call sites as mase_gemm_bf16_tn, for at most 128 rows of activations
 *   mase_gemm_bf16_tn_packed, mase_gemm_bf16_pack_b   the same F.linear with the weight in fragment order
 *   mase_gemm_mxint8_tn_packed, mase_gemm_mxint8_pack_b   the same with the weight as MXINT8 codes in fragment order
 *   mase_gemm_bf16_tn       nn/quantized/modules/linear.py:972 and :895 (the F.linear of LinearMXInt.forward /
 *                           LinearMXFP.forward on the quantize-dequantized operands)
 */
#ifndef MASE_AMD_H
#define MASE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MASE_OK 0
#define MASE_ERR_NULL (-1)      /* a required pointer is NULL */
#define MASE_ERR_SHAPE (-2)     /* sizes inconsistent (e.g. numel not divisible by the block size) */
#define MASE_ERR_ALIGN (-3)     /* a pointer is not aligned as the call requires */
#define MASE_ERR_DTYPE (-4)     /* unknown dtype code */
#define MASE_ERR_PARAM (-5)     /* format parameter outside the supported domain */
#define MASE_ERR_LAUNCH (-6)    /* the HIP runtime rejected a launch */
#define MASE_ERR_WORKSPACE (-7) /* workspace missing or too small */

#define MASE_DT_F32 0
#define MASE_DT_BF16 1
#define MASE_DT_F16 2

/* number of uint32 entries in a log2 correction table (see mase_log2_table_layout below) */
#define MASE_LOG2_TABLE_WORDS 576

int mase_abi_version(void);
const char* mase_error_string(int code);

/*
 * log2 correction tables.  The reference evaluates ceil(log2(v)) / floor(log2(v)) with the host math
 * library *in the tensor dtype*, whose rounded result differs from the exact integer answer for values
 * a few ulps away from a power of two.  To be bit-exact the kernels take a table measured on the host
 * (one per dtype), in device memory, MASE_LOG2_TABLE_WORDS uint32 words:
 *   tab[k+149]       largest normalised 23-bit mantissa M>0 with ceil(log2(2^k*(1+M/2^23))) == k, else 0
 *   tab[288+k+149]   smallest M with floor(log2(2^k*(1+M/2^23))) == k+1, else 0x800000
 * for k = floor(log2 v) in [-149, 127].  Words 277..279 of each half are reserved (the host tooling stores a
 * summary there; the kernels do not read them).  A table of all 0 in the first half and all 0x800000 in the
 * second gives the exact integer answers.  Kernels keep the entries for k in [-32, 31] in one register per lane.
 */

/* MXINT quantize-dequantize over contiguous runs of `block_size` elements of a flat array.
 * in: numel elements of `dtype` (all arithmetic follows that dtype); out: numel elements of `out_dtype` (the
 * reference's final `.to(dtype)`; MXINT8 values are exact in bf16, which is how the Linear path takes them).
 * codes (int8, numel) and scales (uint8, numel/block_size) are optional packed outputs (both or neither;
 * element_bits <= 8): value = codes * 2^(scales - 134). */
int mase_mxint_qdq(const void* in, void* out, int8_t* codes, uint8_t* scales, size_t numel, int dtype,
                   int out_dtype, int block_size, int element_bits, int scale_bits, const uint32_t* log2_tab,
                   void* stream);

/* Block floating point over [batch, rows, cols] with tiles of tile_rows x tile_cols inside each batch
 * item (ragged edges behave as if zero padded).  exponent_bias < 0 selects 2^(exponent_width-1)-1.
 * zero_sign_mode: 0 = an element that quantizes to zero keeps the sign of the input (the reference's
 * reshape-based blocking of 1-D tensors and of 2-D activations), 1 = it becomes +0 (the reference's
 * unfold/fold blocking of 2-D weights and 3-D activations, where fold adds into a zero buffer).
 * workspace: mase_block_fp_workspace_bytes() bytes of device memory; may be NULL when tile_rows == 1,
 * tile_cols is a power of two dividing cols, and in/out are 16-byte aligned (single-pass schedule). */
size_t mase_block_fp_workspace_bytes(size_t batch, size_t rows, size_t cols, int tile_rows, int tile_cols,
                                     int dtype);
int mase_block_fp_qdq(const void* in, void* out, size_t batch, size_t rows, size_t cols, int tile_rows,
                      int tile_cols, int dtype, int width, int exponent_width, int exponent_bias,
                      int zero_sign_mode, const uint32_t* log2_tab, void* workspace, size_t workspace_bytes,
                      void* stream);

/* mase_block_fp_qdq for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments and results, without the workspace.  It has no counterpart
 * in the reference.  The per-tile maxima of the two-pass schedule live in a 4 MiB array inside the library's own
 * device image (one copy per GPU, held until the process ends), so at most MASE_BLOCK_FP_STATIC_MAX_TILES
 * tiles per call: MASE_ERR_WORKSPACE beyond that.  The call allocates and frees nothing; the first call on a device
 * looks up the array's address (do it once outside any graph capture).  All calls on one GPU share the array:
 * calls that may overlap on one GPU (different streams, different host threads) race on it and must be serialized by
 * the caller.  The part of the array a call uses is cleared by a fill kernel on `stream` before it is used. */
#define MASE_BLOCK_FP_STATIC_MAX_TILES (1u << 20)
int mase_block_fp_qdq_static(const void* in, void* out, size_t batch, size_t rows, size_t cols, int tile_rows,
                             int tile_cols, int dtype, int width, int exponent_width, int exponent_bias,
                             int zero_sign_mode, const uint32_t* log2_tab, void* stream);

/* Fixed point: clamp(round_or_floor(x * 2^frac_width)) / 2^frac_width. */
int mase_integer_qdq(const void* in, void* out, size_t numel, int dtype, int width, int frac_width,
                     int is_signed, int use_floor, void* stream);

/* Element-wise minifloat, ieee = 0 (no implicit leading bit) or 1 (implicit leading bit). */
int mase_minifloat_qdq(const void* in, void* out, size_t numel, int dtype, int width, int exponent_width,
                       int exponent_bias, int ieee, const uint32_t* log2_tab, void* stream);

/* Bit-level minifloat cast used by the MX formats.  round_mode: 0 rn, 1 ru, 2 rd, 3 rz. */
int mase_minifloat_mx_qdq(const void* in, void* out, size_t numel, int in_dtype, int out_dtype, int exp_bits,
                          int frac_bits, int is_finite, int round_mode, void* stream);

/* MXFP quantize-dequantize over contiguous runs of block_size elements.  log2_tab is the fp32 table.
 * Optional packed outputs: codes (uint8, numel; sign|exp|frac in the low 1+E+F bits) and scales
 * (uint8 E8M0, numel/block_size). */
int mase_mxfp_qdq(const void* in, void* out, uint8_t* codes, uint8_t* scales, size_t numel, int in_dtype,
                  int out_dtype, int block_size, int exp_bits, int frac_bits, const uint32_t* log2_tab,
                  void* stream);

/* Clip search (quantile_search=True, act_tensor=None): per block of 32 elements, 11 quantize-dequantize candidates
 * whose scale comes from the 1.0, 0.995, 0.99, 0.97, 0.95, 0.93, 0.90, 0.80, 0.70, 0.60, 0.50 quantile of |x| (linear
 * interpolation, as the library's quantile) instead of the maximum; the candidate the reference's error measure
 * prefers is written to `out` (same dtype as `in`), its index 0..10 to `choice` (optional, one byte per block).
 * in: the tensor with block_dim moved last, flattened; ref: the tensor in its plain flattening (the reference
 * measures the error against that one; the same array when block_dim is the last dimension).  block_size 16, 32 or 64;
 * in / ref / out 16-byte aligned.  MXINT (nn/quantizers/mxint/mxint.py:40-143): error = L2 norm in `dtype`, first
 * minimum wins.  MXFP (nn/quantizers/mxfp/mxfp.py:40-105): the reference's score on the integer codes, strictly
 * smaller replaces.  Candidates whose errors differ only by the summation order of the 32 squares may swap with respect
 * to the library's reductions. */
int mase_mxint_clip_search(const void* in, const void* ref, void* out, uint8_t* choice, size_t numel, int dtype,
                           int block_size, int element_bits, int scale_bits, const uint32_t* log2_tab, void* stream);
int mase_mxfp_clip_search(const void* in, const void* ref, void* out, uint8_t* choice, size_t numel, int dtype,
                          int block_size, int exp_bits, int frac_bits, const uint32_t* log2_tab, void* stream);

/* All eleven candidates of the clip search instead of the winner, for the search scored on calibration outputs
 * (quantile_search=True with act_tensor: nn/quantizers/mxint/mxint.py:99-131, nn/quantizers/mxfp/mxfp.py:65-93, the
 * clip_search_y option of the GPTQ pass, passes/module/transforms/gptq/run.py:194), whose error measure is a norm over
 * batches of activations times the candidate and is evaluated with matrix products by the caller.  in: the tensor with
 * block_dim moved last, flattened; cand: 11 * numel elements of dtype, cand[P * numel + i] = element i quantized with
 * the scale of percentile P.  score (MXFP only, same shape): the values the reference multiplies with the activations,
 * code / 2^(F-1) * 2^(scale - 127) on the integer codes with the power in uint8 arithmetic.  block_size 16, 32 or 64. */
int mase_mxint_clip_candidates(const void* in, void* cand, size_t numel, int dtype, int block_size, int element_bits,
                               int scale_bits, const uint32_t* log2_tab, void* stream);
int mase_mxfp_clip_candidates(const void* in, void* cand, void* score, size_t numel, int dtype, int block_size,
                              int exp_bits, int frac_bits, const uint32_t* log2_tab, void* stream);

/* Dequantization of the packed outputs of mase_mxint_qdq (kind 0: p0 = element_bits, p1 unused; value = code *
 * 2^(scale - 134)) or mase_mxfp_qdq (kind 1: p0 = exp_bits, p1 = frac_bits; value = minifloat(code) * 2^(scale - 127),
 * NaN for a block whose scale byte is 255): codes (numel bytes), scales (numel / block_size bytes) -> out (numel
 * elements of out_dtype).  The "compose" half of the reference's quantizers (nn/quantizers/mxint/fake.py:59-80,
 * nn/quantizers/mxfp/fake.py:75-104), for loading checkpoints that store codes and scales. */
int mase_mx_unpack(const uint8_t* codes, const uint8_t* scales, void* out, size_t numel, int block_size, int out_dtype,
                   int kind, int p0, int p1, void* stream);

/* C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]): bf16 operands (both K-major, 16-byte aligned, K % 64 == 0), fp32
 * accumulation on the matrix cores, C written in out_dtype.  bias may be NULL; bias_dtype is its MASE_DT_*.
 * Each operand must be smaller than 4 GiB (MASE_ERR_SHAPE otherwise).  Launches one work-group per CU.
 * This is the contraction of LinearMXInt.forward / LinearMXFP.forward (nn/quantized/modules/linear.py:972,
 * :895) on operands whose MX values are held exactly in bf16. */
int mase_gemm_bf16_tn(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N, size_t K,
                      int out_dtype, int bias_dtype, void* stream);

/* batch_outer x batch_inner independent products C[o][i] = A[o][i] (M x K) * B[o][i] (N x K)^T, bf16 operands, fp32
 * accumulation, output in out_dtype, on the same tiled kernel: the batched contractions of the quantized attention
 * modules (torch.matmul of the quantized query with the keys and of the quantized probabilities with the values,
 * nn/quantized/modules/llama/attention.py:398-457) and of bmm_mx* / matmul_mx* on batched operands
 * (nn/quantized/functional/matmul.py:437-512), whose quantized operands are exact in bf16.  All strides in elements:
 * lda / ldb / ldc of a row of A / B / C, and per operand the strides of the outer and the inner batch index (a head
 * of [batch, tokens, heads, d] memory is row stride heads * d, inner stride d, outer stride tokens * heads * d).
 * K % 64 == 0; operand strides multiples of 8 and output strides multiples of 16 bytes; pointers 16-byte aligned;
 * M * lda and N * ldb below 2^31 elements. */
int mase_gemm_bf16_tn_batched(const void* A, const void* B, void* C, size_t batch_outer, size_t batch_inner, size_t M,
                              size_t N, size_t K, size_t lda, size_t ldb, size_t ldc, size_t a_stride_outer,
                              size_t a_stride_inner, size_t b_stride_outer, size_t b_stride_inner, size_t c_stride_outer,
                              size_t c_stride_inner, int out_dtype, void* stream);

/* The same product for shapes whose 256x256 output tiles alone would leave most CUs idle (a few hundred rows of A):
 * K is cut into ranges, every (tile, range) pair is a work item of the same kernel and writes an fp32 partial tile into
 * `workspace` (at least mase_gemm_bf16_tn_splitk_workspace_bytes(M, N, K) bytes, 16-byte aligned), and a second kernel
 * adds the ranges in a fixed order, adds the bias and converts.  _workspace_bytes returns 0 when no split pays, and the
 * call is then mase_gemm_bf16_tn itself (workspace may be NULL). */
size_t mase_gemm_bf16_tn_splitk_workspace_bytes(size_t M, size_t N, size_t K);
int mase_gemm_bf16_tn_splitk(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N, size_t K,
                             int out_dtype, int bias_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* The same product with B given as the fragment-ordered image written by mase_gemm_bf16_pack_b (a weight is packed
 * once when it is loaded): B's fragments then go from the cache straight into registers instead of through LDS, which
 * the kernel otherwise shares between the copies arriving and the fragment reads.  K % 128 == 0; the image takes
 * mase_gemm_bf16_packed_bytes(N, K) = ceil(N/32)*32*K*2 bytes (below 4 GiB), 16-byte aligned; the packer takes any
 * K % 32 == 0.  Same results as mase_gemm_bf16_tn (the same products added in the same order: both compute with the
 * 16x16x32 matrix instruction, K step by K step).  Replaces the same F.linear (nn/quantized/modules/linear.py:972,
 * :895). */
size_t mase_gemm_bf16_packed_bytes(size_t N, size_t K);
int mase_gemm_bf16_pack_b(const void* B, void* B_packed, size_t N, size_t K, void* stream);
int mase_gemm_bf16_tn_packed(const void* A, const void* B_packed, const void* bias, void* C, size_t M, size_t N,
                             size_t K, int out_dtype, int bias_dtype, void* stream);

/* The tiled product with B held as an MXINT8 weight in fragment order: the code image and the scale image written by
 * mase_gemm_mxint8_pack_b from int8 codes [N, K] and scale bytes [N, K/32] (value = code * 2^(scale - 134): the packed
 * outputs of mase_mxint_qdq with element_bits 8, block 32).  1.03 bytes per weight in memory and on the way in; the
 * codes are widened to the same bf16 values in registers, so the result is that of mase_gemm_bf16_tn on the
 * dequantized weight (the same products added in the same order, bit for bit) as long as every scale byte is at least 8
 * (weights of 2^-119 and less are taken as zero).  K % 128 == 0; images 16-byte / 8-byte aligned, the code image below 4 GiB.
 * _code_bytes / _scale_bytes: sizes of the two images (0 when K % 128 != 0).  Replaces the F.linear of
 * LinearMXInt.forward (nn/quantized/modules/linear.py:972) with the weight dequantized on the way into the matrix
 * instruction instead of beforehand. */
size_t mase_gemm_mxint8_packed_code_bytes(size_t N, size_t K);
size_t mase_gemm_mxint8_packed_scale_bytes(size_t N, size_t K);
int mase_gemm_mxint8_pack_b(const int8_t* codes, const uint8_t* scales, void* code_image, void* scale_image, size_t N,
                            size_t K, void* stream);
int mase_gemm_mxint8_tn_packed(const void* A, const void* code_image, const void* scale_image, const void* bias, void* C,
                               size_t M, size_t N, size_t K, int out_dtype, int bias_dtype, void* stream);

/* The same product for few rows of A (M <= 128, the token-by-token shape of serving): bound by streaming B once
 * from HBM.  The work is split over N and over K ranges; the partial results of the K ranges go through
 * `workspace` (device memory, 16-byte aligned, at least mase_gemm_bf16_skinny_workspace_bytes(M, N, K) bytes, which
 * is at most 64*M*N*4) and are added in a fixed order, so results are reproducible; when one K range is enough
 * (wide weights) the workspace is not touched and the output is written by the first kernel.  K % 64 == 0.
 * Replaces the same F.linear as mase_gemm_bf16_tn (nn/quantized/modules/linear.py:972, :895). */
size_t mase_gemm_bf16_skinny_workspace_bytes(size_t M, size_t N, size_t K);
int mase_gemm_bf16_skinny(const void* A, const void* B, const void* bias, void* C, size_t M, size_t N, size_t K,
                          int out_dtype, int bias_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* The few-rows product with B held as packed MXINT8: int8 codes [N, K] and one scale byte per 32 codes [N, K/32]
 * (value = code * 2^(scale - 134): the packed outputs of mase_mxint_qdq with element_bits 8, block 32), so the weight
 * stream is half the bytes of the bf16 image.  Codes are widened to the same bf16 values in registers; A is bf16.
 * M <= 128, K % 128 == 0, N*K < 2^32; workspace as for mase_gemm_bf16_skinny.  Replaces the F.linear of
 * LinearMXInt.forward (nn/quantized/modules/linear.py:972) for decode-sized batches. */
size_t mase_gemm_mxint8_skinny_workspace_bytes(size_t M, size_t N, size_t K);
int mase_gemm_mxint8_skinny(const void* A, const int8_t* B_codes, const uint8_t* B_scales, const void* bias, void* C,
                            size_t M, size_t N, size_t K, int out_dtype, int bias_dtype, void* workspace,
                            size_t workspace_bytes, void* stream);

/* The few-rows product on packed MXFP operands (layout of mase_mxfp_pack): activations e4m3 (a_format 0) or e5m2 (1)
 * codes [M, K] with scales [M, K/32], weights e2m1 codes [N, K/2] with scales [N, K/32], on the block-scaled MFMA.
 * The weight stream is 0.53 bytes per element.  M <= 128, K % 128 == 0; workspace as for mase_gemm_bf16_skinny.
 * LinearMXFP.forward (nn/quantized/modules/linear.py:877-895) for decode-sized batches with MXFP4 weights. */
size_t mase_gemm_mxfp4_skinny_workspace_bytes(size_t M, size_t N, size_t K);
int mase_gemm_mxfp4_skinny(const void* A_codes, const void* A_scales, int a_format, const void* B_codes,
                           const void* B_scales, const void* bias, void* C, size_t M, size_t N, size_t K, int out_dtype,
                           int bias_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* MXFP packing for the block-scaled matrix instruction.  in: numel elements (numel % 32 == 0, blocks of 32
 * consecutive elements); element format (exp_bits, frac_bits) in {(4,3), (5,2), (2,1)}.  codes: one byte per
 * element for 8-bit formats, two elements per byte (even element in the low nibble) for (2,1); scales: one E8M0
 * byte per block.  codes/scales decode to the values of mase_mxfp_qdq, except that a block using a code the
 * OCP format reserves (e4m3 S.1111.111, e5m2 exponent 31) is stored with scale+1 and halved elements.
 * Quantizer part: nn/quantizers/mxfp/fake.py:12-72. */
int mase_mxfp_pack(const void* in, uint8_t* codes, uint8_t* scales, size_t numel, int in_dtype, int exp_bits,
                   int frac_bits, const uint32_t* log2_tab, void* stream);

/* C[M,N] = A[M,K] * B[N,K]^T (+ bias[N]) on packed MXFP operands (layout of mase_mxfp_pack, K % 128 == 0), using
 * the block-scaled MFMA.  a_format / b_format: 0 = e4m3, 1 = e5m2, 4 = e2m1 (B only).  M*K and N*K must be below
 * 2^32 (MASE_ERR_SHAPE otherwise).  Inside one instruction the 8 products of a register pair are added after
 * alignment to the largest of them with about 12 bits kept below its leading bit; sums across such groups and
 * across instructions are fp32.  The contraction of
 * LinearMXFP.forward (nn/quantized/modules/linear.py:877-895) for hardware formats. */
int mase_gemm_mxfp_scaled(const void* A, const void* A_scales, int a_format, const void* B, const void* B_scales,
                          int b_format, const void* bias, void* C, size_t M, size_t N, size_t K, int out_dtype,
                          int bias_dtype, void* stream);

/* The same product with both code matrices as tile images: for a [rows, K] code matrix of 8-bit (4-bit) codes the image
 * is [row tile of 256][K tile of 128][row in tile][128 (64) bytes], the 16-byte chunks of each row segment exchanged by
 * chunk ^= (row >> 1) & 7 (chunk ^= (row >> 2) & 3), rows past the end repeating the last one: the bytes one K tile of
 * one row tile occupies in the kernel's LDS stage, contiguous, so that every copy reads one 1 KB run.  Scales stay
 * row-major.  mase_mxfp_tiled_bytes: size of an image (0 for K % 128 != 0 or bits other than 4, 8).
 * mase_mxfp_tile_codes: image of a row-major code matrix (done once for a weight).  mase_mxfp_pack_tiled: mase_mxfp_pack
 * for a [rows, K] matrix of e4m3 / e5m2 activations writing the image directly (tiled_codes holds
 * mase_mxfp_tiled_bytes(rows, K, 8) bytes; rows past the end are left unwritten and only ever feed output rows that are
 * not stored).  mase_gemm_mxfp4_scaled_tiled: A e4m3 / e5m2 image, B e2m1 image; result bit-identical to
 * mase_gemm_mxfp_scaled on the row-major forms; both images must be below 2^32 bytes.  Same contraction of
 * LinearMXFP.forward (nn/quantized/modules/linear.py:877-895). */
size_t mase_mxfp_tiled_bytes(size_t rows, size_t K, int bits);
int mase_mxfp_tile_codes(const void* codes, void* tiled, size_t rows, size_t K, int bits, void* stream);
int mase_mxfp_pack_tiled(const void* in, uint8_t* tiled_codes, uint8_t* scales, size_t rows, size_t K, int in_dtype,
                         int exp_bits, int frac_bits, const uint32_t* log2_tab, void* stream);
int mase_gemm_mxfp4_scaled_tiled(const void* A_tiled, const void* A_scales, int a_format, const void* B_tiled,
                                 const void* B_scales, const void* bias, void* C, size_t M, size_t N, size_t K,
                                 int out_dtype, int bias_dtype, void* stream);

/* Attention probabilities of the MX-quantized Llama attention in one pass: for scores [batch, heads, q_len, kv_len]
 * (dense, dtype) and an optional additive mask [batch, 1, q_len, kv_len] of the same dtype (rows mask_row_stride
 * elements apart, batches q_len rows apart):
 *   w = scores * scaling; w += mask; w = minifloat cast (cast_exp_bits > 0; bit-level cast of mase_minifloat_mx_qdq);
 *   p = softmax(float(w)) along kv_len, rounded to dtype; p = MX quantize-dequantize in blocks of 32 along kv_len
 *   (mx_kind 0 none, 1 MXINT with mx_p0 element bits, 2 MXFP with mx_p0 / mx_p1 exponent / fraction bits),
 * each intermediate rounded to dtype as the separate tensor operations would.  kv_len % 32 == 0, kv_len <= 8192.
 * log2_tab_dtype: table of `dtype` (MXINT), log2_tab_f32: fp32 table (MXFP); the one not needed may be NULL.
 * Replaces the score-to-probability part of _eager_attention_forward_mxfp / _mxint
 * (nn/quantized/modules/llama/attention.py:363-392) with softmax_minifloat (nn/quantized/functional/softmax.py:41-57). */
int mase_attn_softmax_mx(const void* scores, const void* mask, void* out, size_t batch, size_t heads, size_t q_len,
                         size_t kv_len, size_t mask_row_stride, int dtype, float scaling, int cast_exp_bits,
                         int cast_frac_bits, int cast_is_finite, int cast_round_mode, int mx_kind, int mx_p0, int mx_p1,
                         const uint32_t* log2_tab_dtype, const uint32_t* log2_tab_f32, void* stream);

/* RMSNorm over the last dimension of x [rows, cols] with optional bit-level minifloat casts (exp_bits 0 = off) of the
 * input and of the weight [cols], all in dtype:  h = cast(x);  h = float(h) * rsqrt(mean(h^2) + eps);
 * out = cast(weight) * dtype(h).  cols % 8 == 0, cols <= 8192.  LlamaRMSNormMinifloat.forward
 * (nn/quantized/modules/llama/rms_norm.py:72-84); with both casts off the plain Llama RMSNorm
 * (models/llama/modeling_llama.py:79-93). */
int mase_rmsnorm_minifloat(const void* x, const void* weight, void* out, size_t rows, size_t cols, int dtype, float eps,
                           int x_exp_bits, int x_frac_bits, int x_is_finite, int x_round_mode, int w_exp_bits,
                           int w_frac_bits, int w_is_finite, int w_round_mode, void* stream);

/* out = silu(cast(gate)) * up, element-wise over numel elements of dtype (numel % 8 == 0), the cast optional
 * (exp_bits 0 = off): LlamaMLPMXInt / LlamaMLPMXFP.forward's silu_minifloat(gate_proj(x)) * up_proj(x)
 * (nn/quantized/modules/llama/mlp.py:60-62, nn/quantized/functional/silu.py:41-57). */
int mase_silu_mul_minifloat(const void* gate, const void* up, void* out, size_t numel, int dtype, int exp_bits,
                            int frac_bits, int is_finite, int round_mode, void* stream);

/* The same RMSNorm (casts off) and SwiGLU product (cast off) with the MXINT quantize-dequantize of the LinearMXInt that
 * consumes the result applied to it before it is stored: out = mxint_quantizer(result, block 32 along the last
 * dimension, element_bits), the arithmetic of mase_mxint_qdq on the result rounded to dtype, so out holds what that
 * Linear's forward would compute from the stored result (nn/quantized/modules/linear.py:956-972 after
 * models/llama/modeling_llama.py:79-93 / :219-236) and a pass over the tensor is saved.  cols % 32 == 0 (numel % 32 == 0),
 * log2_tab as for mase_mxint_qdq in dtype. */
int mase_rmsnorm_mxint(const void* x, const void* weight, void* out, size_t rows, size_t cols, int dtype, float eps,
                       int element_bits, const uint32_t* log2_tab, void* stream);
int mase_silu_mul_mxint(const void* gate, const void* up, void* out, size_t numel, int dtype, int element_bits,
                        const uint32_t* log2_tab, void* stream);

/* The same operation for 16-bit tensors with R(silu(gate)) read from a table of its 65536 possible values, which
 * mase_silu_table fills once per dtype (bf16 or fp16; 128 KB of device memory, 16-byte aligned) with the expression
 * mase_silu_mul_mxint evaluates per element: same results bit for bit, without the exponential and the division per
 * element (a third of that kernel's time on large tensors).  The table sits in LDS, one work-group per CU.
 * Same call site as mase_silu_mul_mxint (nn/quantized/modules/llama/mlp.py:60-62 followed by the activation quantizer of
 * nn/quantized/modules/linear.py:956-972). */
int mase_silu_table(void* table, int dtype, void* stream);
int mase_silu_mul_mxint_lut(const void* gate, const void* up, void* out, size_t numel, int dtype, int element_bits,
                            const uint32_t* log2_tab, const void* silu_table, void* stream);

/* The residual addition of a pre-norm block followed by mase_rmsnorm_mxint, in one pass: sum_out = x + residual (rounded
 * to dtype, as the tensor addition rounds it) and out = mxint_quantizer(rmsnorm(sum_out)) as above
 * (models/llama/modeling_llama.py:901-905: hidden = residual + hidden; residual = hidden;
 * hidden = post_attention_layernorm(hidden)).  x, residual, sum_out, out: [rows, cols] contiguous; sum_out may be x or
 * residual. */
int mase_add_rmsnorm_mxint(const void* x, const void* residual, const void* weight, void* sum_out, void* out, size_t rows,
                           size_t cols, int dtype, float eps, int element_bits, const uint32_t* log2_tab, void* stream);

/* Causal self-attention core out = softmax(q k^T * scaling + causal mask) v for bf16 q, k, v [batch, heads, tokens, 128]
 * given by element strides of batch / head / token (last dimension contiguous, strides multiples of 8), out likewise;
 * tokens % 128 == 0.  Scores and softmax statistics in fp32, probabilities rounded to bf16 before the product with v
 * (as the tensor operations of the reference's Llama attention core do on unquantized operands,
 * models/llama/modeling_llama.py:362-480); no [tokens, tokens] matrix is materialised and no workspace is needed.
 * MASE_ERR_SHAPE for another head dimension or token count, MASE_ERR_DTYPE for another dtype. */
int mase_attention_causal(const void* q, const void* k, const void* v, void* out, size_t batch, size_t heads,
                          size_t tokens, size_t head_dim, size_t q_stride_b, size_t q_stride_h, size_t q_stride_t,
                          size_t k_stride_b, size_t k_stride_h, size_t k_stride_t, size_t v_stride_b, size_t v_stride_h,
                          size_t v_stride_t, size_t o_stride_b, size_t o_stride_h, size_t o_stride_t, int dtype,
                          float scaling, void* stream);
/* The same with work of the neighbouring operations folded in, each part optional:
 *   q_cos / q_sin (both or neither; bf16 tables [batch or 1, tokens, 128] with element strides cs_stride_b (0 for a
 *   table shared by the batch) and cs_stride_t, multiples of 8): q is given BEFORE its rotary embedding, which is
 *   applied as q is loaded with the roundings of mase_rope (nn/quantized/functional/rope.py:17-27);
 *   element_bits != 0: the result is written as its MXINT quantize-dequantize (blocks of 32 along the head dimension,
 *   E8M0 scales; log2_tab as for mase_mxint_qdq in bf16): what the LinearMXInt that reads the
 *   [batch, tokens, heads * 128] result would compute from it in a pass of its own
 *   (nn/quantized/modules/linear.py:956-972), bit for bit. */
int mase_attention_causal_fused(const void* q, const void* k, const void* v, void* out, size_t batch, size_t heads,
                                size_t tokens, size_t head_dim, size_t q_stride_b, size_t q_stride_h, size_t q_stride_t,
                                size_t k_stride_b, size_t k_stride_h, size_t k_stride_t, size_t v_stride_b,
                                size_t v_stride_h, size_t v_stride_t, size_t o_stride_b, size_t o_stride_h,
                                size_t o_stride_t, int dtype, float scaling, const void* q_cos, const void* q_sin,
                                size_t cs_stride_b, size_t cs_stride_t, int element_bits, const uint32_t* log2_tab,
                                void* stream);

/* Transposed copy of the trailing two dimensions of a 16-bit tensor: in[o][i][r][c] (row stride in_stride_row, batch
 * strides in_stride_outer / in_stride_inner, all in elements, columns contiguous) -> out[o][i][c][r] contiguous with r
 * padded with zeros to rows_padded (the next multiple of 64).  Prepares the second operand of the reference's
 * torch.matmul / torch.bmm calls ([K, N] rows: the values of an attention block,
 * nn/quantized/modules/llama/attention.py:449; y of bmm_mx*, nn/quantized/functional/matmul.py:437-512) for
 * mase_gemm_bf16_tn_batched, which contracts rows with rows.  cols % 8 == 0; strides multiples of 8; pointers 16-byte
 * aligned; at most 65535 batch items per call. */
int mase_transpose16(const void* in, void* out, size_t batch_outer, size_t batch_inner, size_t rows, size_t cols,
                     size_t rows_padded, size_t in_stride_outer, size_t in_stride_inner, size_t in_stride_row, void* stream);

/* Rotary embedding out = x * cos + rotate_half(x) * sin for x [B, H, T, D] with the last dimension contiguous and
 * element strides (x_stride_b, x_stride_h, x_stride_t); out has the same strides; cos / sin tables [B or 1, T, D] with
 * strides (cs_stride_b, cs_stride_t), cs_stride_b = 0 for one table shared by the batch.  Products and sum are rounded to
 * dtype one by one, as the tensor operations of _apply_rope round them (nn/quantized/functional/rope.py:17-27).
 * D % 16 == 0, all strides multiples of 8. */
int mase_rope(const void* x, const void* cos, const void* sin, void* out, size_t B, size_t H, size_t T, size_t D,
              size_t x_stride_b, size_t x_stride_h, size_t x_stride_t, size_t cs_stride_b, size_t cs_stride_t, int dtype,
              void* stream);

/* test/diagnostic helpers (host only, no device work) */
uint32_t mase_isclose_zero_threshold_bits(int dtype); /* largest |x| (fp32 bits) that isclose(x, 0) accepts */
float mase_round_scalar_to_dtype(double v, int dtype); /* how a clamp bound is represented in dtype */

#ifdef __cplusplus
}
#endif
#endif /* MASE_AMD_H */
