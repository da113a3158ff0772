/*
 * e2h_quant.h -- C ABI of libe2h_quant.so: the weight-only quantized linear path of gpt-accelera's
 * models/quantize.py as hand-written HIP kernels for AMD MI355X (gfx950).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer into memory the caller owns; nothing here allocates, frees
 *     or synchronises.  Kernels are enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     default stream) and are safe to record into a HIP graph.
 *   - bfloat16 values travel as uint16_t bit patterns.
 *   - every entry point returns E2H_OK (0) or a negative E2H_ERR_* code; no exception crosses the ABI.
 *     e2h_status_string() names a code.
 *   - "reference" below is gpt-accelera (Edward-Sun/easy-to-hard), file models/quantize.py unless
 *     another file is named.
 */
#ifndef E2H_QUANT_H
#define E2H_QUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define E2H_ABI_VERSION 1

#define E2H_OK 0
#define E2H_ERR_NULL_POINTER (-1)      /* a required pointer is NULL */
#define E2H_ERR_BAD_SHAPE (-2)         /* m/n/k violate the reference's shape asserts */
#define E2H_ERR_BAD_GROUPSIZE (-3)     /* groupsize not in {32,64,128,256} or does not divide k */
#define E2H_ERR_BAD_INNER_K_TILES (-4) /* inner_k_tiles not in {2,4,8} or 16*ikt does not divide k */
#define E2H_ERR_MISALIGNED (-5)        /* a pointer is not aligned as documented */
#define E2H_ERR_LAUNCH (-6)            /* the HIP runtime rejected the launch */
#define E2H_ERR_NO_DEVICE (-7)         /* no gfx950 device is current */
#define E2H_ERR_BAD_OPTION (-8)        /* unknown option name or value out of range */
#define E2H_ERR_SCRATCH_TOO_SMALL (-9) /* the call needs more scratch than the fixed built-in buffer holds */

/* Library identity / diagnostics (no reference counterpart). */
int e2h_abi_version(void);
const char *e2h_status_string(int status);

/* Tuning knobs for experiments: launch-geometry overrides such as "int4_rows_per_wave", "int4_k_slices", "int4_k_groups",
 * "int4_col_waves", "int8_rows_per_wave", "int8_k_groups", "int8_k_slices", "int8_force_generic", "row_tiles", "int4_no_xsum",
 * "int4_no_gemm32", "int4_gemm32_min_rows", "int4_gemm_tile", "int8_gemm_tile", "int8_gemm_waves", "int8_gemm_wave_cols", "attention_waves",
 * "attention_no_mfma", "staged_tiles", "staged_slices", "staged_no_rows64";
 * value 0 restores the built-in heuristic.  Not thread safe; set before launching. */
int e2h_set_option(const char *name, int value);

/* ------------------------------------------------------------------------------------------------
 * int8, per-output-channel symmetric
 * ---------------------------------------------------------------------------------------------- */

/* dynamically_quantize_per_channel(x, -128, 127, torch.int8), reference :39-71.
 *   w          [n, k] row-major; float32 if w_is_bf16 == 0 (what the reference's callers pass,
 *              :357-359 and :388-390), bfloat16 if w_is_bf16 != 0 (converted exactly to float32 on
 *              the fly, i.e. the same result as quantizing weight.float()).
 *   q          [n, k] int8 codes.
 *   scales_f32 [n] float32 scales (the function's second return value); may be NULL.
 *   scales_bf16[n] the same scales rounded to bfloat16 (what the handler stores, :392); may be NULL.
 * IEEE float32 division, round-half-even, clamp to [-128, 127]; scale >= float32 eps.
 * Requires 16-byte aligned w and 4-byte aligned q rows when k % 4 == 0 (any k is accepted). */
int e2h_int8_quantize_per_channel(const void *w, int w_is_bf16, int8_t *q, float *scales_f32,
                                  uint16_t *scales_bf16, int64_t n, int64_t k, void *stream);

/* WeightOnlyInt8Linear.forward, reference :428-429:  y = F.linear(x, weight.to(bf16)) * scales.
 *   x [m, k] bf16, q [n, k] int8, scales [n] bf16, y [m, n] bf16.  float32 accumulation; the result
 *   is rounded to bfloat16 before and after the multiplication by the scale, as in the reference.
 * Any m >= 1, n >= 1, k >= 1 (k % 128 == 0 with 16-byte aligned x and q takes the streaming kernel).
 * workspace / workspace_bytes: optional scratch as for e2h_int4_mm (NULL / 0 allowed). */
int e2h_int8_mm(const uint16_t *x, const int8_t *q, const uint16_t *scales, uint16_t *y, int64_t m,
                int64_t n, int64_t k, void *workspace, int64_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------------------
 * int4, group-wise asymmetric
 * ---------------------------------------------------------------------------------------------- */

/* get_group_qparams(w, 4, groupsize), reference :74-92.  w [n, k] bf16 -> scales, zeros [n, k/g] bf16.
 * bfloat16 arithmetic: every step is computed in float32 and rounded to bfloat16 (ties to even). */
int e2h_int4_group_qparams(const uint16_t *w, uint16_t *scales, uint16_t *zeros, int64_t n, int64_t k,
                           int groupsize, void *stream);

/* group_quantize_tensor_from_qparams(w, scales, zeros, 4, groupsize), reference :118-144.
 * w [n, k] bf16, scales/zeros [n, k/g] bf16 -> codes [n, k] int32 in 0..15. */
int e2h_int4_quantize_from_qparams(const uint16_t *w, const uint16_t *scales, const uint16_t *zeros,
                                   int32_t *codes, int64_t n, int64_t k, int groupsize, void *stream);

/* group_quantize_tensor(w, 4, groupsize), reference :147-151 (get_group_qparams +
 * group_quantize_tensor_from_qparams + pack_scales_and_zeros :95-109) in one pass.
 * -> codes [n, k] int32, scales_and_zeros [k/g, n, 2] bf16 ([..,0] scale, [..,1] zero). */
int e2h_int4_group_quantize(const uint16_t *w, int32_t *codes, uint16_t *scales_and_zeros, int64_t n,
                            int64_t k, int groupsize, void *stream);

/* torch.ops.aten._convert_weight_to_int4pack(codes, inner_k_tiles) as called at reference :439-441
 * and :585-587 (PyTorch 2.2.0 CUDA nibble order).
 * codes [n, k] int32 (0..15) -> packed [n/8, k/(16*ikt), 32, ikt/2] int32.  n % 8 == 0, k % (16*ikt) == 0. */
int e2h_int4_pack(const int32_t *codes, int32_t *packed, int64_t n, int64_t k, int inner_k_tiles,
                  void *stream);

/* Inverse of e2h_int4_pack (test aid and checkpoint inspection; no reference counterpart). */
int e2h_int4_unpack(const int32_t *packed, int32_t *codes, int64_t n, int64_t k, int inner_k_tiles,
                    void *stream);

/* prepare_int4_weight_and_scales_and_zeros(weight_bf16, groupsize, inner_k_tiles), reference :435-442,
 * fused: bf16 weight -> tile-packed codes + scales_and_zeros without materialising the int32 codes. */
int e2h_int4_quantize_pack(const uint16_t *w, int32_t *packed, uint16_t *scales_and_zeros, int64_t n,
                           int64_t k, int groupsize, int inner_k_tiles, void *stream);

/* group_dequantize_tensor_from_qparams, reference :154-171, applied to the tile-packed weight:
 * w_out [n, k] bf16 = bf16(bf16((q - 8) * scale) + zero). */
int e2h_int4_dequantize(const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *w_out,
                        int64_t n, int64_t k, int groupsize, int inner_k_tiles, void *stream);

/* group_dequantize_tensor_from_qparams(w_int32, scales, zeros, 4, groupsize), reference :154-171, on
 * plain codes: codes [n, k] int32, scales/zeros [n, k/g] bf16 -> w_out [n, k] bf16
 * = bf16(bf16((q - 8) * scale) + zero).  Any groupsize >= 2 dividing k. */
int e2h_int4_dequantize_codes(const int32_t *codes, const uint16_t *scales, const uint16_t *zeros,
                              uint16_t *w_out, int64_t n, int64_t k, int groupsize, void *stream);

/* torch.ops.aten._weight_int4pack_mm(x, packed, groupsize, scales_and_zeros) as called by
 * linear_forward_int4, reference :445-453 (WeightOnlyInt4Linear.forward :658-666).
 *   x [m, k] bf16, packed [n/8, k/(16*ikt), 32, ikt/2] int32, scales_and_zeros [k/g, n, 2] bf16
 *   -> y [m, n] bf16,  y[m,n] = sum_k x[m,k] * ((q[n,k] - 8) * scale[k/g, n] + zero[k/g, n]),
 * float32 accumulation.  n % 8 == 0, k % g == 0, k % (16*ikt) == 0, g in {32,64,128,256},
 * ikt in {2,4,8}; x, packed, scales_and_zeros 16-byte aligned; any m >= 1.
 *   workspace  optional scratch of workspace_bytes bytes (16-byte aligned; e2h_workspace_bytes() is the
 *              recommended size) that lets small problems split K across workgroups.  It must be zero
 *              when first used and is left zeroed where it matters by every launch; launches that share
 *              it must be ordered on one stream.  NULL / 0 selects the single-slice kernels.
 * Every kernel behind this entry point forms exact bf16 x code products and applies scale and zero per group in
 * float32, so a row's result does not depend on how many rows share the call.  Only with
 * e2h_set_option("int4_gemm_tile", 256) calls of more than 64 rows (k % 256 == 0, g <= 128, ikt 8) run a kernel that
 * rounds every weight to bfloat16 first (the arithmetic of the kernel the reference calls; 15-20 % faster at thousands
 * of rows): results then differ from the default by that rounding, for every row of such a call alike. */
int e2h_int4_mm(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *y,
                int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles, void *workspace,
                int64_t workspace_bytes, void *stream);

/* e2h_int4_mm for callers that cannot allocate or pass scratch memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, checks and results (bit for
 * bit) as e2h_int4_mm, but the split-K tickets and partial tiles live in a fixed buffer inside the library
 * (e2h_int4_mm_static_scratch_bytes() = 64 KiB of tickets + 8 MiB of tiles, one copy per GPU, held until the process
 * ends), and nothing is allocated or freed.  Limits: m <= 64 (decode batches); a shape whose launch geometry would need
 * more scratch than the buffer holds returns E2H_ERR_SCRATCH_TOO_SMALL (no 7B / 34B linear at m <= 64 does).  All calls
 * on one GPU share the buffer: calls that overlap on one GPU (two streams) race; order them on one stream.  The first
 * call on a device resolves the buffer's device address (hipGetSymbolAddress); make that call before capturing a
 * graph. */
int e2h_int4_mm_static_scratch(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *y,
                               int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles, void *stream);
int64_t e2h_int4_mm_static_scratch_bytes(void);

/* Gated feed-forward front half in one launch:  y = F.silu(w1(x)) * w3(x)  for two WeightOnlyInt4Linear
 * modules of equal shape (FeedForward.forward, reference models/model.py:343-344, with linear_forward_int4
 * :445-453 for each product).  Rounding points as the reference's bfloat16 tensors: each product is rounded
 * to bfloat16, silu's result is rounded, the final product is rounded.
 *   x [m, k] bf16, packed_gate / packed_up [n/8, k/128, 32, 4] int32, sz_gate / sz_up [k/g, n, 2] bf16
 *   -> y [m, n] bf16.  1 <= m <= 64 (decode batches; larger m: call e2h_int4_mm twice and e2h_silu_mul),
 *   inner_k_tiles == 8, g in {32,64,128}, k % 128 == 0, n % 8 == 0; 16-byte aligned inputs. */
int e2h_int4_mm_silu_gate(const uint16_t *x, const int32_t *packed_gate, const uint16_t *sz_gate,
                          const int32_t *packed_up, const uint16_t *sz_up, uint16_t *y, int64_t m, int64_t n,
                          int64_t k, int groupsize, int inner_k_tiles, void *stream);

/* Decode-step attention front half in one launch: the fused q|k|v projection of a WeightOnlyInt4Linear
 * (Attention.forward, reference models/model.py:283-296: wqkv, split, apply_rotary_emb on q and k :400-412,
 * KVCache.update :94-104) for ONE new token per sequence.  Row b of x is sequence b.
 *   x [batch, k] bf16, packed [n/8, k/128, 32, 4] int32 with n = (n_head + 2*n_kv_head) * head_dim,
 *   scales_and_zeros [k/g, n, 2] bf16, freqs_cis [>= cache_len, head_dim/2, 2] bf16 (cos, sin),
 *   input_pos [1] int64 on the device (the position being written; a position outside [0, cache_len)
 *   writes nothing).
 *   -> q_out [batch, n_head, head_dim] bf16 (rotated), k_cache / v_cache [batch, n_kv_head, cache_len,
 *   head_dim] bf16 updated at input_pos (k rotated).  The projection is rounded to bfloat16 before the
 *   rotation, which is evaluated in float32 and rounded again, as in the reference.
 * 1 <= batch <= 64, inner_k_tiles == 8, g in {32,64,128}, k % 128 == 0, n % 8 == 0, head_dim even. */
int e2h_int4_mm_rope_kv(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros,
                        const uint16_t *freqs_cis, uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache,
                        const int64_t *input_pos, int64_t batch, int64_t n_head, int64_t n_kv_head,
                        int64_t head_dim, int64_t cache_len, int64_t k, int groupsize, int inner_k_tiles,
                        void *stream);

/* int8 forms of the two fused decode-step launches above (WeightOnlyInt8Linear modules, reference
 * models/quantize.py:405-429, in FeedForward.forward models/model.py:343-344 and Attention.forward :283-296).
 * Each linear's output is formed with the reference's two roundings, bf16(bf16(x @ q^T) * scales), before the SiLU-gate
 * or the rotation is applied, so the results equal the unfused sequence of calls bit for bit.
 *   q_* int8 [n, k] row-major, scales_* bf16 [n]; 1 <= m (batch) <= 64, k % 128 == 0, 16-byte aligned x and q rows;
 *   the other arguments as in e2h_int4_mm_silu_gate / e2h_int4_mm_rope_kv. */
int e2h_int8_mm_silu_gate(const uint16_t *x, const int8_t *q_gate, const uint16_t *scales_gate, const int8_t *q_up,
                          const uint16_t *scales_up, uint16_t *y, int64_t m, int64_t n, int64_t k, void *stream);
int e2h_int8_mm_rope_kv(const uint16_t *x, const int8_t *q, const uint16_t *scales, const uint16_t *freqs_cis, uint16_t *q_out,
                        uint16_t *k_cache, uint16_t *v_cache, const int64_t *input_pos, int64_t batch, int64_t n_head,
                        int64_t n_kv_head, int64_t head_dim, int64_t cache_len, int64_t k, void *stream);

/* Recommended size in bytes of the workspace accepted by the matmul entry points (no reference counterpart). */
int64_t e2h_workspace_bytes(void);

/* ------------------------------------------------------------------------------------------------
 * Decode-step kernels around the quantized linears (callers of the hot path; stock-op equivalents in the
 * reference's models/model.py).  bf16 everywhere, float32 arithmetic inside.
 * ---------------------------------------------------------------------------------------------- */

/* Single-query attention over the KV cache, reference Attention.forward models/model.py:310-349 with
 * KVCache :112-129 and the mask of Transformer.forward :221-228, for one new token per sequence.
 *   q [batch, n_head, head_dim]; k_cache, v_cache [>= batch, n_kv_head, cache_len, head_dim]; out [batch, n_head, head_dim].
 *   input_pos: device pointer to the position of the new token (positions 0..pos are attended);
 *   left_pad_mask_pos: NULL or device [batch]: positions below it are masked except the new token itself.
 * head_dim in {64, 128}; n_head / n_kv_head in {1, 2, 4, 8}. */
int e2h_decode_attention(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out,
                         const int64_t *input_pos, const int64_t *left_pad_mask_pos, int64_t batch,
                         int64_t n_head, int64_t n_kv_head, int64_t cache_len, int64_t head_dim, float scale,
                         void *stream);

/* RMSNorm, reference models/model.py:363-377: y = bf16(bf16(x * rsqrt(mean(x^2) + eps)) * weight). x, y [rows, dim]. */
int e2h_rmsnorm(const uint16_t *x, const uint16_t *weight, uint16_t *y, int64_t rows, int64_t dim, float eps,
                void *stream);

/* Residual add + RMSNorm in one pass (TransformerBlock.forward, reference :279-282):
 * h_out = bf16(x + delta), y = RMSNorm(h_out).  All [rows, dim]. */
int e2h_add_rmsnorm(const uint16_t *x, const uint16_t *delta, const uint16_t *weight, uint16_t *h_out,
                    uint16_t *y, int64_t rows, int64_t dim, float eps, void *stream);

/* The wo / w2 projection of a decoder block and the residual add + RMSNorm that consumes it (TransformerBlock.forward,
 * reference models/model.py:279-283; the projections are WeightOnlyInt4Linear.forward, models/quantize.py:445-453), as a
 * pair of launches that never meet inside the matmul: for up to 64 rows of x, inner_k_tiles 8 and group size <= 128,
 * e2h_int4_mm_partials writes the float32 sums of `slices` contiguous parts of K to partials [slices, m, n] (row-major),
 * and e2h_add_rmsnorm_partials forms delta = bf16(partials[0] + partials[1] + ... in that order) -- bit for bit the
 * value e2h_int4_mm stores for the same operands -- before h_out = bf16(x + delta), y = RMSNorm(h_out).
 * e2h_int4_mm_partial_slices returns the number of slices the library uses for a shape (>= 1; it depends on the shape
 * and on e2h_set_option only), or a negative status for shapes this form does not take; e2h_int4_mm_partials rejects
 * any other `slices`.  No workspace is involved.  The bit-for-bit statement holds for e2h_int4_mm called with a workspace
 * of at least e2h_workspace_bytes() and default options; with a smaller or no workspace, or with launch-geometry options
 * set, e2h_int4_mm may split K differently (or not at all) and the two then agree to float32 rounding only.
 * The int8 pair (WeightOnlyInt8Linear.forward, models/quantize.py:428-429; K % 128 == 0, 16-byte aligned rows) hands on the
 * unscaled sums; col_scales [n] bf16 (NULL for int4) makes the consumer form delta = bf16(bf16(sum) * scale[column]), the
 * linear's two roundings. */
int e2h_int4_mm_partial_slices(int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles);
int e2h_int4_mm_partials(const uint16_t *x, const int32_t *packed, const uint16_t *scales_and_zeros, float *partials,
                         int64_t m, int64_t n, int64_t k, int groupsize, int inner_k_tiles, int slices, void *stream);
int e2h_int8_mm_partial_slices(int64_t m, int64_t n, int64_t k);
int e2h_int8_mm_partials(const uint16_t *x, const int8_t *q, float *partials, int64_t m, int64_t n, int64_t k, int slices,
                         void *stream);
int e2h_add_rmsnorm_partials(const uint16_t *x, const float *partials, int slices, const uint16_t *col_scales,
                             const uint16_t *weight, uint16_t *h_out, uint16_t *y, int64_t rows, int64_t dim, float eps,
                             void *stream);

/* ------------------------------------------------------------------------------------------------
 * Decode batches on staged activations.  The single-token steps of the decode loop (reference
 * inference_generate.py:123-157, decode_one_token :110-120) give every quantized linear at most a few dozen rows;
 * these entry points are linear_forward_int4 (reference :445-453) and its callers for that case with the activations
 * handed from kernel to kernel in matrix-core operand order instead of row-major [m, k]:
 *
 *   staged buffer for m rows (1 <= m <= 64) of k values (k % 128 == 0), mpad = m rounded up to 16,
 *   e2h_int4_staged_bytes(m, k) = mpad*k*2 + (k/128)*mpad*32 bytes, 16-byte aligned:
 *     bf16 [k/32][mpad][32]   the 64-byte piece of row r and 32-wide k segment p; inside it dword 4j + i holds the
 *                             row's dwords j + 4i of the segment (values k = 32p + 2(j+4i), +1) -- the k order of the
 *                             packed weight words, so a matrix-core lane loads its operand with one 16-byte load;
 *     f32  [k/128][mpad][8]   sums over each run of 16 consecutive k (balanced tree in index order).
 *   Rows m .. mpad-1 may hold anything.
 *
 * Common limits: inner_k_tiles == 8 weights, g in {32, 64, 128}, n % 16 == 0, k % 128 == 0, 1 <= m <= 64, and a
 * launch geometry for the shape (e2h_int4_mm_staged_supported tells; every 7B / 34B linear has one) -- otherwise
 * E2H_ERR_BAD_SHAPE, and the row-major entry points above take the call.  Results: float32 accumulation of exact
 * products, scale and zero applied per group in float32, fixed summation order (run-to-run identical); they agree with
 * the row-major entry points to bfloat16 rounding of the result, not bit for bit (the sums over K are split differently).
 * ---------------------------------------------------------------------------------------------- */

/* Size of a staged buffer (see above), or a negative status. */
int64_t e2h_int4_staged_bytes(int64_t m, int64_t k);

/* x [m, k] bf16 row-major -> staged (one pass; padding rows are written as zeros).  No reference counterpart: it is the
 * layout conversion for activations that do not come from one of the producing kernels below. */
int e2h_int4_stage_x(const uint16_t *x, void *staged, int64_t m, int64_t k, void *stream);

/* 1 if a staged decode-batch kernel exists for the shape and epilogue (0 = e2h_int4_mm_staged, 1 = _silu_gate,
 * 2 = _rope_kv, 3 = _partials, 4 = _argmax), else 0. */
int e2h_int4_mm_staged_supported(int64_t m, int64_t n, int64_t k, int groupsize, int epilogue);

/* linear_forward_int4, reference :445-453: y [m, n] bf16 = staged x times the packed weight. */
int e2h_int4_mm_staged(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, uint16_t *y, int64_t m,
                       int64_t n, int64_t k, int groupsize, void *stream);

/* Greedy next token straight from the LM head (reference inference_generate.py:110-120 with sampling switched off:
 * torch.argmax over the logits of the last position; models/model.py:247 is the head): tokens[r] = argmax_n of
 * bf16(staged x times the packed weight)[r, n] without the logits ever being stored -- every workgroup of the matmul
 * reduces its columns to one candidate per row, a second small launch picks each row's best.  The same answer as
 * e2h_argmax_rows over e2h_int4_mm_staged's result (lowest index among ties, a NaN counts as the maximum).
 *   scratch: e2h_int4_mm_staged_argmax_scratch_bytes(m, n, k, groupsize) bytes (or a negative status), 8-byte aligned,
 *   overwritten; tokens int64 [m]. */
int64_t e2h_int4_mm_staged_argmax_scratch_bytes(int64_t m, int64_t n, int64_t k, int groupsize);
int e2h_int4_mm_staged_argmax(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, void *scratch,
                              int64_t *tokens, int64_t m, int64_t n, int64_t k, int groupsize, void *stream);

/* The same product left as float32 sums over `slices` contiguous parts of K, partials [slices, m, n], for
 * e2h_add_rmsnorm_staged to add in slice order (the wo / w2 projections of a decoder block, reference
 * models/model.py:279-283).  e2h_int4_mm_staged_partial_slices returns the library's slice count for the shape (>= 1) or
 * a negative status; any other `slices` is rejected.  (33 .. 64 rows run a kernel of their own that covers all rows in
 * one pass over the weights; same arguments, same layout of the result.) */
int e2h_int4_mm_staged_partial_slices(int64_t m, int64_t n, int64_t k, int groupsize);
int e2h_int4_mm_staged_partials(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, float *partials,
                                int64_t m, int64_t n, int64_t k, int groupsize, int slices, void *stream);

/* F.silu(w1(x)) * w3(x) (FeedForward.forward, reference models/model.py:359-360) with the rounding points of
 * e2h_int4_mm_silu_gate.  y [m, n] bf16 row-major and / or staged_out, the result in staged form for the w2 projection
 * (n % 128 == 0 then); at least one of the two must be given. */
int e2h_int4_mm_staged_silu_gate(const void *staged, const int32_t *packed_gate, const uint16_t *sz_gate, const int32_t *packed_up,
                                 const uint16_t *sz_up, uint16_t *y, void *staged_out, int64_t m, int64_t n, int64_t k,
                                 int groupsize, void *stream);

/* e2h_int4_mm_rope_kv on staged activations: fused q|k|v projection, RoPE, cache write (reference models/model.py:321-333
 * with :400-412 and :121-129); arguments as there. */
int e2h_int4_mm_staged_rope_kv(const void *staged, const int32_t *packed, const uint16_t *scales_and_zeros, const uint16_t *freqs_cis,
                               uint16_t *q_out, uint16_t *k_cache, uint16_t *v_cache, const int64_t *input_pos, int64_t batch,
                               int64_t n_head, int64_t n_kv_head, int64_t head_dim, int64_t cache_len, int64_t k, int groupsize,
                               void *stream);

/* RMSNorm (reference models/model.py:363-377) with the optional residual add of TransformerBlock.forward (:279-282) in
 * front -- e2h_rmsnorm, e2h_add_rmsnorm and e2h_add_rmsnorm_partials in one entry point -- whose normalised rows go to y
 * (row-major, may be NULL) and / or to `staged` (may be NULL; rows <= 64 and dim % 128 == 0 then).  Exactly as those
 * three: delta bf16 [rows, dim] or partials float32 [slices, rows, dim] (col_scales as there) or neither; h_out is
 * required with delta / partials and unused otherwise.  The staged values are bit for bit the values of y. */
int e2h_add_rmsnorm_staged(const uint16_t *x, const uint16_t *delta, const float *partials, int slices, const uint16_t *col_scales,
                           const uint16_t *weight, uint16_t *h_out, uint16_t *y, void *staged, int64_t rows, int64_t dim, float eps,
                           void *stream);

/* e2h_decode_attention whose result [batch, n_head * head_dim] goes to `out` (row-major, may be NULL) and / or to
 * `staged` (may be NULL), the input of the output projection; batch <= 64 and n_head * head_dim % 128 == 0 with staged. */
int e2h_decode_attention_staged(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out, void *staged,
                                const int64_t *input_pos, const int64_t *left_pad_mask_pos, int64_t batch, int64_t n_head,
                                int64_t n_kv_head, int64_t cache_len, int64_t head_dim, float scale, void *stream);

/* Measurement aid, no reference counterpart: one launch of 256 workgroups that only reads `bytes` (a multiple of 16,
 * < 2 GB) of device memory at src with streaming 16-byte loads and writes nothing (sink may be NULL).  It is the floor
 * of what a launch that has to read that many bytes of weights can cost on this machine; bytes == 0 is an empty launch.
 * With shared_bytes > 0 every workgroup additionally reads all of `shared` (a multiple of 16, < 2 GB): the pattern of
 * a decode batch's activations, which every CU needs whole next to its share of the weights. */
int e2h_stream_read_probe(const void *src, int64_t bytes, const void *shared, int64_t shared_bytes, uint32_t *sink, void *stream);

/* apply_rotary_emb (reference :400-412) on the q and k parts of a fused qkv row + KVCache.update (:121-129) for
 * one new token per sequence.  qkv [batch, (n_head + 2 n_kv_head) * head_dim]; freqs_cis [positions, head_dim/2, 2]
 * bf16 (cos, sin); q_out [batch, n_head, head_dim]; caches as above, written at *input_pos. */
int e2h_rope_kv_write(const uint16_t *qkv, const uint16_t *freqs_cis, uint16_t *q_out, uint16_t *k_cache,
                      uint16_t *v_cache, const int64_t *input_pos, int64_t batch, int64_t n_head,
                      int64_t n_kv_head, int64_t cache_len, int64_t head_dim, void *stream);

/* The same for seqlen new tokens per sequence (prefill, scoring): qkv [batch * seqlen, (n_head + 2 n_kv_head) * head_dim]
 * with row b * seqlen + t, input_pos [seqlen] int64 on the device, q_out [batch, n_head, seqlen, head_dim] (head-major,
 * as scaled_dot_product_attention takes it, reference :296 transposes to it); k (rotated) and v go to
 * [batch, n_kv_head, cache_len, head_dim] at row input_pos[t], or at row t when rows_by_token != 0 (a pass without
 * KV cache: fresh k / v tensors with cache_len = seqlen; the rotation still uses input_pos[t]).  Rows outside
 * [0, cache_len) are not written. */
int e2h_rope_kv_write_seq(const uint16_t *qkv, const uint16_t *freqs_cis, uint16_t *q_out, uint16_t *k_cache,
                          uint16_t *v_cache, const int64_t *input_pos, int64_t batch, int64_t seqlen, int64_t n_head,
                          int64_t n_kv_head, int64_t cache_len, int64_t head_dim, int rows_by_token, void *stream);

/* F.silu(a) * b with bf16 rounding after each op (reference FeedForward.forward :359-360). n elements, n % 8 == 0. */
int e2h_silu_mul(const uint16_t *a, const uint16_t *b, uint16_t *y, int64_t n, void *stream);

/* Next-token sampling, reference inference_generate.py:53-85 (sample -> logits_to_probs ->
 * multinomial_sample_one_no_sync) on the last position's logits:
 *   l = float(logits) / max(temperature, 1e-5);  with top_k > 0: l = (l < k-th largest l of the row) ? -inf : l;
 *   probs = softmax(l);  idx = argmax(probs / q).
 *   logits [rows, >= vocab] bf16 with row_stride elements between rows; q [rows, vocab] float32, the Exp(1) draws
 *   (the caller makes them, as the reference does with exponential_(1)); probs [rows, vocab] float32 out;
 *   idx [rows] int32 out.  top_k == 0 or top_k >= vocab: no truncation.  Ties at the pivot all survive. */
int e2h_sample_top_k(const uint16_t *logits, int64_t row_stride, const float *q, float *probs, int32_t *idx,
                     int64_t rows, int64_t vocab, float temperature, int top_k, void *stream);

/* Greedy next token: idx[r] = argmax(float(logits[r, :])) (the harness's temperature-free path; the reference's
 * torch.argmax over the last position's logits, inference_generate.py:110-120 with sampling switched off).
 *   logits bf16, row r starts at logits + r * row_stride (row_stride >= vocab, in elements); idx int64 [rows].
 * Ties go to the lowest index; a NaN counts as the largest value (ATen's arg-max convention). */
int e2h_argmax_rows(const uint16_t *logits, int64_t row_stride, int64_t *idx, int64_t rows, int64_t vocab, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* E2H_QUANT_H */
