/* C ABI of libawq_hip.so, part 2 -- the kernels of a Qwen3 decode step that sit between the AWQ
 * linears (include/awq_hip.h): residual add + RMSNorm, per-head q/k RMSNorm + rotary + KV-cache
 * write, attention of one new token per sequence over a paged KV cache, SiLU(gate) * up.
 *
 * Conventions are those of awq_hip.h: device pointers, dense row-major tensors, `dtype` is AWQ_F16
 * or AWQ_BF16 for every 16-bit tensor of a call, `stream` is a hipStream_t as void*, the return
 * value is an awq_status and awq_hip_last_error() holds the message of a failure.
 *
 * The reference runs these steps as torch modules inside its model (no kernels, no KV cache);
 * citations name the module code whose arithmetic each entry point reproduces.
 */
#ifndef NQ_ENGINE_OPS_H_
#define NQ_ENGINE_OPS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* residual [rows, hidden] += delta (skipped when delta is NULL; the sum is rounded to dtype as
 * `x + sublayer(x)` is), then y = dtype(residual_f32 * rsqrt(mean(residual_f32^2) + eps)) * weight.
 * hidden % 8 == 0, hidden <= 8192.
 * RMSNorm.rms_norm, nanoquantization/layers/norm.py:18-32; the residual adds of
 * Qwen3QuantizedBlock.forward, nanoquantization/models/qwen3_quantized.py:194-215. */
int nq_add_rmsnorm(void* residual, const void* delta, const void* weight, void* y, int64_t rows,
                   int64_t hidden, float eps, int dtype, void* stream);

/* ssq [ceil(hidden / 128)][rows] (fp32): ssq[t][r] = sum of squares of x[r, 128 t .. 128 t + 127], in the summation
 * order of nq_add_rmsnorm.  The RMSNorm statistics that awq_gemv_rmsnorm (include/awq_hip.h) reads, for a residual
 * stream that no awq_gemv_add_residual has produced (the embedding output of a decode step).  hidden % 8 == 0,
 * hidden <= 8192.  The mean of squares of RMSNorm.rms_norm, nanoquantization/layers/norm.py:18-32. */
int nq_row_ssq(const void* x, float* ssq, int64_t rows, int64_t hidden, int dtype, void* stream);
/* The same with the embedding lookup in front: x_out[r] = table[ids[r]] (ids clamped to [0, table_rows)), ssq of x_out.
 * Qwen3QuantizedModel.forward's embed_tokens, nanoquantization/models/qwen3_quantized.py:259-273. */
int nq_embed_row_ssq(const int64_t* ids, const void* table, void* x_out, float* ssq, int64_t rows, int64_t hidden,
                     int64_t table_rows, int dtype, void* stream);

/* qkv [rows, (num_heads + 2*num_kv_heads) * head_dim] is the output of the q|k|v projections
 * side by side.  Every q and k head is RMS-normalised (q_weight / k_weight, [head_dim]) and rotated
 * (half-split rotary, angle table cos_sin f32 [max_positions, head_dim] = cos | sin) at
 * positions[row]; q goes to q_out [rows, num_heads, head_dim], k and the untouched v go to
 * k_cache / v_cache [num_slots / block_size, num_kv_heads, block_size, head_dim] (a head's tokens of one
 * block are contiguous) at slot slots[row] = block * block_size + offset (a row whose slot is outside
 * [0, num_slots) writes no k/v).  If k_out is not NULL the normalised, rotated k heads are also written
 * densely to k_out [rows, num_kv_heads, head_dim] (what a causal prefill attention over the same rows
 * reads).  head_dim even, <= 256.
 * Qwen3QuantizedAttention.forward, nanoquantization/models/qwen3_quantized.py:79-93;
 * RoPE.apply_rope / forward, nanoquantization/layers/rope.py:24-45. */
int nq_qk_norm_rope_store(const void* qkv, const void* q_weight, const void* k_weight,
                          const float* cos_sin, const int64_t* positions, const int64_t* slots,
                          void* q_out, void* k_out, void* k_cache, void* v_cache, int64_t rows, int64_t num_heads,
                          int64_t num_kv_heads, int64_t head_dim, int64_t max_positions,
                          int64_t num_slots, int64_t block_size, float eps, int dtype, void* stream);

/* Bytes of device workspace nq_paged_attention_decode needs (0 is possible); no initialisation
 * needed.  max_context = block_size * max_blocks_per_seq. */
size_t nq_paged_attention_workspace_bytes(int64_t batch, int64_t num_heads, int64_t num_kv_heads,
                                          int64_t head_dim, int64_t max_context);

/* out[b, h, :] = softmax(scale * q[b, h, :] . K_b^T) V_b over the first context_lens[b] tokens of
 * sequence b (the new token's k/v already written).  Token t of sequence b is token t % block_size
 * of block block_table[b, t / block_size] in k_cache / v_cache
 * [num_blocks, num_kv_heads, block_size, head_dim]; query head h reads kv head
 * h / (num_heads / num_kv_heads).  q, out: [batch, num_heads, head_dim].  head_dim 64 or 128,
 * num_heads / num_kv_heads in {1, 2, 4, 8} -- with head_dim 128 and block_size % 16 == 0 any ratio up to 16 (Qwen3-14B
 * has 5); block indices are clamped to the cache.
 * F.scaled_dot_product_attention(..., enable_gqa) of Qwen3QuantizedAttention.forward,
 * nanoquantization/models/qwen3_quantized.py:94-99, restricted to the last query position. */
int nq_paged_attention_decode(const void* q, const void* k_cache, const void* v_cache,
                              const int32_t* block_table, const int32_t* context_lens, void* out,
                              int64_t batch, int64_t num_heads, int64_t num_kv_heads,
                              int64_t head_dim, int64_t block_size, int64_t max_blocks_per_seq,
                              int64_t num_blocks, float scale, int dtype, void* workspace,
                              size_t workspace_bytes, void* stream);

/* out[r, i] = dtype(SiLU(gate_up[r, i])) * gate_up[r, inter + i]; gate_up [rows, 2*inter] is the
 * output of the gate|up projections side by side, out [rows, inter].  inter % 8 == 0.
 * Qwen3QuantizedMLP.forward, nanoquantization/models/qwen3_quantized.py:147-152. */
int nq_silu_mul(const void* gate_up, void* out, int64_t rows, int64_t inter, int dtype, void* stream);

/* The same for gate|up interleaved in words of 8 columns (word 2t = gate outputs 8t..8t+7, word 2t+1 = the up
 * columns of the same outputs): the output layout of a plain product with the interleaved buffers of
 * awq_gemv_swiglu (include/awq_hip.h). */
int nq_silu_mul_interleaved(const void* gate_up, void* out, int64_t rows, int64_t inter, int dtype, void* stream);

/* out[r] = argmax_i logits[r, i] as int64, the lowest index among equal maxima (NaNs are never selected);
 * logits [rows, vocab] dense.  Greedy sampling for the engine's decode loop; the reference has no generation
 * loop, the logits are those of Qwen3QuantizedForCausalLM.forward
 * (nanoquantization/models/qwen3_quantized.py:312-314). */
int nq_argmax_rows(const void* logits, int64_t* out, int64_t rows, int64_t vocab, int dtype, void* stream);

/* Bookkeeping of a decode step over the paged cache (the reference has no generation loop; one launch each instead of
 * a dozen elementwise ones).  `active` is one byte per row (torch.bool).
 * nq_decode_prepare: slots[r] = active[r] ? block_table[r][positions[r] / block_size] * block_size +
 *   positions[r] % block_size : -1 (the slot convention of nq_qk_norm_rope_store), context_lens[r] = positions[r] + 1.
 * nq_decode_advance: out_log[step[0]][r] = next_tokens[r] (skipped when step[0] is outside [0, out_rows)),
 *   ids[r] = next_tokens[r], positions[r] += active[r], step[0] += 1. */
int nq_decode_prepare(const int64_t* positions, const uint8_t* active, const int32_t* block_table, int64_t* slots,
                      int32_t* context_lens, int64_t rows, int64_t max_blocks, int64_t block_size, void* stream);
int nq_decode_advance(const int64_t* next_tokens, const uint8_t* active, int64_t* out_log, int64_t* ids,
                      int64_t* positions, int64_t* step, int64_t rows, int64_t out_rows, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NQ_ENGINE_OPS_H_ */
