/* C ABI of libawq_hip.so -- the MI355X (gfx950) AWQ W4A16 linear path.
 *
 * Every pointer is a DEVICE pointer on the current HIP device unless said
 * otherwise; `stream` is a hipStream_t passed as void* (NULL = default stream).
 * Tensors are dense row-major:
 *   qweight int32 [K, N/8]   nibble j of a word = logical column 8i + {0,2,4,6,1,3,5,7}[j]
 *   qzeros  int32 [K/g, N/8] same nibble order
 *   qscales f16|bf16 [K/g, N]
 *   x       f16|bf16 [M, K]      y  f16|bf16 [M, N]     bias f16|bf16 [N] or NULL
 * `dtype` is AWQ_F16 or AWQ_BF16 and names the type of x, qscales, bias and y.
 * Inputs are borrowed and never written.  Calls are asynchronous on `stream`
 * and return an awq_status; awq_hip_last_error() gives the message of the
 * last failing call on the calling thread.
 *
 * Citations name the interface of the reference (liyuan24/nanoquantization)
 * that an entry point stands in for.
 */
#ifndef AWQ_HIP_H_
#define AWQ_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    AWQ_OK = 0,
    AWQ_ERR_INVALID_ARG = 1,  /* null pointer, bad shape, bad dtype                       */
    AWQ_ERR_UNSUPPORTED = 2,  /* a shape/group size this build has no kernel for          */
    AWQ_ERR_WORKSPACE = 3,    /* workspace missing or smaller than *_workspace_bytes()    */
    AWQ_ERR_HIP = 4           /* the HIP runtime refused the launch                       */
} awq_status;

typedef enum { AWQ_F16 = 0, AWQ_BF16 = 1 } awq_dtype;

/* Library version (major*10000 + minor*100 + patch). */
int awq_hip_version(void);

/* Message of the last failing call on this thread ("" if none). Host pointer, do not free. */
const char* awq_hip_last_error(void);

/* out[k, 8i+c] = RN_dtype(float(q - z) * s), bit-exact with the reference's
 * dequantised weight.  out: dtype [K, N].
 * Replaces awq_dequantize(qweight, qscales, qzeros) + awq_dequantize_kernel,
 * nanoquantization/layers/gemm.py:126-180 and :10-123. */
int awq_dequantize(const int32_t* qweight, const void* qscales, const int32_t* qzeros, void* out,
                   int64_t K, int64_t N, int64_t group_size, int dtype, void* stream);

/* The same weight transposed: out [N, K] row-major (k-contiguous rows), out[n, k] = awq_dequantize's [k, n],
 * bit for bit.  This is the layout a dense GEMM library multiplies fastest (y = x @ out^T); the host layer
 * uses it for the reference's large-M branch, awq_dequantize + torch.matmul,
 * nanoquantization/layers/gemm.py:558-561.  K % 64 == 0; group sizes 8, 16, 32 or a multiple of 64. */
int awq_dequantize_transposed(const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                              void* out, int64_t K, int64_t N, int64_t group_size, int dtype,
                              void* stream);

/* Offline path: weight f32 [N, K] (the nn.Linear layout) -> packed AWQ buffers in one pass:
 * per group of `group_size` input features s = max(max - min, 1e-5) / 15,
 * z = clamp(-round(min / s), 0, 15), q = clamp(round(w / s) + z, 0, 15); qweight [K, N/8] and
 * qzeros [K/g, N/8] hold q and z in the nibble order above, qscales [K/g, N] holds s in `dtype`.
 * fp32 arithmetic with true divisions and round-half-to-even, word for word what
 * pseudo_quantize(w, g, 4, zero_point=True) (nanoquantization/utils/quantization.py:5-58), the
 * transposes of awq/quantizer.py:156-158 and WQLinear_GEMM.from_linear
 * (nanoquantization/layers/gemm.py:447-550) produce for an fp32 weight.  The weight must hold no NaN. */
int awq_quantize_pack(const float* weight, int32_t* qweight, void* qscales, int32_t* qzeros,
                      int64_t N, int64_t K, int64_t group_size, int dtype, void* stream);

/* Bytes of device workspace awq_gemv / awq_gemm / awq_linear need for this
 * problem (0 is possible).  The workspace must be zero-filled ONCE when it is
 * allocated; every call leaves it in that state (its counters are reset by
 * the kernel), so it can be reused by later calls on the same stream.  Calls
 * that share a workspace must not overlap in time. */
size_t awq_gemv_workspace_bytes(int64_t M, int64_t N, int64_t K);
size_t awq_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
size_t awq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* Decode regime, 1 <= M <= 16 (up to 128 rows where N % 128 == 0 and group_size % 128 == 0: batched
 * decode, as blocks of 16 rows): y = x @ dequant(W) (+ bias), fp32 accumulation, split-K with a
 * fixed-order (run-to-run bit-stable) reduction, inside the kernel or, from 5 rows on the widest and
 * from 17 rows on the largest weights, as a second kernel on the same stream.
 * Replaces awq_gemm(x, qweight, qscales, qzeros, split_k_iters) for small M:
 * nanoquantization/layers/gemm.py:329-379 (kernel :183-326, torch.zeros :361,
 * out.sum :378). */
int awq_gemv(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
             const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size,
             int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* awq_gemv for callers that cannot allocate device memory or bring a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): same arguments without the workspace, same kernels, same bits.
 * The split-K scratch (arrival counters + fp32 partials) is a static device array of
 * awq_gemv_static_scratch_bytes() = 16 KiB + 16 MiB inside the library, held by every GPU the library runs on until
 * the process ends; its address is looked up once per device on the first call there.  The call allocates nothing
 * (no hipMalloc / hipFree, no allocating library routine).  A problem whose split-K plan needs more scratch than
 * that (awq_gemv_workspace_bytes(M, N, K) tells) is refused with AWQ_ERR_UNSUPPORTED: every 1..16-row shape of the
 * Qwen3 family fits, 64-row calls on the widest MLP weights do not.  All calls on one GPU share the array: calls that
 * overlap in time on one GPU (two streams, two threads) race; calls ordered on one stream do not.  The counters are
 * zero at load and every launch leaves them zero.  It has no counterpart in the reference. */
size_t awq_gemv_static_scratch_bytes(void);
int awq_gemv_static(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                    const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size, int dtype,
                    void* stream);

/* awq_gemv with the gate/up epilogue of the MLP fused in.  The packed buffers hold the gate and the up
 * projection interleaved word by word along N: packed word column 2t = the 8 gate columns 8t..8t+7,
 * word column 2t+1 = the up columns of the same outputs (qzeros and qscales alike), N = 2 * intermediate.
 * y [M, N/2] = dtype(SiLU(dtype(x @ Wgate))) * dtype(x @ Wup), the rounding points of the reference's
 * F.silu(self.gate_proj(x)) * self.up_proj(x), nanoquantization/models/qwen3_quantized.py:147-152.
 * M <= 64, N % 128 == 0, group_size % 128 == 0; workspace as for awq_gemv(M, N, K). */
int awq_gemv_swiglu(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                    void* y, int64_t M, int64_t N, int64_t K, int64_t group_size, int dtype,
                    void* workspace, size_t workspace_bytes, void* stream);

/* The same gated product for any M: the GEMV above for M <= 64 where it applies, the pipelined MFMA GEMM with the
 * gate applied in its epilogue otherwise (K % 64 == 0, N % 16 == 0).  Same interleaved buffers, y [M, N/2].
 * Replaces the two linears and the activation of Qwen3QuantizedMLP.forward,
 * nanoquantization/models/qwen3_quantized.py:147-152, for prefill as well as decode. */
size_t awq_linear_swiglu_workspace_bytes(int64_t M, int64_t N, int64_t K);
int awq_linear_swiglu(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                      void* y, int64_t M, int64_t N, int64_t K, int64_t group_size, int dtype,
                      void* workspace, size_t workspace_bytes, void* stream);

/* awq_gemv on the fused q|k|v projection of a decode step with what follows it fused in (head_dim 128, so a
 * 128-column tile is one head): per-head RMSNorm of q and k, half-split rotary at positions[row], q written to
 * q_out [M, num_heads, 128], k and v to slot slots[row] of the paged cache [blocks, kv heads, block_size, 128]
 * (a negative slot writes no k/v).  N = (num_heads + 2 * num_kv_heads) * 128, M <= 64, N % 128 == 0,
 * group_size % 128 == 0; cos_sin fp32 [max_positions, 128] (64 cosines, 64 sines); workspace as for
 * awq_gemv(M, N, K).  Same arithmetic as awq_gemv followed by nq_qk_norm_rope_store (include/nq_engine_ops.h):
 * Qwen3QuantizedAttention.forward, nanoquantization/models/qwen3_quantized.py:79-92. */
int awq_gemv_qkv_rope_store(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                            const void* q_weight, const void* k_weight, const float* cos_sin,
                            const int64_t* positions, const int64_t* slots, void* q_out, void* k_cache,
                            void* v_cache, int64_t M, int64_t N, int64_t K, int64_t group_size,
                            int64_t num_heads, int64_t num_kv_heads, int64_t max_positions, int64_t num_slots,
                            int64_t block_size, float eps, int dtype, void* workspace, size_t workspace_bytes,
                            void* stream);

/* A decode step without stand-alone residual-add + RMSNorm launches (Qwen3QuantizedBlock.forward,
 * nanoquantization/models/qwen3_quantized.py:194-215: x + attn(norm(x)), x + mlp(norm(x))).  The statistics
 * travel between the GEMVs as ssq, fp32 [hidden / 128][M]: ssq[t][m] = sum of squares of residual[m, 128 t .. 128 t + 127]
 * (8 consecutive squares per lane by fused multiply-add in column order, 16 lanes combined by xor 8, 4, 2, 1; the
 * tiles are added in index order).  nq_row_ssq (include/nq_engine_ops.h) produces the same statistics for a residual
 * stream that comes from elsewhere (the embedding), and nq_add_rmsnorm sums in the same order, so every entry point
 * below returns the bits of the separate kernels.  All of them: M <= 64, N % 128 == 0, K % 128 == 0,
 * group_size % 128 == 0, no bias, workspace as for awq_gemv(M, N, K).
 *
 * awq_gemv_add_residual: residual [M, N] = dtype(residual + dtype(x @ W)) in place (o_proj, down_proj), and
 *   ssq [N / 128][M] of the new residual.
 * awq_gemv_rmsnorm: y = (RMSNorm(x) * norm_weight) @ W with x [M, K] the residual stream and ssq [K / 128][M] its
 *   statistics: the operand is h = dtype(dtype(x * rsqrt(sum(ssq[:, m]) / K + norm_eps)) * norm_weight), the
 *   arithmetic of RMSNorm.rms_norm, nanoquantization/layers/norm.py:18-32.  gated != 0: the interleaved gate/up
 *   buffers and the SiLU(gate) * up epilogue of awq_gemv_swiglu, y [M, N / 2].
 * awq_gemv_rmsnorm_qkv_rope_store: awq_gemv_qkv_rope_store with the same prologue on x. */
int awq_gemv_add_residual(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                          void* residual, float* ssq, int64_t M, int64_t N, int64_t K, int64_t group_size,
                          int dtype, void* workspace, size_t workspace_bytes, void* stream);
/* awq_gemv_add_rmsnorm: the residual add and the RMSNorm that follow o_proj and down_proj in
 * Qwen3QuantizedBlock.forward (nanoquantization/models/qwen3_quantized.py:194-215; RMSNorm.add_rms_norm,
 * nanoquantization/layers/norm.py:34-50) inside the GEMV's second pass: residual [M, N] = dtype(residual +
 * dtype(x @ W)) in place and normed [M, N] = dtype(dtype(residual * rsqrt(mean(residual^2) + norm_eps)) * norm_weight),
 * the bits of awq_gemv followed by nq_add_rmsnorm.  Only for problems whose plan (awq_gemv_plan) is a shared-chunk
 * variant (name "wide...") without the in-kernel tail (no trailing 't') and with split_k > 1, and N <= 8192; others
 * are refused with AWQ_ERR_UNSUPPORTED and take the two calls.  Workspace as for awq_gemv(M, N, K). */
int awq_gemv_add_rmsnorm(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                         void* residual, const void* norm_weight, float norm_eps, void* normed, int64_t M, int64_t N,
                         int64_t K, int64_t group_size, int dtype, void* workspace, size_t workspace_bytes,
                         void* stream);
int awq_gemv_rmsnorm(const void* x, const float* ssq, const void* norm_weight, float norm_eps,
                     const int32_t* qweight, const void* qscales, const int32_t* qzeros, void* y, int64_t M,
                     int64_t N, int64_t K, int64_t group_size, int gated, int dtype, void* workspace,
                     size_t workspace_bytes, void* stream);
int awq_gemv_rmsnorm_qkv_rope_store(const void* x, const float* ssq, const void* norm_weight, float norm_eps,
                                    const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                                    const void* q_weight, const void* k_weight, const float* cos_sin,
                                    const int64_t* positions, const int64_t* slots, void* q_out, void* k_cache,
                                    void* v_cache, int64_t M, int64_t N, int64_t K, int64_t group_size,
                                    int64_t num_heads, int64_t num_kv_heads, int64_t max_positions,
                                    int64_t num_slots, int64_t block_size, float eps, int dtype, void* workspace,
                                    size_t workspace_bytes, void* stream);

/* Optional hint for latency-bound decode loops: names a region [ptr, ptr + bytes) -- meant to be the packed
 * qweight of the launch AFTER the next one -- that the next linear call of the calling thread (any awq_gemv*,
 * awq_gemm*, awq_linear* entry point) may pull into the 256 MB Infinity Cache.  That call takes every pending
 * region on entry, before it checks its arguments: if it runs the one-tile staged GEMV and leaves compute units
 * idle it launches a few spare workgroups that read the regions; any other kernel, and any error return, drops
 * them.  Hints therefore never outlive the next linear call and never change results.  Up to four regions
 * (qweight, qscales, qzeros ...) can be pending; further ones are ignored.  ptr must be 128-byte aligned and stay
 * mapped until that next call's kernel has run; NULL clears the pending hints.  No reference counterpart (the
 * reference launches each linear on its own). */
int awq_prefetch_hint(const void* ptr, size_t bytes);
/* Number of regions pending on the calling thread (0..4); host-only, for callers and tests that want to see the
 * rule above at work.  No reference counterpart. */
int awq_prefetch_pending(void);

/* Prefill regime, any M >= 1 (meant for M > 16): fused dequant + MFMA GEMM,
 * y = x @ dequant(W) (+ bias), W rounded to dtype exactly as the reference
 * does before the product, fp32 accumulation.
 * Replaces awq_dequantize + torch.matmul, nanoquantization/layers/gemm.py:559-561,
 * and awq_gemm for 16 < M < 256, :562-564. */
int awq_gemm(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
             const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size,
             int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* The whole forward of one AWQ linear: picks the regime from M (awq_gemv for
 * M <= 16, up to 64 where it takes the shape, and up to 128 on weights of at most 20 Mi elements;
 * awq_gemm above) and applies the bias.
 * A K that is a multiple of 32 but not of 64 (which awq_gemm does not take) is served by
 * awq_gemv in blocks of 16 rows.  Replaces WQLinear_GEMM.forward, nanoquantization/layers/gemm.py:552-567
 * (the reshape of x/y to 2-D stays with the caller). */
int awq_linear(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
               const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size,
               int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* awq_gemv / awq_gemm with the launch configuration forced, for tuning and for
 * tests that must reach every compiled variant.  `variant` indexes the
 * kernel-shape table (see awq_gemv_variant_count / awq_gemm_variant_count),
 * `split_k` >= 1 is the number of K-splits across workgroups.  No reference
 * counterpart (the reference exposes block sizes as keyword arguments of
 * awq_gemm, nanoquantization/layers/gemm.py:334-337). */
int awq_gemv_variant_count(void);
int awq_gemm_variant_count(void);
const char* awq_gemv_variant_name(int variant);
const char* awq_gemm_variant_name(int variant);
/* The variant and K-split that awq_gemv / awq_gemm pick by themselves for a problem (host-only: no device call), so
 * that a caller can see, log or pin what will run: awq_gemv_ex / awq_gemm_ex with the returned pair launch exactly
 * what awq_gemv / awq_gemm launch for the same arguments.  The GEMM's choice depends on the tensor type and the
 * group size as well as on the shape (which of the two 256 x 256 kernels runs), the workspace size does not.  The
 * rules are tuned for the 256 compute units of a whole MI355X; on a partition with fewer the results are the same
 * and only the balance of the launch is not the best one. */
int awq_gemv_plan(int64_t M, int64_t N, int64_t K, int64_t group_size, int* variant, int* split_k);
int awq_gemm_plan(int64_t M, int64_t N, int64_t K, int64_t group_size, int dtype, int* variant, int* split_k);
size_t awq_gemv_ex_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant, int split_k);
size_t awq_gemm_ex_workspace_bytes(int64_t M, int64_t N, int64_t K, int variant, int split_k);
int awq_gemv_ex(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size,
                int dtype, void* workspace, size_t workspace_bytes, void* stream, int variant,
                int split_k);
int awq_gemm_ex(const void* x, const int32_t* qweight, const void* qscales, const int32_t* qzeros,
                const void* bias, void* y, int64_t M, int64_t N, int64_t K, int64_t group_size,
                int dtype, void* workspace, size_t workspace_bytes, void* stream, int variant,
                int split_k);

#ifdef __cplusplus
}
#endif
#endif /* AWQ_HIP_H_ */
