/*
 * metaseq_amd.h - C ABI of libmetaseq_amd.so: hand-written gfx950 (MI355X) HIP kernels
 * for metaseq's OPT incremental-decoding forward path.
 *
 * Conventions
 *   - every entry point returns 0 on success and a negative msa_status otherwise;
 *     msa_last_error() returns a thread-local description of the last failure.
 *   - all pointers are DEVICE pointers unless the name ends in _host; the library never
 *     allocates or frees device memory on behalf of these calls; `stream` is a hipStream_t
 *     (NULL = the default stream).  Nothing synchronises: work is enqueued on `stream`.
 *   - fp16 tensors are IEEE binary16, row-major, innermost dimension contiguous.
 *   - "round" below means round-to-nearest-even to fp16.  Every kernel accumulates in fp32
 *     and rounds at exactly the points where the reference materialises an fp16 tensor.
 *
 * Each declaration cites the reference code (paths relative to the metaseq tree) whose
 * arithmetic it replaces.
 */
#ifndef METASEQ_AMD_H
#define METASEQ_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  MSA_OK = 0,
  MSA_ERR_INVALID_ARG = -1, /* null pointer, bad shape, unsupported size  */
  MSA_ERR_CAPACITY = -2,    /* sequence longer than the cache / table      */
  MSA_ERR_HIP = -3          /* a HIP runtime call or kernel launch failed  */
} msa_status;

/* epilogue flags for msa_linear_f16 / msa_linear_w8a16 */
#define MSA_EPI_RELU 1u /* y = max(y, 0) after the bias add                       */

const char* msa_last_error(void);
int msa_version(void);

/* Pre-LN LayerNorm forward: y[r,:] = round(gamma * (x[r,:] - mean) * rsqrt(var + eps) + beta),
 * mean / biased variance in fp32.  D % 8 == 0, D <= 16384.
 * Replaces metaseq/modules/layer_norm.py:28-33 -> apex cuApplyLayerNorm
 * (metaseq/modules/apex/layer_norm_cuda_kernel.cu:441-455, host :868-893). */
int msa_layernorm_f16(const void* x, const void* gamma, const void* beta, void* y,
                      int64_t rows, int D, float eps, void* stream);

/* Token + learned-position embedding for the last `T_out` columns of tokens[B, n]:
 *   pos(b,t) = pad_idx                      if tokens[b,t] == pad_idx
 *            = pad_idx + #non-pad in tokens[b, 0..t]   otherwise
 *   x[b*T_out + j, :] = round(E[tokens[b,t], :] + P[pos(b,t), :]),  t = n - T_out + j
 * tokens are int64 with row stride `tok_stride` elements.  positions_out (optional, int64
 * [B, T_out]) receives pos.  Ids outside [0,V) or positions >= n_pos_rows set *status_dev
 * (optional int32) to 1 and are clamped.
 * Replaces TransformerDecoder.forward_embedding (metaseq/models/transformer_decoder.py:263-346),
 * utils.make_positions (metaseq/utils.py:83-93), LearnedPositionalEmbedding.forward
 * (metaseq/modules/learned_positional_embedding.py:30-54) and VocabParallelEmbedding.forward
 * (metaseq/modules/megatron/mpu/layers.py:220-250). */
int msa_embed_f16(const int64_t* tokens, int64_t tok_stride, int B, int n, int T_out,
                  const void* E, int V, const void* P, int n_pos_rows, int pad_idx, int D,
                  void* x, int64_t* positions_out, int32_t* status_dev, void* stream);

/* y[M,N] = epilogue(x[M,K] . W[N,K]^T):
 *   t = round(acc); if bias: t = round(t + bias[n]); if RELU: t = max(t,0);
 *   if residual: t = round(t + residual[m,n]);  y[m,n] = t.
 * K % 32 == 0, N % 8 == 0.  M <= 64 selects the weight-streaming kernel (HBM bound),
 * larger M the LDS-tiled MFMA kernel.  `workspace` (fp32, >= msa_linear_workspace_bytes)
 * is used for split-K partial sums and tile counters and must be zero on first use; the
 * kernels leave the counter region zero again.
 * Replaces LinearWithGradAccumulationAndAsyncCommunication.forward
 * (metaseq/modules/megatron/mpu/layers.py:290-292) as used by qkv_proj
 * (metaseq/modules/multihead_attention.py:316), out_proj (:553, bias and residual added in
 * metaseq/modules/transformer_decoder_layer.py:222-230), fc1/fc2
 * (metaseq/modules/feedforward.py:19-22; residual transformer_decoder_layer.py:283) and the
 * tied vocabulary projection (metaseq/models/transformer_decoder.py:413-420). */
int msa_linear_f16(const void* x, const void* W, const void* bias, const void* residual,
                   void* y, int64_t M, int N, int K, unsigned flags, void* workspace,
                   size_t workspace_bytes, void* stream);

/* Same contract with int8 weights Wq[N,K] and per-output-channel fp16 scales[N]:
 * the product uses the dequantised weight round(Wq[n,k] * scales[n]) (formed in registers).
 * No reference counterpart: the reference hands int8 serving to FasterTransformer
 * (metaseq/scripts/convert_metaseq_ft.py:99-133); semantics are the benchmark's definition. */
int msa_linear_w8a16(const void* x, const int8_t* Wq, const void* scales, const void* bias,
                     const void* residual, void* y, int64_t M, int N, int K, unsigned flags,
                     void* workspace, size_t workspace_bytes, void* stream);

size_t msa_linear_workspace_bytes(int64_t M, int N, int K);

/* Fused QKV projection: kvq = round(round(x . Wqkv^T) + bqkv) with rows of Wqkv ordered
 * K | V | Q; then for row m = b*T + t and head h:
 *   Kcache[b,h,S0+t,:] = k,  Vcache[b,h,S0+t,:] = v,  q_out[m, h*hd:(h+1)*hd] = round(q * hd^-0.5).
 * Caches are [B, H, S_cap, hd] fp16.  Same size rules as msa_linear_f16 with N = 3*H*hd.
 * Replaces metaseq/modules/multihead_attention.py:316-319 (projection + split), :429
 * (q scaling) and :449-479 (cache growth by torch.cat, here an in-place append). */
int msa_qkv_proj_f16(const void* x, const void* Wqkv, const void* bqkv, void* q_out,
                     void* Kcache, void* Vcache, int B, int T, int H, int hd, int S0, int S_cap,
                     int K, void* workspace, size_t workspace_bytes, void* stream);
int msa_qkv_proj_w8a16(const void* x, const int8_t* Wq, const void* scales, const void* bqkv,
                       void* q_out, void* Kcache, void* Vcache, int B, int T, int H, int hd,
                       int S0, int S_cap, int K, void* workspace, size_t workspace_bytes,
                       void* stream);

/* Causal attention of T new queries (already scaled, q[B*T, H*hd]) over the cache, whose
 * positions 0 .. S0+T-1 are valid: query t sees keys 0 .. S0+t.
 *   s = round(q . k);  s = -inf where key_pad_mask[b, key] != 0;
 *   p = round(softmax_fp32(s));  out[b*T+t, h*hd:(h+1)*hd] = round(sum_key p * v).
 * key_pad_mask (optional) is uint8 [B, mask_stride].  hd in {64, 128}.  T == 1 is the
 * bandwidth-bound decode kernel; T > 1 the prefill kernel.
 * Replaces metaseq/modules/multihead_attention.py:492 (bmm q k^T), :516-531 (causal and
 * padding masks), :533-534 (fp32 softmax, cast back), :543-552 (bmm p v, transpose). */
int msa_attention_f16(const void* q, const void* Kcache, const void* Vcache,
                      const uint8_t* key_pad_mask, int64_t mask_stride, void* out, int B, int H,
                      int hd, int T, int S0, int S_cap, void* stream);

/* One step of greedy selection over fp16 logits[B, V] (row stride ld_logits), with the
 * generator's bookkeeping fused in:
 *   z = logits / temperature (only if temperature > 0 and != 1);
 *   lprob(v) = (z[v] - max z) - log(sum(exp(z - max z))) in fp32 over ALL v; if any z is NaN every
 *   lprob of the row is -inf;
 *   ids in banned_host[0..n_banned) -> -inf (pad always, eos and stop ids while step < min_len);
 *   if force_eos_all != 0 (last step) or finished[b] != 0, only eos_idx stays eligible;
 *   tok[b*tok_stride] = lowest index attaining the max lprob; score[b*score_stride] = that max;
 *   finished[b] |= tok == eos_idx or tok in stop_host[0..n_stop).
 * banned_host / stop_host are HOST arrays of at most 16 ids, copied into the launch.
 * finished (uint8[B], device, in/out) is optional.
 * Replaces the per-step vocabulary passes of SequenceGenerator._generate
 * (metaseq/sequence_generator.py:272-308, :319-323), _sample_topp's greedy branch (:413-415)
 * and BaseDecoder.get_normalized_probs (metaseq/models/base_decoder.py:95-100). */
int msa_greedy_select_f16(const void* logits, int64_t ld_logits, int B, int V, float temperature,
                          const int32_t* banned_host, int n_banned, const int32_t* stop_host,
                          int n_stop, uint8_t* finished, int force_eos_all, int eos_idx,
                          int64_t* tok, int64_t tok_stride, float* score, int64_t score_stride,
                          void* stream);

/* Log-probabilities of given target ids under fp16 logits rows:
 *   out[r] = logits[r, target[r]]/temperature - logsumexp_fp32(logits[r,:]/temperature).
 * Replaces the prompt scoring gather of SequenceGenerator._generate
 * (metaseq/sequence_generator.py:235-258). */
int msa_target_logprob_f16(const void* logits, int64_t ld_logits, int64_t rows, int V,
                           float temperature, const int64_t* target, float* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* METASEQ_AMD_H */
