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
 *   - the calls act on the calling thread's current device and may be made from several
 *     threads and for several devices of one process, a msa_decoder handle (below) included:
 *     the handle is read-only after msa_decoder_create, every call's state lives in its own
 *     arguments and workspace.
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

/* flags */
#define MSA_EPI_RELU 1u   /* y = max(y, 0) after the bias add                                  */
#define MSA_IN_PACKED 2u  /* the input activation is in the packed layout (M <= 128, see below)*/
#define MSA_OUT_PACKED 4u /* write the output activation in the packed layout (M <= 128)       */
#define MSA_EMBED_COL_FROM_LEN 8u /* msa_embed_f16: the new token sits in column len_dev[b]      */
#define MSA_EMBED_ROWS_GIVEN 32u /* msa_embed_f16: E holds the B*T_out token embeddings themselves */
/* per-row bits of the optional `row_mode` array of the selection entry points */
#define MSA_ROW_BAN_EARLY 1u /* eos_idx and the stop ids are not eligible for this row (the row
                                has not reached its minimum length)                             */
#define MSA_ROW_ONLY_EOS 2u  /* only eos_idx is eligible for this row (its last allowed step)   */
#define MSA_ROW_SKIP 4u      /* msa_sample_topp_f16: leave this row's outputs untouched          */

const char* msa_last_error(void);
int msa_version(void);

/* ---- memory layouts --------------------------------------------------------------------------
 * Weights are consumed in a TILE-PACKED layout: the 16 x 32 block of W[N,K] that one
 * v_mfma_f32_16x16x32_f16 reads as its A operand is one contiguous KB in lane order, and the
 * blocks of a 16-row tile follow each other along K, so a wave instruction reads a whole KB and
 * a tile's K sweep is one linear HBM stream.
 *   fp16: block (t = n/16, ks = k/32) at half offset (t*K/32 + ks)*512; lane l = 16*((k%32)/8) +
 *         n%16 owns halves 8l..8l+7 = W[n][8*(k/8) .. +7].                N % 16 == 0, K % 32 == 0.
 *   int8: block (t, ks8 = k/64) at byte offset (t*K/64 + ks8)*1024; lane l = 16g + r owns 16 bytes:
 *         0..7 = W[16t+r][64ks8 + 8g ..+7], 8..15 = W[16t+r][64ks8 + 32 + 8g ..+7], each byte
 *         stored biased (q + 128, unsigned).                                     K % 64 == 0.
 * The pack / unpack calls convert from / to row-major [N,K] (src != dst).
 * Activations of at most 128 rows may be PACKED the same way (the MFMA B operand in lane order):
 * with MB = ceil(M/16) row blocks up to 64 rows and MB = 8 for 65 .. 128 rows, element (m,k) sits
 * at half offset
 *   ((k/32*MB + m/16)*64 + 16*((k%32)/8) + m%16)*8 + k%8;   the buffer holds MB*16*K halves.
 * No reference counterpart: the reference keeps torch's row-major tensors
 * (metaseq/modules/megatron/mpu/layers.py:290). */
int msa_pack_weight_f16(const void* src, void* dst, int N, int K, void* stream);
int msa_unpack_weight_f16(const void* src, void* dst, int N, int K, void* stream);
int msa_pack_weight_i8(const int8_t* src, int8_t* dst, int N, int K, void* stream);
int msa_unpack_weight_i8(const int8_t* src, int8_t* dst, int N, int K, void* stream);
/* Tile-packed int8 weights Wq with per-output-channel fp16 scales[N] -> tile-packed fp16 weights
 * Wp (N*K halves), every element round(Wq[n,k] * scales[n]): exactly the values the w8a16 kernels
 * form in registers, so msa_linear_f16 / msa_qkv_proj_f16 on Wp compute the product
 * msa_linear_w8a16 / msa_qkv_proj_w8a16 compute on Wq.  For products of thousands of rows
 * (prefill), where expanding a matrix once (3 bytes moved per weight) and running the fp16 kernel
 * beats dequantising every fragment in every workgroup.  K % 64 == 0.  No reference counterpart
 * (see msa_linear_w8a16). */
int msa_expand_weight_w8_f16(const int8_t* Wq, const void* scales, void* Wp, int N, int K,
                             void* stream);

/* ---- device-resident per-row sequence lengths -------------------------------------------------
 * The entry points of a decode step (T == 1) take an optional `len_dev`: int32 [B] on the device,
 * len_dev[b] = number of positions of row b already in the KV cache (= the number of non-pad
 * tokens of its history before the new one); NULL = use the host arguments, every row at S0.
 * With it, rows of one batch may have different lengths (right-padded prompts, requests that
 * joined a running batch at different times): each row appends at, and attends up to, its own
 * length, and pads are never stored.  A NEGATIVE entry marks a row as inactive (an empty slot):
 * nothing is appended or attended for it and its outputs are undefined.  A captured hipGraph
 * bakes no length into its launch arguments and replays for every step.
 *   msa_embed_f16 (T_out == 1): position = pad_idx + 1 + len_dev[b] (no scan of the history);
 *                               the token is column n - 1 of the row, or column len_dev[b] with
 *                               MSA_EMBED_COL_FROM_LEN (a full-history token buffer, no pads);
 *                               step_len_out (optional int32 [B]) receives len_dev[b], or -1 if
 *                               the row is inactive or its new token is a pad: passed on as the
 *                               `len_dev` of the step's other kernels and as the gate of
 *                               msa_advance_len, it keeps such a row out of the step, the way
 *                               the reference masks a pad for good;
 *   msa_qkv_proj_* (T == 1):    row b appends at position len_dev[b] (skipped if >= S_cap);
 *   msa_attention_f16 (T == 1): row b attends positions 0 .. len_dev[b];
 *   msa_greedy_select_f16 and the fused forms: the output column is len_dev[0] (graph replay of
 *                               a batch whose rows all have the same length).
 * msa_advance_len adds `delta` to those of the n entries of len_dev that are not negative and
 * whose gate entry (optional int32 [n]) is not negative either, on the stream.
 * No reference counterpart: the reference re-launches every op from Python each step and keeps
 * pads inside its key/value history, masked (metaseq/modules/multihead_attention.py:485-531). */
int msa_advance_len(int32_t* len_dev, const int32_t* gate, int n, int delta, void* stream);

/* Pre-LN LayerNorm forward: y[r,:] = round(gamma * (x[r,:] - mean) * rsqrt(var + eps) + beta),
 * mean / biased variance in fp32.  D % 8 == 0, D <= 16384.  flags: MSA_OUT_PACKED.
 * Replaces metaseq/modules/layer_norm.py:28-33 -> apex cuApplyLayerNorm
 * (metaseq/modules/apex/layer_norm_cuda_kernel.cu:441-455, host :868-893). */
int msa_layernorm_f16(const void* x, const void* gamma, const void* beta, void* y,
                      int64_t rows, int D, float eps, unsigned flags, void* stream);

/* Tail of a split-K linear layer fused with the LayerNorm that follows it:
 *   x[r,:] = round(round(round(sum_{s<S} part[s][r,:]) + bias) + x[r,:])          (in place)
 *   y[r,:] = LayerNorm(x[r,:]; gamma, beta)      (skipped when gamma, beta and y are all NULL)
 * part is fp32 [S, rows, D] as written by msa_linear_partial_*.  flags: MSA_OUT_PACKED (y).
 * Replaces the bias and residual adds of metaseq/modules/transformer_decoder_layer.py:222-230
 * (attention block) and :283 with metaseq/modules/megatron/mpu/layers.py:669-671 (fc2 bias),
 * followed by the LayerNorm at :275, the next layer's :264 or the final one at
 * metaseq/models/transformer_decoder.py:392-393. */
int msa_residual_layernorm_f16(const float* part, int S, const void* bias, void* x,
                               const void* gamma, const void* beta, void* y, int64_t rows, int D,
                               float eps, unsigned flags, void* stream);

/* Token + learned-position embedding for the last `T_out` columns of tokens[B, n]:
 *   pos(b,t) = pad_idx                      if tokens[b,t] == pad_idx
 *            = pad_idx + #non-pad in tokens[b, 0..t]   otherwise
 *   x[b*T_out + j, :] = round(E[tokens[b,t], :] + P[pos(b,t), :]),  t = n - T_out + j
 * tokens are int64 with row stride `tok_stride` elements.  positions_out (optional, int64
 * [B, T_out]) receives pos.  Ids outside [0,V) or positions >= n_pos_rows set *status_dev
 * (optional int32) to 1 and are clamped.  flags: MSA_EMBED_COL_FROM_LEN (with len_dev);
 * MSA_EMBED_ROWS_GIVEN: E is not the table but fp16 [B*T_out, D], the token embeddings of the
 * embedded columns as the caller computed them (the reference's `token_embeddings` argument);
 * `tokens` then only says where the pads are.
 * Replaces TransformerDecoder.forward_embedding (metaseq/models/transformer_decoder.py:263-346),
 * utils.make_positions (metaseq/utils.py:83-93), LearnedPositionalEmbedding.forward
 * (metaseq/modules/learned_positional_embedding.py:30-54) and VocabParallelEmbedding.forward
 * (metaseq/modules/megatron/mpu/layers.py:220-250). */
int msa_embed_f16(const int64_t* tokens, int64_t tok_stride, int B, int n, int T_out,
                  const void* E, int V, const void* P, int n_pos_rows, int pad_idx, int D,
                  void* x, int64_t* positions_out, int32_t* status_dev, const int32_t* len_dev,
                  int32_t* step_len_out, unsigned flags, void* stream);

/* y[M,N] = epilogue(x[M,K] . W[N,K]^T) with W tile-packed:
 *   t = round(acc); if bias: t = round(t + bias[n]); if RELU: t = max(t,0);
 *   if residual: t = round(t + residual[m,n]);  y[m,n] = t.
 * N % 16 == 0, K % 32 == 0.  With MSA_IN_PACKED (M <= 128) the HBM-bound weight-streaming kernel
 * runs; otherwise (any M, row-major x) a kernel chosen for the product's size: up to 64 rows
 * (int8 weights: 256) sweeps of the weight-streaming kernel over row-major activations, 64 rows
 * each; above that MFMA tiles, 256 rows by 256, 128 or 64 features with weights read straight
 * from the packed layout (K % 64 == 0; a ragged bottom block of at most 128 rows may be
 * streamed instead), and 128 x 128 LDS tiles for what is left.  All variants round at the same
 * points.  residual is row-major and may
 * alias a row-major y.  flags: MSA_EPI_RELU | MSA_IN_PACKED | MSA_OUT_PACKED.
 * Replaces LinearWithGradAccumulationAndAsyncCommunication.forward
 * (metaseq/modules/megatron/mpu/layers.py:290-292) as used by out_proj
 * (metaseq/modules/multihead_attention.py:553, bias and residual added in
 * metaseq/modules/transformer_decoder_layer.py:222-230), fc1/fc2
 * (metaseq/modules/feedforward.py:19-22; residual transformer_decoder_layer.py:283) and the
 * tied vocabulary projection (metaseq/models/transformer_decoder.py:413-420). */
int msa_linear_f16(const void* x, const void* Wp, const void* bias, const void* residual,
                   void* y, int64_t M, int N, int K, unsigned flags, void* stream);

/* Same contract with tile-packed int8 weights Wq and per-output-channel fp16 scales[N]:
 * the product uses the dequantised weight round(Wq[n,k] * scales[n]) (formed in registers).
 * K % 64 == 0.  No reference counterpart: the reference hands int8 serving to FasterTransformer
 * (metaseq/scripts/convert_metaseq_ft.py:99-133); semantics are the benchmark's definition. */
int msa_linear_w8a16(const void* x, const int8_t* Wq, const void* scales, const void* bias,
                     const void* residual, void* y, int64_t M, int N, int K, unsigned flags,
                     void* stream);

/* Split-K form for the decode step (packed activations, MSA_IN_PACKED: 1 <= M <= 128): K is cut into S
 * ranges and part[s][m][n] (fp32, [S, M, N]) receives the exact fp32 partial sums of range s;
 * the consumer adds them in slice order (msa_residual_layernorm_f16).  Used where N alone gives
 * the chip too few weight tiles (out_proj, fc2).  msa_linear_default_splits suggests S.  The
 * ranges hold ceil(K/32 / S) 32-wide steps (rounded up to an even count for int8); an S that would
 * leave the last range(s) empty is rejected.
 * Without MSA_IN_PACKED (msa_linear_partial_f16 only): x is row-major [M, K], any M >= 1, and the
 * MFMA tile kernel sums over S equal ranges (K % (64 S) == 0, K / S >= 128): for decode batches
 * above 128 rows, whose 256-row tiles against d_model output features occupy a quarter of the
 * chip; msa_linear_default_splits_rows suggests S (1: one pass of msa_linear_f16 is as good). */
int msa_linear_partial_f16(const void* x, const void* Wp, float* part, int64_t M, int N, int K,
                           int S, unsigned flags, void* stream);
int msa_linear_partial_w8a16(const void* x, const int8_t* Wq, const void* scales, float* part,
                             int64_t M, int N, int K, int S, unsigned flags, void* stream);
int msa_linear_default_splits(int64_t M, int N, int K);
int msa_linear_default_splits_w8a16(int64_t M, int N, int K);
int msa_linear_default_splits_rows(int64_t M, int N, int K);

/* Fused QKV projection: kvq = round(round(x . Wqkv^T) + bqkv) with rows of Wqkv ordered
 * K | V | Q; then for row m = b*T + t and head h:
 *   Kcache[b,h,S0+t,:] = k,  Vcache[b,h,S0+t,:] = v,  q_out[m, h*hd:(h+1)*hd] = round(q * hd^-0.5).
 * Caches are [B, H, S_cap, hd] fp16, q_out row-major.  Same size rules as msa_linear_f16 with
 * N = 3*H*hd.  flags: MSA_IN_PACKED.  With len_dev (T == 1) row b appends at len_dev[b].
 * Replaces metaseq/modules/multihead_attention.py:316-319 (projection + split), :429
 * (q scaling) and :449-479 (cache growth by torch.cat, here an in-place append). */
int msa_qkv_proj_f16(const void* x, const void* Wqkv, const void* bqkv, void* q_out,
                     void* Kcache, void* Vcache, int B, int T, int H, int hd, int S0, int S_cap,
                     int K, unsigned flags, const int32_t* len_dev, void* stream);
int msa_qkv_proj_w8a16(const void* x, const int8_t* Wq, const void* scales, const void* bqkv,
                       void* q_out, void* Kcache, void* Vcache, int B, int T, int H, int hd,
                       int S0, int S_cap, int K, unsigned flags, const int32_t* len_dev,
                       void* stream);

/* Causal attention of T new queries (already scaled, q[B*T, H*hd]) over the cache, whose
 * positions 0 .. S0+T-1 are valid: query t sees keys 0 .. S0+t.
 *   s = round(q . k);  s = -inf where key_pad_mask[b, key] != 0;
 *   p = round(softmax_fp32(s));  out[b*T+t, h*hd:(h+1)*hd] = round(sum_key p * v).
 * key_pad_mask (optional) is uint8 [B, mask_stride].  hd in {64, 128}.  T == 1 is the
 * bandwidth-bound decode kernel; T > 1 the prefill kernel.  q is row-major; flags:
 * MSA_OUT_PACKED (T == 1, B <= 128).  With len_dev (T == 1) row b attends its own
 * len_dev[b] + 1 positions and S0 only has to bound them.
 * Replaces metaseq/modules/multihead_attention.py:492 (bmm q k^T), :516-531 (causal and
 * padding masks), :533-534 (fp32 softmax, cast back), :543-552 (bmm p v, transpose). */
int msa_attention_f16(const void* q, const void* Kcache, const void* Vcache,
                      const uint8_t* key_pad_mask, int64_t mask_stride, void* out, int B, int H,
                      int hd, int T, int S0, int S_cap, unsigned flags, const int32_t* len_dev,
                      void* stream);

/* EXPERIMENTAL: pays only beyond OPT's 2048 positions (no benchmark configuration selects it;
 * msa_decoder_step takes it for a single request over more than 4096 keys at head_dim 128).
 * The decode step's attention (T == 1) in two launches, for few (batch row, head) pairs over long
 * histories (batch-1 serving, a nearly empty slot cache): one workgroup per pair leaves most
 * CUs idle and pulls the pair's K and V rows through a single CU.  Launch 1 writes the rounded
 * scores of 8 key ranges per pair to `workspace` (fp32 [B*H, S_cap],
 * msa_attention_split_workspace_bytes); launch 2, one workgroup per pair and 32-column slice of
 * the head, repeats the softmax over all scores and streams its slice of the V rows.  Every sum
 * is formed in the order msa_attention_f16 uses for B*H < 512, so the two give identical bits
 * and a caller may choose per step; msa_attention_prefers_split says when the split form pays
 * (measured: B*H <= 64 and n_keys*hd >= 512 K, i.e. histories beyond OPT's 2048 positions; below
 * that the second launch costs more than the idle CUs).  Arguments and reference as for
 * msa_attention_f16 with T == 1. */
int64_t msa_attention_split_workspace_bytes(int B, int H, int S_cap);
int msa_attention_prefers_split(int B, int H, int hd, int n_keys);
int msa_attention_split_f16(const void* q, const void* Kcache, const void* Vcache,
                            const uint8_t* key_pad_mask, int64_t mask_stride, void* out,
                            void* workspace, int B, int H, int hd, int S0, int S_cap,
                            unsigned flags, const int32_t* len_dev, void* stream);

/* One step of greedy selection over fp16 logits[B, V] (row stride ld_logits), with the
 * generator's bookkeeping fused in:
 *   z = logits / temperature (only if temperature > 0 and != 1);
 *   lprob(v) = (z[v] - max z) - log(sum(exp(z - max z))) in fp32 over ALL v; if any z is NaN every
 *   lprob of the row is -inf;
 *   ids in banned_host[0..n_banned) -> -inf (pad always, eos and stop ids while step < min_len);
 *   if force_eos_all != 0 (last step) or finished[b] != 0, only eos_idx stays eligible;
 *   row_mode (optional uint8[B], device) adds the same two regimes per row, for batches whose
 *   rows are at different points of their own requests: MSA_ROW_BAN_EARLY makes eos_idx and
 *   the stop ids ineligible for row b, MSA_ROW_ONLY_EOS leaves only eos_idx eligible;
 *   tok[b*tok_stride] = lowest index attaining the max lprob; score[b*score_stride] = that max;
 *   finished[b] |= tok == eos_idx or tok in stop_host[0..n_stop).
 * banned_host / stop_host are HOST arrays of at most 16 (stop: 15 in the fused forms) ids,
 * copied into the launch.  finished (uint8[B], device, in/out) is optional.
 * Replaces the per-step vocabulary passes of SequenceGenerator._generate
 * (metaseq/sequence_generator.py:272-308, :319-323), _sample_topp's greedy branch (:413-415)
 * and BaseDecoder.get_normalized_probs (metaseq/models/base_decoder.py:95-100). */
int msa_greedy_select_f16(const void* logits, int64_t ld_logits, int B, int V, float temperature,
                          const int32_t* banned_host, int n_banned, const int32_t* stop_host,
                          int n_stop, uint8_t* finished, const uint8_t* row_mode,
                          int force_eos_all, int eos_idx, int64_t* tok, int64_t tok_stride,
                          float* score, int64_t score_stride, const int32_t* len_dev,
                          void* stream);

/* One step of nucleus (top-p) sampling over fp16 logits[B, V], with the same bookkeeping as
 * msa_greedy_select_f16 (masks, row_mode, finished rows, token / score write-back) plus the
 * repetition penalties:
 *   z = logits / temperature (temperature_rows[b] if given, else `temperature`; no division for
 *   0 or 1);  lp = log_softmax_fp32(z) over all ids (a NaN anywhere: the row gets token 0 with
 *   score -inf, as does a row with no eligible id);
 *   banned / early / only-eos ids -> -inf;  lp[v] -= counts[b,v] * alpha_frequency +
 *   (counts[b,v] > 0) * alpha_presence, likewise counts_src (int64 [B, V] device, optional);
 *   penalty_rows (optional, fp32 [B, 4] device: presence, frequency, presence_src, frequency_src)
 *   gives every row its own four weights in place of the scalar arguments (rows of one batch
 *   that belong to different requests);
 *   lprobs_out (optional, fp32, row stride ld_lprobs) receives that masked, penalised row: what
 *   the reference stores as the step's distribution;
 *   p = softmax(lp);  with the ids in order of decreasing p (ties: increasing id), id k belongs
 *   to the nucleus iff the mass of the ids before it is < topp (topp_rows[b] if given, else
 *   topp_all);  the token is the arg-max over the nucleus of p[v] / noise[b, v], noise (fp32
 *   [B, V]) holding independent Exp(1) draws: an exponential race, which picks v with probability
 *   p[v] / mass(nucleus);  score = log p[tok].
 *   Without noise, or with topp <= 0 or temperature 0 for the row (the reference's greedy
 *   cases, :412), the choice is greedy: arg-max of lp (lowest id on ties), score = lp[tok].
 *   counts[b, tok] += 1 when counts is given.
 *   A row whose row_mode has MSA_ROW_SKIP is left alone (no output is written for it): a batch
 *   whose other rows were chosen by another entry point.
 * The nucleus is found without sorting (radix descent over the bit patterns of p with exact
 * fixed-point masses), so the result does not depend on the order of any summation.  The first
 * call on a device raises the kernel's dynamic LDS limit (it keeps 160 KB of per-id values between
 * its passes): make one call outside any stream capture.
 * Replaces SequenceGenerator._sample_topp and _apply_repetition_penalties
 * (metaseq/sequence_generator.py:399-441, :478-534), the masking in front of them (:272-293)
 * and the copy of the step's distribution (:301-303); the reference draws with
 * torch.multinomial over the sorted, renormalised nucleus, which is the same distribution. */
int msa_sample_topp_f16(const void* logits, int64_t ld_logits, int B, int V, float temperature,
                        const float* temperature_rows, const int32_t* banned_host, int n_banned,
                        const int32_t* stop_host, int n_stop, uint8_t* finished,
                        const uint8_t* row_mode, int force_eos_all, int eos_idx,
                        const float* topp_rows, float topp_all, const float* noise,
                        int64_t* counts, const int64_t* counts_src, float alpha_presence,
                        float alpha_frequency, float alpha_presence_src,
                        float alpha_frequency_src, const float* penalty_rows,
                        float* lprobs_out, int64_t ld_lprobs, int64_t* tok, int64_t tok_stride,
                        float* score, int64_t score_stride, void* stream);

/* fp32 log-softmax of n_outer x n_inner fp16 logits rows of V ids:
 *   out[o*out_outer_stride + i*ld_out + v] = z[v] - max z - log(sum(exp(z - max z))),
 *   z = logits[o*in_outer_stride + i*ld_logits + v] / temperature (no division for 0 or 1).
 * The two-level strides let one call copy the rows of every prompt into a [B, max_len, V] buffer.
 * Replaces BaseDecoder.get_normalized_probs over the prompt positions
 * (metaseq/models/base_decoder.py:95-100 as called at metaseq/sequence_generator.py:235-250). */
int msa_log_softmax_f16(const void* logits, int64_t in_outer_stride, int64_t ld_logits,
                        int n_outer, int n_inner, int V, float temperature, float* out,
                        int64_t out_outer_stride, int64_t ld_out, void* stream);

/* Log-probabilities of given target ids under fp16 logits rows:
 *   out[r] = logits[r, target[r]]/temperature - logsumexp_fp32(logits[r,:]/temperature).
 * Replaces the prompt scoring gather of SequenceGenerator._generate
 * (metaseq/sequence_generator.py:235-258). */
int msa_target_logprob_f16(const void* logits, int64_t ld_logits, int64_t rows, int V,
                           float temperature, const int64_t* target, float* out, void* stream);

/* Vocabulary projection fused with the greedy selection (M <= 64 rows, packed activations):
 * the logits round(x . E^T) of msa_linear_f16 are reduced inside the projection's epilogue to one
 * (running log-sum-exp, best eligible id) partial per row and workgroup, and a second small
 * kernel merges the partials and finishes the step exactly as msa_greedy_select_f16 does (same
 * masks, tie-break, outputs and `len_dev` meaning).  The logits are only stored if `logits`
 * ([M, V] fp16, row-major) is not NULL.  `workspace` needs
 * msa_lm_head_select_workspace_bytes(M) bytes of device memory (contents are scratch).
 * Replaces metaseq/models/transformer_decoder.py:398-428 (output_layer) followed by
 * metaseq/sequence_generator.py:272-308,319-323 (log-softmax, masks, max, bookkeeping). */
int64_t msa_lm_head_select_workspace_bytes(int M);
int msa_lm_head_greedy_select_f16(const void* x, const void* Ep, void* logits, void* workspace,
                                  int M, int V, int K, float temperature,
                                  const int32_t* banned_host, int n_banned,
                                  const int32_t* stop_host, int n_stop, uint8_t* finished,
                                  const uint8_t* row_mode, int force_eos_all, int eos_idx,
                                  int64_t* tok, int64_t tok_stride, float* score,
                                  int64_t score_stride, const int32_t* len_dev, void* stream);

/* msa_lm_head_greedy_select_f16 for callers that cannot allocate device memory (code under
 * hipGraph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, results and kernels, minus `workspace`: the
 * selection partials go to a fixed device array inside the library (512 KiB per GPU, held until
 * the process ends), whose address is looked up once per device on the first call there.  The
 * call allocates and frees nothing.  Limits: M <= 64 rows and at most 256 compute units
 * (MSA_ERR_CAPACITY beyond).  All calls on one GPU share that array: calls that overlap on one
 * GPU (different streams or threads) race; calls on one stream are ordered and safe.  Nothing
 * in the array needs to start at zero: every partial that is read is written by the same call.
 * The FIRST call on a device looks the array's address up (hipGetDevice, hipGetSymbolAddress,
 * which may load the code object): make one call per device outside any stream capture before
 * capturing calls into a graph; every later call issues kernel launches only. */
int msa_lm_head_greedy_select_noalloc_f16(const void* x, const void* Ep, void* logits, int M,
                                          int V, int K, float temperature,
                                          const int32_t* banned_host, int n_banned,
                                          const int32_t* stop_host, int n_stop, uint8_t* finished,
                                          const uint8_t* row_mode, int force_eos_all, int eos_idx,
                                          int64_t* tok, int64_t tok_stride, float* score,
                                          int64_t score_stride, const int32_t* len_dev,
                                          void* stream);

/* ---- one decode step of the whole decoder in one call ------------------------------------------
 * msa_decoder_create copies a table of device pointers (it allocates host memory only and
 * touches no GPU); msa_decoder_step then launches, on `stream`, exactly the sequence a caller
 * would issue entry point by entry point for T == 1 and at most 128 rows: msa_embed_f16,
 * msa_layernorm_f16, per layer msa_qkv_proj_* / msa_attention_f16 / msa_linear_partial_* /
 * msa_residual_layernorm_f16 / msa_linear_* (ReLU) / msa_linear_partial_* /
 * msa_residual_layernorm_f16, then msa_lm_head_greedy_select_f16 (if `tok` is given; `logits`
 * optional; beyond 64 rows msa_linear_f16 into `logits` or the workspace followed by
 * msa_greedy_select_f16) or msa_linear_f16 into `logits` - same arguments, same order, so
 * bit-identical results.  Every linear weight is in the packed layout, int8 with scales if cfg.int8 (the
 * embedding tables stay row-major fp16, lm_head_packed is the packed copy of embed_tokens).
 * With len_dev (per-row lengths, see above) the rows that took part are advanced by one at the
 * end of the step unless MSA_STEP_NO_ADVANCE; MSA_EMBED_COL_FROM_LEN as for msa_embed_f16.
 * k_cache / v_cache are HOST arrays of cfg.layers device pointers ([B, H, S_cap, hd] each).
 * workspace: msa_decoder_step_workspace_bytes(dec, B) bytes of device memory (scratch).
 * Replaces one pass of ModelParallelTransformerDecoder.forward with a non-empty
 * incremental_state (metaseq/models/transformer_decoder.py:494-537) plus, with `tok`, the
 * per-step vocabulary passes of SequenceGenerator._generate
 * (metaseq/sequence_generator.py:272-308, :319-323). */
#define MSA_STEP_NO_ADVANCE 16u

typedef struct {
  int layers, d_model, heads, ffn, vocab;
  int n_pos_rows; /* rows of the positional table */
  int pad_idx;
  int int8;       /* the four per-layer matrices are packed int8 with fp16 scales */
} msa_decoder_config;

typedef struct {
  const void *ln1_gamma, *ln1_beta;                 /* self_attn_layer_norm */
  const void *qkv_weight, *qkv_scales, *qkv_bias;   /* rows K | V | Q */
  const void *out_weight, *out_scales, *out_bias;
  const void *ln2_gamma, *ln2_beta;                 /* final_layer_norm */
  const void *fc1_weight, *fc1_scales, *fc1_bias;
  const void *fc2_weight, *fc2_scales, *fc2_bias;
} msa_layer_weights;

typedef struct {
  const int64_t* tokens;  /* [B, n] ids; the new token of row b is column n - 1 */
  int64_t tok_stride;
  int n, B;
  void* const* k_cache;
  void* const* v_cache;
  int S0, S_cap;                /* with len_dev: S0 = the caller's bound on the lengths, 0 if
                                   it has none (it only steers the choice of attention form) */
  int32_t* len_dev;             /* optional int32 [B] */
  const uint8_t* key_pad_mask;  /* optional uint8 [B, mask_stride] */
  int64_t mask_stride;
  unsigned flags;
  void* workspace;
  int64_t workspace_bytes;
  void* logits;                 /* optional fp16 [B, vocab] */
  int64_t* tok;                 /* optional: greedy selection, as msa_lm_head_greedy_select_f16 */
  int64_t tok_stride_out;
  float* score;
  int64_t score_stride;
  float temperature;
  const int32_t* banned;
  int n_banned;
  const int32_t* stop;
  int n_stop;
  uint8_t* finished;
  const uint8_t* row_mode;
  int force_eos_all, eos_idx;
  const int32_t* col_dev;
} msa_step_args;

typedef struct msa_decoder msa_decoder;

int msa_decoder_create(const msa_decoder_config* cfg, const void* embed_tokens,
                       const void* embed_positions, const void* lm_head_packed,
                       const void* final_ln_gamma, const void* final_ln_beta,
                       const msa_layer_weights* layers, msa_decoder** out);
void msa_decoder_destroy(msa_decoder* dec);
int64_t msa_decoder_step_workspace_bytes(msa_decoder* dec, int B);
int msa_decoder_step(msa_decoder* dec, const msa_step_args* args, void* stream);

/* Measurement aid with no counterpart in the reference: reads `bytes` bytes (a multiple of 16,
 * 16-byte aligned) of device memory once with 16-byte streaming loads and discards them.  The
 * benchmark times it to report the read rate this GPU actually sustains beside the published
 * peak that the roofline fractions are quoted against. */
int msa_probe_stream_read(const void* p, int64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* METASEQ_AMD_H */
