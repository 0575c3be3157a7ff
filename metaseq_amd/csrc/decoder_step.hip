// One decode step of the whole decoder in a single C call: embedding, L layers, final LayerNorm
// and the vocabulary projection (stored logits and / or the fused greedy selection), launched
// back to back on the caller's stream from a table of device pointers.  It runs the same entry
// points, in the same order and with the same arguments, as a caller that drives them one by one
// (so the results are bit-identical); what it removes is the per-launch cost of crossing the
// language boundary a few hundred times per token.
#include <stdlib.h>
#include <string.h>

#include <new>

#include "common.h"

struct msa_decoder {
  msa_decoder_config cfg;
  const void* embed_tokens;
  const void* embed_positions;
  const void* lm_head;
  const void* final_ln_gamma;
  const void* final_ln_beta;
  msa_layer_weights* layers;
};

namespace {

int64_t align256(int64_t n) { return (n + 255) & ~(int64_t)255; }

// workspace layout for B rows
struct StepBuffers {
  char *x, *q, *h, *o, *u, *part, *positions, *step_len, *select_ws, *attn_ws, *logits;
  int64_t attn_keys;  // key positions per (b, h) that attn_ws holds scores for (0: none)
  int64_t bytes;
};

// most keys the split attention's score buffer is sized for
int64_t split_attention_keys(const msa_decoder* d, int B) {
  const int hd = d->cfg.d_model / d->cfg.heads;
  const int64_t keys = d->cfg.n_pos_rows < 8192 ? d->cfg.n_pos_rows : 8192;
  // the form can only ever be chosen for few (b, h) pairs; ask with the longest history
  return msa_attention_prefers_split(B, d->cfg.heads, hd, (int)keys) ? keys : 0;
}

// split-K counts of out_proj and fc2 for B rows.  Computed per call (a few integer operations) and
// kept out of the handle: the handle holds nothing that a call writes.
struct Splits {
  int out, fc2;
};

Splits pick_splits(const msa_decoder* d, int B) {
  const int D = d->cfg.d_model, F = d->cfg.ffn;
  Splits s;
  s.out = d->cfg.int8 ? msa_linear_default_splits_w8a16(B, D, D)
                      : msa_linear_default_splits(B, D, D);
  s.fc2 = d->cfg.int8 ? msa_linear_default_splits_w8a16(B, D, F)
                      : msa_linear_default_splits(B, D, F);
  return s;
}

StepBuffers carve(const msa_decoder* d, int B, const Splits& sp, char* base) {
  const int64_t D = d->cfg.d_model, F = d->cfg.ffn, MP = packed_row_blocks(B) * 16;
  const int64_t S = sp.out > sp.fc2 ? sp.out : sp.fc2;
  StepBuffers w{};
  int64_t off = 0;
  auto take = [&](int64_t n) {
    char* p = base ? base + off : nullptr;
    off += align256(n);
    return p;
  };
  w.x = take(B * D * 2);
  w.q = take(B * D * 2);
  w.h = take(MP * D * 2);
  w.o = take(MP * D * 2);
  w.u = take(MP * F * 2);
  w.part = take(S * B * D * 4);
  w.positions = take(B * 8);
  w.step_len = take(B * 4);
  // up to 64 rows the selection runs inside the vocabulary projection (partials per workgroup);
  // beyond, the projection stores its logits and a second kernel selects from them
  w.select_ws = take(B <= 64 ? msa_lm_head_select_workspace_bytes(B) : 0);
  w.logits = take(B <= 64 ? 0 : (int64_t)B * d->cfg.vocab * 2);
  w.attn_keys = split_attention_keys(d, B);
  w.attn_ws = take(msa_attention_split_workspace_bytes(B, d->cfg.heads, (int)w.attn_keys));
  w.bytes = off;
  return w;
}

}  // namespace

extern "C" int msa_decoder_create(const msa_decoder_config* cfg, const void* embed_tokens,
                                  const void* embed_positions, const void* lm_head_packed,
                                  const void* final_ln_gamma, const void* final_ln_beta,
                                  const msa_layer_weights* layers, msa_decoder** out) {
  const char* name = "msa_decoder_create";
  MSA_REQUIRE(cfg && embed_tokens && embed_positions && lm_head_packed && final_ln_gamma &&
                  final_ln_beta && layers && out,
              MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(cfg->layers > 0 && cfg->d_model > 0 && cfg->heads > 0 && cfg->ffn > 0 &&
                  cfg->vocab > 0 && cfg->d_model % cfg->heads == 0 &&
                  cfg->n_pos_rows > cfg->pad_idx && cfg->pad_idx >= 0,
              MSA_ERR_INVALID_ARG, "%s: bad configuration", name);
  const int hd = cfg->d_model / cfg->heads;
  MSA_REQUIRE(hd == 64 || hd == 128, MSA_ERR_INVALID_ARG,
              "%s: head_dim %d not supported (64 or 128)", name, hd);
  for (int i = 0; i < cfg->layers; ++i) {
    const msa_layer_weights& l = layers[i];
    MSA_REQUIRE(l.ln1_gamma && l.ln1_beta && l.qkv_weight && l.qkv_bias && l.out_weight &&
                    l.out_bias && l.ln2_gamma && l.ln2_beta && l.fc1_weight && l.fc1_bias &&
                    l.fc2_weight && l.fc2_bias,
                MSA_ERR_INVALID_ARG, "%s: layer %d has a null pointer", name, i);
    MSA_REQUIRE(!cfg->int8 || (l.qkv_scales && l.out_scales && l.fc1_scales && l.fc2_scales),
                MSA_ERR_INVALID_ARG, "%s: layer %d lacks int8 scales", name, i);
  }
  msa_decoder* d = new (std::nothrow) msa_decoder();
  msa_layer_weights* lw =
      (msa_layer_weights*)malloc(sizeof(msa_layer_weights) * (size_t)cfg->layers);
  if (!d || !lw) {
    delete d;
    free(lw);
    msa_set_error("%s: out of host memory", name);
    return MSA_ERR_INVALID_ARG;
  }
  memcpy(lw, layers, sizeof(msa_layer_weights) * (size_t)cfg->layers);
  d->cfg = *cfg;
  d->embed_tokens = embed_tokens;
  d->embed_positions = embed_positions;
  d->lm_head = lm_head_packed;
  d->final_ln_gamma = final_ln_gamma;
  d->final_ln_beta = final_ln_beta;
  d->layers = lw;
  *out = d;
  return MSA_OK;
}

extern "C" void msa_decoder_destroy(msa_decoder* d) {
  if (!d) return;
  free(d->layers);
  delete d;
}

extern "C" int64_t msa_decoder_step_workspace_bytes(msa_decoder* d, int B) {
  if (!d || B < 1 || B > MSA_PACKED_MAX_ROWS) return 0;
  return carve(d, B, pick_splits(d, B), nullptr).bytes;
}

extern "C" int msa_decoder_step(msa_decoder* d, const msa_step_args* a, void* stream) {
  const char* name = "msa_decoder_step";
  MSA_REQUIRE(d && a, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(a->tokens && a->k_cache && a->v_cache && a->workspace, MSA_ERR_INVALID_ARG,
              "%s: null pointer in the step's arguments", name);
  const int B = a->B;
  MSA_REQUIRE(B >= 1 && B <= MSA_PACKED_MAX_ROWS, MSA_ERR_INVALID_ARG, "%s: B=%d outside 1..%d",
              name, B, MSA_PACKED_MAX_ROWS);
  MSA_REQUIRE(a->logits || a->tok, MSA_ERR_INVALID_ARG,
              "%s: neither logits nor a token output was asked for", name);
  MSA_REQUIRE(!a->tok || a->score, MSA_ERR_INVALID_ARG, "%s: tok needs score", name);
  MSA_REQUIRE((a->flags & ~(MSA_EMBED_COL_FROM_LEN | MSA_STEP_NO_ADVANCE)) == 0,
              MSA_ERR_INVALID_ARG, "%s: unsupported flags 0x%x", name, a->flags);
  const Splits sp = pick_splits(d, B);
  const StepBuffers w = carve(d, B, sp, (char*)a->workspace);
  MSA_REQUIRE(a->workspace_bytes >= w.bytes, MSA_ERR_CAPACITY,
              "%s: workspace of %lld bytes, %lld needed", name, (long long)a->workspace_bytes,
              (long long)w.bytes);
  const msa_decoder_config& c = d->cfg;
  const int D = c.d_model, H = c.heads, hd = D / H, F = c.ffn, V = c.vocab;
  const unsigned IN = MSA_IN_PACKED, OUT = MSA_OUT_PACKED;
  const float eps = 1e-5f;
  // a row whose new token is a pad, or whose slot is empty, sits the step out
  const bool gate = a->len_dev != nullptr && !(a->flags & MSA_EMBED_COL_FROM_LEN);
  int32_t* step_len = gate ? (int32_t*)w.step_len : nullptr;
  int rc = msa_embed_f16(a->tokens, a->tok_stride, B, a->n, 1, d->embed_tokens, V,
                         d->embed_positions, c.n_pos_rows, c.pad_idx, D, w.x,
                         (int64_t*)w.positions, nullptr, a->len_dev, step_len,
                         a->flags & MSA_EMBED_COL_FROM_LEN, stream);
  if (rc) return rc;
  const int32_t* len = gate ? step_len : a->len_dev;
  rc = msa_layernorm_f16(w.x, d->layers[0].ln1_gamma, d->layers[0].ln1_beta, w.h, B, D, eps, OUT,
                         stream);
  if (rc) return rc;
  // few (b, h) pairs over a long history: the two-launch attention (same bits).  With lengths
  // on the device S0 is the caller's bound on them if it has one (0: only the capacity is known).
  const int keys_bound = a->len_dev && a->S0 == 0 ? a->S_cap : a->S0 + 1;
  const bool split_attention =
      a->S_cap <= w.attn_keys && msa_attention_prefers_split(B, H, hd, keys_bound);
  for (int i = 0; i < c.layers; ++i) {
    const msa_layer_weights& l = d->layers[i];
    void* kc = a->k_cache[i];
    void* vc = a->v_cache[i];
    if (c.int8)
      rc = msa_qkv_proj_w8a16(w.h, (const int8_t*)l.qkv_weight, l.qkv_scales, l.qkv_bias, w.q, kc,
                              vc, B, 1, H, hd, a->S0, a->S_cap, D, IN, len, stream);
    else
      rc = msa_qkv_proj_f16(w.h, l.qkv_weight, l.qkv_bias, w.q, kc, vc, B, 1, H, hd, a->S0,
                            a->S_cap, D, IN, len, stream);
    if (rc) return rc;
    if (split_attention)
      rc = msa_attention_split_f16(w.q, kc, vc, a->key_pad_mask, a->mask_stride, w.o, w.attn_ws, B,
                                   H, hd, a->S0, a->S_cap, OUT, len, stream);
    else
      rc = msa_attention_f16(w.q, kc, vc, a->key_pad_mask, a->mask_stride, w.o, B, H, hd, 1, a->S0,
                             a->S_cap, OUT, len, stream);
    if (rc) return rc;
    if (c.int8)
      rc = msa_linear_partial_w8a16(w.o, (const int8_t*)l.out_weight, l.out_scales,
                                    (float*)w.part, B, D, D, sp.out, IN, stream);
    else
      rc = msa_linear_partial_f16(w.o, l.out_weight, (float*)w.part, B, D, D, sp.out, IN,
                                  stream);
    if (rc) return rc;
    rc = msa_residual_layernorm_f16((const float*)w.part, sp.out, l.out_bias, w.x,
                                    l.ln2_gamma, l.ln2_beta, w.h, B, D, eps, OUT, stream);
    if (rc) return rc;
    if (c.int8)
      rc = msa_linear_w8a16(w.h, (const int8_t*)l.fc1_weight, l.fc1_scales, l.fc1_bias, nullptr,
                            w.u, B, F, D, MSA_EPI_RELU | IN | OUT, stream);
    else
      rc = msa_linear_f16(w.h, l.fc1_weight, l.fc1_bias, nullptr, w.u, B, F, D,
                          MSA_EPI_RELU | IN | OUT, stream);
    if (rc) return rc;
    if (c.int8)
      rc = msa_linear_partial_w8a16(w.u, (const int8_t*)l.fc2_weight, l.fc2_scales,
                                    (float*)w.part, B, D, F, sp.fc2, IN, stream);
    else
      rc = msa_linear_partial_f16(w.u, l.fc2_weight, (float*)w.part, B, D, F, sp.fc2, IN,
                                  stream);
    if (rc) return rc;
    const bool last = i + 1 == c.layers;
    rc = msa_residual_layernorm_f16((const float*)w.part, sp.fc2, l.fc2_bias, w.x,
                                    last ? d->final_ln_gamma : d->layers[i + 1].ln1_gamma,
                                    last ? d->final_ln_beta : d->layers[i + 1].ln1_beta, w.h, B, D,
                                    eps, OUT, stream);
    if (rc) return rc;
  }
  if (gate && !(a->flags & MSA_STEP_NO_ADVANCE)) {
    rc = msa_advance_len(a->len_dev, step_len, B, 1, stream);
    if (rc) return rc;
  }
  if (a->tok && B > 64) {
    void* logits = a->logits ? a->logits : (void*)w.logits;
    rc = msa_linear_f16(w.h, d->lm_head, nullptr, nullptr, logits, B, V, D, IN, stream);
    if (rc) return rc;
    return msa_greedy_select_f16(logits, V, B, V, a->temperature, a->banned, a->n_banned, a->stop,
                                 a->n_stop, a->finished, a->row_mode, a->force_eos_all,
                                 a->eos_idx, a->tok, a->tok_stride_out, a->score,
                                 a->score_stride, a->col_dev, stream);
  }
  if (a->tok)
    return msa_lm_head_greedy_select_f16(w.h, d->lm_head, a->logits, w.select_ws, B, V, D,
                                         a->temperature, a->banned, a->n_banned, a->stop,
                                         a->n_stop, a->finished, a->row_mode, a->force_eos_all,
                                         a->eos_idx, a->tok, a->tok_stride_out, a->score,
                                         a->score_stride, a->col_dev, stream);
  return msa_linear_f16(w.h, d->lm_head, nullptr, nullptr, a->logits, B, V, D, IN, stream);
}
