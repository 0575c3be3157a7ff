"""CPU restatement of metaseq's OPT incremental-decoding forward and greedy loop.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file; it is
the checker that the parity tests, the smoke test and the benchmark's CPU-baseline
leg compare the HIP path against.  It is written from the reference's sources (cited
per function, paths relative to the metaseq tree) in plain PyTorch ops and runs on
any torch device.

Two arithmetic modes, selected by ``dtype`` (and, orthogonally, ``lean=True`` keeps weights
and the key/value history stored in ``dtype`` and upcasts them where they are used, and walks
the attention over batch rows in chunks: the same values at a fraction of the memory, for the
30B / 66B shapes):

* ``torch.float32`` - everything in fp32.
* ``torch.float16`` - "rounding faithful": every tensor the reference materialises
  in fp16 is rounded to fp16 here at the same point (after each matmul, after each
  separate bias add, after ``q *= scaling``, after the softmax cast-back, after each
  residual add, after each LayerNorm), while the arithmetic between two rounding
  points runs in fp32, which is what the BLAS / softmax / LayerNorm kernels behind
  the reference's torch calls do (fp32 accumulation, one rounding on output).

How each function is pinned (tests/test_oracle_*.py):

* ``make_positions``           - the reference's own known-answer table
                                 (cpu_tests/test_utils.py:55-93), committed as
                                 tests/golden/make_positions.json.
* ``layer_norm``               - closed form in float64 numpy; constant-row and
                                 affine special cases.
* ``attention`` (prefill and   - brute-force python loops on tiny inputs and
  incremental)                   ``F.scaled_dot_product_attention(is_causal=True)``;
                                 invariant: incremental logits at step t equal the
                                 last row of a full forward on tokens[:t+1].
* whole decoder, K|V|Q order,  - Hugging Face ``OPTForCausalLM`` built from a config
  position offset, pad mask      object with the same weights mapped in (the
                                 relation the reference's own
                                 gpu_tests/test_hf_compatibility.py:128-155 asserts).
* ``generate`` /               - scripted-logit fake decoders with hand-derived
  ``greedy_generate``            expected token/score tables (the idea of the
                                 reference's tests/utils.py:420-465).
* ``sample_topp``,             - hand-derived closed forms (mass-before-token rule,
  ``update_sampling_topp``,      renormalisation, score of the untruncated probability,
  ``apply_repetition_penalties`` decay / reset / bound sequence, penalty arithmetic) and
                                 empirical draw frequencies; the reference holds no test of
                                 these functions (tests/test_sequence_generator.py predates
                                 them).
* ``quantize_int8``            - parity unpinned by the reference (its int8
                                 quantiser lives in FasterTransformer and no
                                 reference test touches it); pinned by the closed
                                 form stated in the function and brute force.
"""

import math
import uuid
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F


@dataclass
class OracleConfig:
    """Attribute names follow the reference's args namespace
    (metaseq/models/transformer_decoder.py:73-117)."""

    decoder_layers: int
    decoder_embed_dim: int
    decoder_attention_heads: int
    decoder_ffn_embed_dim: int
    vocab_size: int
    max_target_positions: int = 2048
    padding_idx: int = 1
    eos_idx: int = 2

    @property
    def head_dim(self) -> int:
        return self.decoder_embed_dim // self.decoder_attention_heads


def make_positions(tokens: torch.Tensor, padding_idx: int) -> torch.Tensor:
    """metaseq/utils.py:83-93: non-pad symbols get cumsum(non-pad) + padding_idx,
    pads get padding_idx."""
    mask = tokens.ne(padding_idx).int()
    return (torch.cumsum(mask, dim=1).type_as(mask) * mask).long() + padding_idx


def layer_norm(x, gamma, beta, eps=1e-5):
    """metaseq/modules/layer_norm.py:28-33 (torch.nn.LayerNorm / apex
    cuApplyLayerNorm, apex/layer_norm_cuda_kernel.cu:441-455): statistics in fp32,
    biased variance, y = gamma * (x - mean) * rsqrt(var + eps) + beta."""
    x = x.float()
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) * torch.rsqrt(var + eps) * gamma.float() + beta.float()


def quantize_int8(w: torch.Tensor):
    """Symmetric per-output-channel weight-only int8 (the benchmark's definition; the
    reference delegates this to FasterTransformer, scripts/convert_metaseq_ft.py:99-133).

    w [out, in] -> (q int8 [out, in], scale fp16 [out]) with
    scale_j = fp16(max_i |w_ji| / 127), q = clamp(rint(w / scale_j), -127, 127),
    dequantised weight = fp16(q * scale_j).
    """
    wf = w.float()
    scale = (wf.abs().amax(dim=1) / 127.0).to(torch.float16)
    s = scale.float().clamp_min(1e-30).unsqueeze(1)
    q = torch.clamp(torch.round(wf / s), -127, 127).to(torch.int8)
    return q, scale


def dequantize_int8(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    return (q.float() * scale.float().unsqueeze(1)).to(torch.float16)


def linear(x, w, b, r):
    """mpu/layers.py:290-292: output = matmul(x, W.t()), then output = output + bias as a
    separate op; ``r`` is the rounding applied where the reference materialises a tensor."""
    y = r(x @ w.t())
    if b is not None:
        y = r(y + b)
    return y


class _Weights:
    """name -> fp32 tensor; the stored tensor may be narrower (lean mode) and is then upcast on
    access, which changes no value."""

    def __init__(self, tensors):
        self.t = tensors

    def __getitem__(self, k):
        return self.t[k].float()

    def raw(self, k):
        return self.t[k]

    def __contains__(self, k):
        return k in self.t


class OracleDecoder:
    """Restates ModelParallelTransformerDecoder.forward at tensor-parallel size 1
    (metaseq/models/transformer_decoder.py:494-537) with the inference branch of
    ModelParallelMultiheadAttention (metaseq/modules/multihead_attention.py:428-556).

    ``state_dict`` uses the reference's parameter names
    (metaseq/scripts/convert_metaseq_ft.py:74-90): decoder.embed_tokens.weight,
    decoder.embed_positions.weight, decoder.layers.{i}.self_attn_layer_norm.*,
    decoder.layers.{i}.self_attn.qkv_proj.* (rows K | V | Q),
    decoder.layers.{i}.self_attn.out_proj.*, decoder.layers.{i}.final_layer_norm.*,
    decoder.layers.{i}.fc1.*, decoder.layers.{i}.fc2.*, decoder.layer_norm.*.
    """

    def __init__(self, cfg: OracleConfig, state_dict: Dict[str, torch.Tensor],
                 dtype=torch.float32, device="cpu", lean=False, native_matmul=False,
                 store_dtype=None):
        self.cfg = cfg
        self.dtype = dtype
        self.device = torch.device(device)
        self.lean = lean
        # trace: None, or {layer index: []}; every pass through such a layer appends a dict of
        # the tensors the reference materialises there (batch-major, in `dtype`), for tests that
        # feed one op of another implementation the oracle's own input of that op
        self.trace: Optional[Dict[int, list]] = None
        # what to record: None = everything, a set of names, or {layer index: set or None}
        self.trace_keys = None
        self.trace_device = None  # where recorded tensors are kept (None = where they are)
        # native_matmul: matrix products are handed to torch in `dtype` itself (what the
        # reference does on a GPU: the BLAS accumulates in fp32 and rounds once on output)
        # instead of as fp32 products of `dtype` values that are rounded afterwards.  Same
        # rounding points, another summation order: a second valid evaluation of the reference,
        # used to measure how far two such evaluations drift apart.
        self.native_matmul = native_matmul and dtype != torch.float32
        # weights are values already rounded to `dtype`, held as fp32 copies - or, when lean, in
        # `dtype` itself (no copy if the caller's tensor already is) and upcast at each use
        # store_dtype (lean only): the dtype the weights are kept in when it is narrower than the
        # arithmetic `dtype` (fp16 weights evaluated in fp32 throughout: exact upcasts at each use)
        store = store_dtype if (lean and store_dtype is not None) else dtype
        self.w = _Weights({
            k: (v.detach().to(self.device).to(store) if lean
                else v.detach().to(self.device).to(dtype).float())
            for k, v in state_dict.items()
            if v.is_floating_point()
        })
        self.layer_ids = [str(uuid.uuid4()) for _ in range(cfg.decoder_layers)]
        # lean: rows of the batch whose attention is evaluated together (bounds the fp32
        # score tensors to about 2 GB)
        self.attn_chunk_bytes = 2 << 30

    # -- rounding point --------------------------------------------------
    def _r(self, t: torch.Tensor) -> torch.Tensor:
        if self.dtype == torch.float32:
            return t
        return t.to(self.dtype).float()

    def max_positions(self) -> int:
        # transformer_decoder.py:430-434 with learned_positional_embedding.py:25-28
        return min(
            self.cfg.max_target_positions,
            self.w.raw("decoder.embed_positions.weight").shape[0] - self.cfg.padding_idx - 1,
        )

    # -- linear: matmul -> round -> (+ bias -> round) ----------------------
    def _linear(self, x, wname, bname=None):
        b = self.w[bname] if bname is not None else None
        if self.native_matmul:
            y = (x.to(self.dtype) @ self.w.raw(wname).to(self.dtype).t()).float()
            return self._r(y + b) if b is not None else y
        return linear(x, self.w[wname], b, self._r)

    def _bmm(self, a, b):
        if self.native_matmul:
            return torch.bmm(a.to(self.dtype), b.to(self.dtype)).float()
        return self._r(torch.bmm(a, b))

    def attention_core(self, q, k, v, B, attn_mask=None, key_padding_mask=None):
        """multihead_attention.py:492-543 on q [B*H, T, hd] (already scaled) and
        k, v [B*H, S, hd]: scores, additive causal mask, key padding mask, fp32 softmax cast
        back to the activation dtype, weighted sum of values."""
        BH, T, _ = q.shape
        H, S = BH // B, k.shape[1]
        s = self._bmm(q, k.transpose(1, 2))  # :492
        if attn_mask is not None:
            s = s + attn_mask.unsqueeze(0)  # :516-518
        if key_padding_mask is not None:  # :520-531
            assert key_padding_mask.shape == (B, S)
            s = s.view(B, H, T, S).masked_fill(
                key_padding_mask.unsqueeze(1).unsqueeze(2).to(torch.bool), float("-inf")
            ).view(BH, T, S)
        pr = self._r(F.softmax(s, dim=-1, dtype=torch.float32))  # :533-534
        return self._bmm(pr, v)  # :543

    def _attention_rows(self, q, k, v, B, attn_mask, key_padding_mask):
        """attention_core over the whole batch, or (lean) over groups of batch rows: rows are
        independent, so the values are the same."""
        BH, T, _ = q.shape
        H, S = BH // B, k.shape[1]
        rows = B
        if self.lean:
            rows = max(1, min(B, int(self.attn_chunk_bytes // max(1, H * T * S * 4))))
        if rows >= B:
            return self.attention_core(q, k, v, B, attn_mask, key_padding_mask)
        out = []
        for b0 in range(0, B, rows):
            b1 = min(B, b0 + rows)
            kp = None if key_padding_mask is None else key_padding_mask[b0:b1]
            out.append(self.attention_core(q[b0 * H:b1 * H], k[b0 * H:b1 * H],
                                           v[b0 * H:b1 * H], b1 - b0, attn_mask, kp))
        return torch.cat(out, dim=0)

    def _attention(self, i, x, incremental_state, attn_mask, key_padding_mask):
        """multihead_attention.py:278-556, inference branch. x is [T, B, D]."""
        cfg = self.cfg
        T, B, D = x.shape
        H, hd = cfg.decoder_attention_heads, cfg.head_dim
        p = f"decoder.layers.{i}.self_attn."
        kvq = self._linear(x, p + "qkv_proj.weight", p + "qkv_proj.bias")
        k, v, q = kvq.split(D, dim=-1)  # :316-319, thirds are K | V | Q
        q = self._r(q * (hd ** -0.5))  # :429
        tr = self._tr(i)
        self._rec(tr, k=k, v=v, q=q)
        q = q.contiguous().view(T, B * H, hd).transpose(0, 1)  # :431-435
        k = k.contiguous().view(-1, B * H, hd).transpose(0, 1)
        v = v.contiguous().view(-1, B * H, hd).transpose(0, 1)
        if incremental_state is not None:
            key = self.layer_ids[i] + ".attn_state"
            saved = incremental_state.get(key, {})
            if "prev_key" in saved:  # :451-467
                k = torch.cat([saved["prev_key"].view(B * H, -1, hd).float(), k], dim=1)
                v = torch.cat([saved["prev_value"].view(B * H, -1, hd).float(), v], dim=1)
            # the history holds values already rounded to `dtype`: storing it in `dtype` (lean)
            # loses nothing
            keep = (lambda t: t.to(self.dtype)) if self.lean else (lambda t: t)
            saved["prev_key"] = keep(k.view(B, H, -1, hd))
            saved["prev_value"] = keep(v.view(B, H, -1, hd))
            saved["prev_key_padding_mask"] = key_padding_mask
            incremental_state[key] = saved
        o = self._attention_rows(q, k, v, B, attn_mask, key_padding_mask)
        o = o.transpose(0, 1).contiguous().view(T, B, D)  # :552
        self._rec(tr, o=o)
        return self._linear(o, p + "out_proj.weight", None), self.w[p + "out_proj.bias"]

    def _tr(self, i):
        """The dict the current pass through layer ``i`` records into, or None."""
        if self.trace is None or not self.trace.get(i):
            return None
        return self.trace[i][-1]

    def _rec(self, tr, **tensors):
        """Records [T, B, D] tensors as batch-major [B * T, D] copies in the activation dtype
        (the values are already rounded to it, so nothing is lost)."""
        if tr is None:
            return
        keys = self.trace_keys
        if isinstance(keys, dict):
            keys = keys.get(tr["layer"])
        for name, t in tensors.items():
            if keys is None or name in keys:
                t = t.transpose(0, 1).reshape(-1, t.shape[-1]).to(self.dtype)
                tr[name] = t if self.trace_device is None else t.to(self.trace_device)

    def _layer(self, i, x, incremental_state, attn_mask, key_padding_mask):
        """transformer_decoder_layer.py:233-284 (pre-LN, ReLU FFN)."""
        p = f"decoder.layers.{i}."
        tr = None
        if self.trace is not None and i in self.trace:
            tr = {"layer": i}
            self.trace[i].append(tr)
        residual = x
        h = self._r(layer_norm(x, self.w[p + "self_attn_layer_norm.weight"],
                               self.w[p + "self_attn_layer_norm.bias"]))
        self._rec(tr, x_in=x, h1=h)
        a, a_bias = self._attention(i, h, incremental_state, attn_mask, key_padding_mask)
        a = self._r(a + a_bias)  # :222-223
        x = self._r(a + residual)  # :230
        residual = x
        h = self._r(layer_norm(x, self.w[p + "final_layer_norm.weight"],
                               self.w[p + "final_layer_norm.bias"]))
        u = F.relu(self._linear(h, p + "fc1.weight", p + "fc1.bias"))  # feedforward.py:21
        self._rec(tr, x_mid=x, h2=h, u=u)
        z = self._linear(u, p + "fc2.weight", p + "fc2.bias")
        x = self._r(residual + z)  # :283
        self._rec(tr, x_out=x)
        return x

    def extract_features(self, prev_output_tokens, incremental_state=None,
                         self_attn_padding_mask=None, token_embeddings=None):
        """transformer_decoder.py:348-396 with forward_embedding :263-346.  ``token_embeddings``
        ([B, T, D]; T = 1 on a decode step) replaces the embedding lookup (:329-330)."""
        cfg = self.cfg
        tokens = prev_output_tokens.to(self.device)
        if self_attn_padding_mask is None and bool(tokens.eq(cfg.padding_idx).any()):
            self_attn_padding_mask = tokens.eq(cfg.padding_idx)  # :357-361
        positions = make_positions(tokens, cfg.padding_idx)
        pos_emb = F.embedding(positions, self.w.raw("decoder.embed_positions.weight")).float()
        if incremental_state:  # non-empty dict == decode step (:324-327)
            tokens = tokens[:, -1:]
            pos_emb = pos_emb[:, -1:]
        if token_embeddings is None:
            emb = F.embedding(tokens, self.w.raw("decoder.embed_tokens.weight")).float()
        else:
            emb = self._r(token_embeddings.to(self.device).float())
        x = self._r(emb + pos_emb)  # embed_scale == 1.0 (:89, :329-335)
        x = x.transpose(0, 1).contiguous()  # [T, B, D] (:341)
        T = x.shape[0]
        if not incremental_state:  # :371-374
            attn_mask = torch.triu(
                torch.full((T, T), float("-inf"), device=self.device), 1)
        else:
            attn_mask = None
        inner_states: List = [{"tok": emb, "pos": pos_emb, "emb": x}]
        for i in range(cfg.decoder_layers):
            x = self._layer(i, x, incremental_state, attn_mask, self_attn_padding_mask)
        inner_states.append(x)
        x = self._r(layer_norm(x, self.w["decoder.layer_norm.weight"],
                               self.w["decoder.layer_norm.bias"]))  # :392-393
        return x, {"inner_states": inner_states}

    def output_layer(self, features):
        """transformer_decoder.py:398-428: tied projection, no bias."""
        return self._linear(features, "decoder.embed_tokens.weight")

    def forward(self, prev_output_tokens, incremental_state=None, features_only=False,
                self_attn_padding_mask=None, token_embeddings=None):
        x, extra = self.extract_features(prev_output_tokens, incremental_state,
                                         self_attn_padding_mask, token_embeddings)
        if not features_only:
            x = self.output_layer(x)
        return x.transpose(0, 1).contiguous(), extra  # :536

    __call__ = forward


def sample_topp(lprobs: torch.Tensor, topp, generator=None, noise=None):
    """Nucleus choice of SequenceGenerator._sample_topp (metaseq/sequence_generator.py:399-441)
    for ``topp`` a float or a [rows, 1] tensor.  Returns (scores, token ids, the truncated
    renormalised distribution in sorted order, the sort indices).

    The reference draws with ``torch.multinomial``.  With ``noise`` ([rows, vocab] independent
    Exp(1) numbers, one per token id) the same categorical draw is made as an exponential race
    instead - the arg-max of probability / noise, which is how multinomial itself draws one
    sample, there over sorted ranks - so that two implementations fed the same noise must pick
    the same token."""
    probs = torch.softmax(lprobs, dim=-1)  # :416
    sprobs, sinds = probs.sort(dim=-1, descending=True)
    if torch.is_tensor(topp):
        topp = topp.to(sprobs.device).expand(sprobs.size())
    mask = (sprobs.cumsum(dim=-1) - sprobs) >= topp  # :420-427
    trunc = sprobs.clone()
    trunc[mask] = 0
    trunc = trunc / trunc.sum(dim=-1, keepdim=True)  # :430
    rows = torch.arange(lprobs.size(0), device=lprobs.device)
    if noise is not None:
        by_id = torch.zeros_like(trunc).scatter_(1, sinds, trunc)
        toks = (by_id / noise).argmax(dim=-1)
        return probs[rows, toks].log(), toks, trunc, sinds
    choices = torch.multinomial(trunc, 1, generator=generator)[:, 0]  # :431
    return sprobs[rows, choices].log(), sinds[rows, choices], trunc, sinds  # :433-434


def update_sampling_topp(tok_ids, toks_since_reset, init_p, full_stop_list, lambda_decay,
                         omega_bound):
    """Factual-nucleus decay of p, one value per row
    (metaseq/sequence_generator.py:443-476, the 1-D-tokens branch :465-476).  Updates
    ``toks_since_reset`` in place and returns the new p per row."""
    new_p = init_p.clone()
    for i, t in enumerate(tok_ids.tolist()):
        if t in full_stop_list:
            toks_since_reset[i] = 0
        else:
            toks_since_reset[i] += 1
        decay = max(0, int(toks_since_reset[i]) - 1)
        new_p[i] = max(omega_bound, float(init_p[i]) * lambda_decay ** decay)
    return new_p


def apply_repetition_penalties(lprobs, count_tokens, count_tokens_src, alpha_presence=0.0,
                               alpha_frequency=0.0, alpha_presence_src=0.0,
                               alpha_frequency_src=0.0):
    """mu[j] - c[j] * alpha_frequency - [c[j] > 0] * alpha_presence, for the generated-token
    counts and the prompt-token counts (metaseq/sequence_generator.py:478-523)."""
    if alpha_frequency > 0 or alpha_presence > 0:
        lprobs = lprobs - count_tokens * alpha_frequency - count_tokens.gt(0) * alpha_presence
    if alpha_frequency_src > 0 or alpha_presence_src > 0:
        lprobs = (lprobs - count_tokens_src * alpha_frequency_src
                  - count_tokens_src.gt(0) * alpha_presence_src)
    return lprobs


def generate(decoder, src_tokens: torch.Tensor, max_len_b: int, min_len: int = 1,
             pad: int = 1, eos: int = 2, stop: Optional[List[int]] = None,
             temperature: float = 1.0, max_positions: Optional[int] = None,
             return_step_logits: bool = False, beam_size: int = 1, topp: float = -1,
             lambda_decay: float = -1, omega_bound: float = 0.3, full_stop_list=(3, 3, 3),
             alpha_presence: float = 0.0, alpha_frequency: float = 0.0,
             alpha_presence_src: float = 0.0, alpha_frequency_src: float = 0.0,
             alpha_src_penalty_end_idx: int = -1, need_logprobs: bool = False,
             generator=None, noise_fn=None):
    """SequenceGenerator._generate (metaseq/sequence_generator.py:142-344; buffers :345-397;
    selection :399-441; factual nucleus :443-476; penalties :478-534).

    ``decoder(tokens, incremental_state=dict)`` must return ``(logits[B, T, V], extra)``.
    ``full_stop_list`` holds the ids the dictionary gives ".", "?" and "!" (:116; the unk id for
    a dictionary of BPE ids).  Factual-nucleus state is kept per row, which is what the
    reference does at beam_size 1 (its indexing fails for more).  ``noise_fn(shape)``, if
    given, supplies the Exp(1) numbers of each sampling step's draw (see ``sample_topp``).
    Returns {"tokens": [B, beam, max_len], "scores": [B, beam, max_len]} (+ "distributions"
    with ``need_logprobs``) and, on request, the logits tensors seen by the loop.
    """
    stop = stop or []
    topp = 0.0 if topp is None else max(0, topp)  # :96-98
    greedy = temperature == 0.0 or topp == 0.0  # :412
    incremental_state: Dict = {}
    device = src_tokens.device
    src_lengths = (src_tokens.ne(eos) & src_tokens.ne(pad)).long().sum(dim=1)  # :164-166
    bsz = src_tokens.shape[0]
    BB = bsz * beam_size
    if max_positions is None:
        max_positions = decoder.max_positions()
    max_len = int(min(max_positions, max_len_b or 1e99))  # :182
    min_len = min(max_len, min_len or 0)
    assert min_len <= max_len
    scores = torch.zeros(BB, max_len, device=device).float()  # :368-371
    tokens = torch.full((BB, max_len), pad, dtype=torch.long, device=device)
    start_step = src_tokens.shape[1]
    tokens[:, :start_step] = src_tokens.repeat_interleave(beam_size, 0)  # :225
    V = None
    step_logits = []
    logits = decoder(tokens[:, :start_step], incremental_state=incremental_state)[0]
    V = logits.shape[-1]
    count_tokens = count_tokens_src = None  # :372-390
    if alpha_presence > 0 or alpha_frequency > 0:
        count_tokens = torch.zeros(BB, V, device=device, dtype=torch.long)
    if alpha_presence_src > 0 or alpha_frequency_src > 0:
        src = src_tokens
        if alpha_src_penalty_end_idx > 0 and not bsz > 1:
            src = src[:, :alpha_src_penalty_end_idx]
        count_tokens_src = torch.zeros(BB, V, device=device, dtype=torch.long)
        for i in range(BB):  # the reference fills rows 0..BB-1 from src rows 0..BB-1 (:385-390)
            count_tokens_src[i] = torch.bincount(src[i], minlength=V)[:V]
    init_p = torch.full((BB,), float(topp))
    topp_rows = init_p.clone()
    toks_since_reset = torch.zeros(BB)
    all_lprobs = torch.zeros(BB, max_len, V, device=device) if need_logprobs else None
    if return_step_logits:
        step_logits.append(logits.clone())
    preds = logits.float()
    if temperature > 0 and temperature != 1.0:
        preds = preds / temperature
    lprobs = F.log_softmax(preds, dim=-1, dtype=torch.float32)  # :240
    if all_lprobs is not None:
        all_lprobs[:, 1:start_step] = lprobs[:, :-1]  # :247-250
    prompt_tokens = tokens[:, 1:start_step].unsqueeze(-1)
    scores[:, 1:start_step] = torch.gather(lprobs, -1, prompt_tokens).squeeze(-1)  # :255-258
    cut = []
    for i in range(bsz):  # :262-267
        prompt_len = int(src_lengths[i])
        scores[i * beam_size:(i + 1) * beam_size, prompt_len + 1:] = 0.0
        cut.append(lprobs[i * beam_size:(i + 1) * beam_size, prompt_len])
    lprobs = torch.cat(cut, dim=0)
    eos_mask = torch.zeros(BB, dtype=torch.bool, device=device)
    for step in range(start_step, max_len):  # :271
        if step < min_len:
            lprobs[:, eos] = -math.inf
            for t in stop:
                lprobs[:, t] = -math.inf
        lprobs[lprobs != lprobs] = -math.inf
        lprobs[:, pad] = -math.inf
        if step >= max_len - 1:  # :282-284
            lprobs[:, :eos] = -math.inf
            lprobs[:, eos + 1:] = -math.inf
        lprobs = apply_repetition_penalties(lprobs, count_tokens, count_tokens_src,
                                            alpha_presence, alpha_frequency, alpha_presence_src,
                                            alpha_frequency_src)  # :287-289
        lprobs[eos_mask, :eos] = -math.inf  # :292-293
        lprobs[eos_mask, eos + 1:] = -math.inf
        if greedy:
            next_scores, next_toks = lprobs.max(dim=-1)  # :413-415
        else:
            p = topp if lambda_decay <= 0 else topp_rows.unsqueeze(1)
            noise = noise_fn(lprobs.shape) if noise_fn is not None else None
            next_scores, next_toks, _, _ = sample_topp(lprobs, p, generator, noise)
            if lambda_decay > 0:
                topp_rows = update_sampling_topp(next_toks, toks_since_reset, init_p,
                                                 list(full_stop_list), lambda_decay, omega_bound)
        if count_tokens is not None:  # :525-534
            count_tokens[torch.arange(BB, device=device), next_toks] += 1
        tokens[:, step] = next_toks
        scores[:, step] = next_scores
        if all_lprobs is not None:
            all_lprobs[:, step] = lprobs
        eos_mask |= next_toks == eos
        for t in stop:
            eos_mask |= next_toks == t
        if bool(torch.all(eos_mask)):
            break
        logits = decoder(tokens[:, :step + 1], incremental_state=incremental_state)[0]
        if return_step_logits:
            step_logits.append(logits.clone())
        preds = logits.float()
        if temperature > 0 and temperature != 1.0:
            preds = preds / temperature
        lprobs = F.log_softmax(preds, dim=-1, dtype=torch.float32)[:, -1, :]
    beamscores = scores.view(bsz, beam_size, -1).cumsum(dim=-1)[:, :, -1]  # :326-333
    indices = beamscores.sort(dim=-1, descending=True).indices
    order = (indices + beam_size * torch.arange(bsz, device=device).unsqueeze(1)).view(-1)
    out = {"tokens": tokens[order].view(bsz, beam_size, -1),
           "scores": scores[order].view(bsz, beam_size, -1)}
    if all_lprobs is not None:
        out["distributions"] = all_lprobs[order].view(bsz, beam_size, -1, V)
    if return_step_logits:
        out["step_logits"] = step_logits
    return out


def greedy_generate(decoder, src_tokens: torch.Tensor, max_len_b: int, min_len: int = 1,
                    pad: int = 1, eos: int = 2, stop: Optional[List[int]] = None,
                    temperature: float = 1.0, max_positions: Optional[int] = None,
                    return_step_logits: bool = False):
    """``generate`` at beam 1 with greedy selection (metaseq/sequence_generator.py:413-415)."""
    return generate(decoder, src_tokens, max_len_b, min_len, pad, eos, stop, temperature,
                    max_positions, return_step_logits)
