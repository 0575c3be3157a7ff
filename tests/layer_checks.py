"""Kernel-local parity at a model's real layer shapes: every op of one decoder layer is fed the
ORACLE's own input of that op (recorded by ``OracleDecoder.trace`` during a full-depth run, so
the magnitudes are those of the real residual stream at that depth) and compared with the
oracle's output of the same op.  Whatever the depth of the model, a difference here can only
come from the op itself: both sides accumulate in fp32 and round to fp16 at the same points,
so they may differ by one fp16 ulp where another summation order straddles a rounding
boundary, on a fraction of the elements that grows with the length of the reduction.

The ops run through the decoder's own dispatch helpers (``_layernorm``, ``_qkv``, ``_linear``,
``_linear_partial``: the same entry points of the C ABI, the same kernel choices - int8
expansion, split-K, packed activations - as a real forward), then the whole layer runs chained
on its own intermediate results (``_rows_layer`` / ``_decode_layer``)."""
import math

import torch

from metaseq_amd import _capi
from metaseq_amd._capi import MSA_IN_PACKED, MSA_OUT_PACKED, check, ptr
from metaseq_amd.kv_cache import KVCache
from tests.fp16util import fp16_stats


def pack_rows(x):
    """[M, K] row-major -> the packed activation layout of include/metaseq_amd.h (M <= 128), on
    x's device."""
    M, K = x.shape
    MB = (M + 15) // 16 if M <= 64 else 8   # 65 .. 128 rows: always eight row blocks
    xp = torch.zeros(MB * 16, K, dtype=x.dtype, device=x.device)
    xp[:M] = x
    return xp.view(MB, 16, K // 32, 4, 8).permute(2, 0, 3, 1, 4).contiguous().view(-1)


def unpack_rows(xp, M, K):
    MB = (M + 15) // 16 if M <= 64 else 8   # 65 .. 128 rows: always eight row blocks
    x = xp.view(K // 32, MB, 4, 16, 8).permute(1, 3, 0, 2, 4).contiguous().view(MB * 16, K)
    return x[:M]


class Report:
    """Collects (op, max ulp, fraction differing, elements beyond the bound) and asserts."""

    def __init__(self, tag):
        self.tag, self.rows = tag, []

    def cmp(self, op, got, want, stages=1, max_frac=3e-2, also=None, acc=None):
        """``stages``: the number of fp16 rounding points the op passes through (matrix product,
        bias add, scaling, residual add ...).  Two implementations that round at the same points
        and differ only in the order of their fp32 sums can end up one ulp apart per stage, so
        an element may be ``stages`` ulp off, or ``stages`` x 2^-10 (one fp16 ulp, relatively) of
        its own magnitude plus ``also``: a tensor (broadcastable to the result) bounding the
        magnitude of the op's INTERMEDIATE results, since a 1-ulp step of an intermediate
        survives at the intermediate's magnitude even where the final value is smaller (a bias
        that cancels, the other summand of a residual add).  ``acc`` = (K, products): the op sums
        K products in fp32, whose own rounding error - about 2^-24 sqrt(K) times the size of the
        running sum, on either side - exceeds an fp16 ulp of results that are small against
        that sum; ``products`` is a tensor with the magnitude of the sums."""
        want = want.to(got.device)
        floor = stages * 2.0 ** -24
        if acc is not None:
            floor += acc_floor(*acc)
        mag = want.abs().to(torch.float16)
        if also is not None:
            mag = mag + also.abs().to(torch.float16)
        worst, frac, n_bad, worst_abs, worst_rel = fp16_stats(
            got, want, max_ulp=stages, mag=mag, rel=stages * 1.01 * 2.0 ** -10, floor=floor)
        self.rows.append((op, worst_rel, frac, n_bad))
        print("  %-28s %-22s %.3f %% of elements differ, the worst by %.2f of its allowance"
              % (self.tag, op, 100 * frac, worst_rel), flush=True)
        assert n_bad == 0, "%s %s: %d elements beyond %d ulp and the magnitude bound (worst " \
            "%.3g abs)" % (self.tag, op, n_bad, stages, worst_abs)
        assert frac <= max_frac, "%s %s: %.4f of the elements differ" % (self.tag, op, frac)

    def cmp_chained(self, got, want, x_in, rms_bound=2.0 ** -9, max_bound=2.0 ** -5):
        """The whole layer on its own intermediate results.  One-ulp steps of an op's output are
        input noise of the next op, so the results are not ulp-close element by element; what
        stays small is the error against the layer's own contribution u = x_out - x_in: every
        intermediate carries a relative rounding noise of about 2^-11, and a handful of them add
        up.  The root-mean-square error is bounded relative to rms(u), the largest error by
        ``max_bound`` rms(u) plus four ulps of the element itself (the residual stream has
        elements many times larger than the layer's contribution)."""
        want = want.to(got.device)
        u = want.float() - x_in.to(got.device).float()
        scale = float(u.pow(2).mean().sqrt())
        d = got.float() - want.float()
        rms = float(d.pow(2).mean().sqrt()) / scale
        mx = float((d.abs() / (max_bound * scale + 2.0 ** -8 * want.float().abs())).max())
        print("  %-28s %-22s rms error %.2e of the layer's rms contribution, the worst element "
              "by %.2f of its allowance" % (self.tag, "whole layer, chained", rms, mx), flush=True)
        assert rms <= rms_bound and mx <= 1.0, (self.tag, rms, mx)


def acc_floor(K, products):
    """Absolute slack for the fp32 rounding error of a K-term sum whose running value has the
    root-mean-square size of ``products``: 8 x 2^-24 sqrt(K) rms."""
    rms = float(products.float().pow(2).mean().sqrt())
    return 8 * 2.0 ** -24 * K ** 0.5 * rms


def ln_also(x, mag, ln, stages=1):
    """Magnitude bound for a LayerNorm of ``x`` whose elements may be off by ``stages`` ulp of
    ``mag`` (the magnitude bound of the op that produced x): the normalised value moves by that
    step over the row's standard deviation, whatever its own size."""
    sigma = x.float().var(dim=-1, unbiased=False, keepdim=True).add(1e-5).sqrt()
    return (mag.float().abs() / sigma * ln.weight.float().abs().view(1, -1)) * stages


def attention_allowance(q, kc, vc, B, T, S, H, hd):
    """What bounds the error of an attention output for T queries ``q`` [B * T, H * hd] over the
    first S positions of the caches (query t sees keys 0 .. S - T + t):

    * sum_j p_j |v_j|, the magnitude of the products the output is summed from (an output that
      cancels to nearly zero is still only as exact as one ulp of those products);
    * the number of rounding stages: the probabilities and the output are rounded once each, and
      a score that lands one fp16 ulp away scales its probability by e^ulp(s): one more stage
      per 2^-10 of ulp(largest |score|).

    Plain torch ops (not the checker: only the allowance of the check is formed here)."""
    out = torch.empty(B, T, H, hd, dtype=torch.float32, device=q.device)
    causal = torch.full((T, S), float("-inf"), device=q.device).triu(S - T + 1)
    q4 = q.view(B, T, H, hd)
    smax = 0.0
    for b in range(B):
        qq = q4[b].permute(1, 0, 2).float()                        # [H, T, hd]
        s = (qq @ kc[b, :, :S].float().transpose(1, 2)).half().float()
        smax = max(smax, float(torch.where(causal == 0, s, torch.zeros_like(s)).abs().max()))
        p = torch.softmax(s + causal, dim=-1)
        out[b] = (p @ vc[b, :, :S].float().abs()).permute(1, 0, 2)
    stages = 2 + max(1, int(2.0 ** math.floor(math.log2(max(smax, 1.0)))))
    return out.reshape(B * T, H * hd), stages


def _heads(t, B, T, H, hd):
    """[B * T, H * hd] -> [B, H, T, hd] (the cache's layout)."""
    return t.view(B, T, H, hd).permute(0, 2, 1, 3)


def check_prefill_layer(dec, i, tr, B, T, tag):
    """Layer ``i`` of ``dec`` over B * T prompt rows against the oracle's trace ``tr`` of the same
    pass (dict of batch-major fp16 tensors)."""
    lib = dec.prepare_()
    stream = _capi.stream_ptr()
    cfg = dec.cfg
    D, H, hd, F = (cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim,
                   cfg.decoder_ffn_embed_dim)
    layer = dec.layers[i]
    M = B * T
    dev = tr["x_in"].device
    rep = Report("%s layer %d prefill" % (tag, i))
    work = dec._rows_buffers(M, dev)
    q, h, o, u = work["q"], work["h"], work["o"], work["u"]
    kv = torch.empty(2, B, H, T, hd, dtype=torch.float16, device=dev)

    dec._layernorm(lib, stream, tr["x_in"], layer.self_attn_layer_norm, M, D, h)
    rep.cmp("LayerNorm 1", h, tr["h1"])
    dec._qkv(lib, stream, tr["h1"], layer.self_attn.qkv_proj, q, kv[0], kv[1], B, T, H, hd, 0, T,
             D, 0)
    # q passes three rounding points (product, bias add, scaling by hd^-0.5), k and v two
    bk, bv, bq = layer.self_attn.qkv_proj.bias.view(3, 1, D)
    rep.cmp("qkv_proj: q", q, tr["q"], stages=3, also=bq * hd ** -0.5, acc=(D, tr["q"]))
    rep.cmp("qkv_proj: k", kv[0], _heads(tr["k"], B, T, H, hd), stages=2,
            also=bk.view(1, H, 1, hd), acc=(D, tr["k"]))
    rep.cmp("qkv_proj: v", kv[1], _heads(tr["v"], B, T, H, hd), stages=2,
            also=bv.view(1, H, 1, hd), acc=(D, tr["v"]))
    kv[0].copy_(_heads(tr["k"], B, T, H, hd))
    kv[1].copy_(_heads(tr["v"], B, T, H, hd))
    check(lib.msa_attention_f16(ptr(tr["q"]), ptr(kv[0]), ptr(kv[1]), None, 0, ptr(o), B, H, hd,
                                T, 0, T, 0, None, stream))
    also, stages = attention_allowance(tr["q"], kv[0], kv[1], B, T, T, H, hd)
    rep.cmp("attention", o, tr["o"], stages=stages, also=also)
    del also
    x = tr["x_in"].clone()
    dec._linear(lib, stream, tr["o"], layer.self_attn.out_proj, M, D, D, residual=x, out=x)
    rep.cmp("out_proj + residual", x, tr["x_mid"], stages=3,
            also=tr["x_in"].abs() + layer.self_attn.out_proj.bias.abs().view(1, D),
            acc=(D, tr["x_mid"].float() - tr["x_in"].float()))
    dec._layernorm(lib, stream, tr["x_mid"], layer.final_layer_norm, M, D, h)
    rep.cmp("LayerNorm 2", h, tr["h2"])
    dec._linear(lib, stream, tr["h2"], layer.fc1, M, F, D, relu=True, out=u)
    rep.cmp("fc1 + ReLU", u, tr["u"], stages=2, also=layer.fc1.bias.view(1, F), acc=(D, tr["u"]))
    x = tr["x_mid"].clone()
    dec._linear(lib, stream, tr["u"], layer.fc2, M, D, F, residual=x, out=x)
    rep.cmp("fc2 + residual", x, tr["x_out"], stages=3,
            also=tr["x_mid"].abs() + layer.fc2.bias.abs().view(1, D),
            acc=(F, tr["x_out"].float() - tr["x_mid"].float()))
    x = tr["x_in"].clone()
    dec._rows_layer(lib, stream, layer, x, work, B, T, 0, kv[0], kv[1], T, None)
    rep.cmp_chained(x, tr["x_out"], tr["x_in"])
    torch.cuda.synchronize()
    return rep


def check_decode_layer(dec, i, trace, j, B, n0, tag):
    """Layer ``i`` of ``dec`` for the decode step that the oracle made as its pass ``j`` >= 1
    (``trace``: the list of that layer's recorded passes; pass 0 is the prefill of n0
    positions), on the packed <= 128-row path."""
    lib = dec.prepare_()
    stream = _capi.stream_ptr()
    cfg = dec.cfg
    D, H, hd, F = (cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim,
                   cfg.decoder_ffn_embed_dim)
    layer = dec.layers[i]
    t = trace[j]
    dev = t["x_in"].device
    S0 = n0 + j - 1                     # positions already in the history
    cap = S0 + 8
    rep = Report("%s layer %d decode step %d" % (tag, i, j))
    cache = KVCache(1, B, H, hd, cap, dev)
    kc, vc = cache.k(0), cache.v(0)
    kc[:, :, :n0].copy_(_heads(trace[0]["k"], B, n0, H, hd))
    vc[:, :, :n0].copy_(_heads(trace[0]["v"], B, n0, H, hd))
    for s in range(1, j):
        kc[:, :, n0 + s - 1].copy_(trace[s]["k"].view(B, H, hd))
        vc[:, :, n0 + s - 1].copy_(trace[s]["v"].view(B, H, hd))
    bufs = dec._step_buffers(cache, B)
    x, q, h, o, u, part = (bufs[k] for k in ("x", "q", "h", "o", "u", "part"))
    S_o, S_f = bufs["S_o"], bufs["S_f"]
    IN, OUT = MSA_IN_PACKED, MSA_OUT_PACKED

    x.copy_(t["x_in"])
    dec._layernorm(lib, stream, x, layer.self_attn_layer_norm, B, D, h, OUT)
    rep.cmp("LayerNorm 1", unpack_rows(h, B, D), t["h1"])
    h.copy_(pack_rows(t["h1"]))
    dec._qkv(lib, stream, h, layer.self_attn.qkv_proj, q, kc, vc, B, 1, H, hd, S0, cap, D, IN, None)
    bk, bv, bq = layer.self_attn.qkv_proj.bias.view(3, 1, D)
    rep.cmp("qkv_proj: q", q, t["q"], stages=3, also=bq * hd ** -0.5, acc=(D, t["q"]))
    rep.cmp("qkv_proj: k", kc[:, :, S0], t["k"].view(B, H, hd), stages=2, also=bk.view(1, H, hd),
            acc=(D, t["k"]))
    rep.cmp("qkv_proj: v", vc[:, :, S0], t["v"].view(B, H, hd), stages=2, also=bv.view(1, H, hd),
            acc=(D, t["v"]))
    kc[:, :, S0].copy_(t["k"].view(B, H, hd))
    vc[:, :, S0].copy_(t["v"].view(B, H, hd))
    q.copy_(t["q"])
    check(lib.msa_attention_f16(ptr(q), ptr(kc), ptr(vc), None, 0, ptr(o), B, H, hd, 1, S0, cap,
                                OUT, None, stream))
    also, stages = attention_allowance(t["q"], kc, vc, B, 1, S0 + 1, H, hd)
    rep.cmp("attention", unpack_rows(o, B, D), t["o"], stages=stages, also=also)
    o.copy_(pack_rows(t["o"]))
    x.copy_(t["x_in"])
    op, ln = layer.self_attn.out_proj, layer.final_layer_norm
    dec._linear_partial(lib, stream, o, op, part, B, D, D, S_o)
    check(lib.msa_residual_layernorm_f16(ptr(part), S_o, ptr(op.bias), ptr(x), ptr(ln.weight),
                                         ptr(ln.bias), ptr(h), B, D, 1e-5, OUT, stream))
    rep.cmp("out_proj + residual", x, t["x_mid"], stages=3,
            also=t["x_in"].abs() + op.bias.abs().view(1, D),
            acc=(D, t["x_mid"].float() - t["x_in"].float()))
    # the fused LayerNorm reads the kernel's own x: where that is an ulp off, so is its row
    rep.cmp("... fused LayerNorm 2", unpack_rows(h, B, D), t["h2"], stages=2,
            also=ln_also(t["x_mid"], t["x_mid"].abs() + t["x_in"].abs() + op.bias.abs().view(1, D),
                         ln, 3))
    h.copy_(pack_rows(t["h2"]))
    dec._linear(lib, stream, h, layer.fc1, B, F, D, relu=True, out=u, flags=IN | OUT)
    rep.cmp("fc1 + ReLU", unpack_rows(u, B, F), t["u"], stages=2, also=layer.fc1.bias.view(1, F),
            acc=(D, t["u"]))
    u.copy_(pack_rows(t["u"]))
    x.copy_(t["x_mid"])
    dec._linear_partial(lib, stream, u, layer.fc2, part, B, D, F, S_f)
    check(lib.msa_residual_layernorm_f16(ptr(part), S_f, ptr(layer.fc2.bias), ptr(x), None, None,
                                         None, B, D, 1e-5, 0, stream))
    rep.cmp("fc2 + residual", x, t["x_out"], stages=3,
            also=t["x_mid"].abs() + layer.fc2.bias.abs().view(1, D),
            acc=(F, t["x_out"].float() - t["x_mid"].float()))
    # chained, from the layer's input
    x.copy_(t["x_in"])
    dec._layernorm(lib, stream, x, layer.self_attn_layer_norm, B, D, h, OUT)
    dec._decode_layer(lib, stream, layer, kc, vc, cap, bufs, B, S0, None, None, None, None, 0)
    rep.cmp_chained(x, t["x_out"], t["x_in"])
    torch.cuda.synchronize()
    return rep


def check_rows_decode_layer(dec, i, trace, j, B, n0, tag):
    """As check_decode_layer for a decode batch above 128 rows: row-major activations through
    ``_rows_layer`` (tile kernels; split-K partial sums + the fused tail where the library
    suggests slices)."""
    lib = dec.prepare_()
    stream = _capi.stream_ptr()
    cfg = dec.cfg
    D, H, hd, F = (cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim,
                   cfg.decoder_ffn_embed_dim)
    layer = dec.layers[i]
    t = trace[j]
    dev = t["x_in"].device
    S0 = n0 + j - 1
    cap = S0 + 8
    rep = Report("%s layer %d decode step %d (row-major)" % (tag, i, j))
    cache = KVCache(1, B, H, hd, cap, dev)
    kc, vc = cache.k(0), cache.v(0)
    kc[:, :, :n0].copy_(_heads(trace[0]["k"], B, n0, H, hd))
    vc[:, :, :n0].copy_(_heads(trace[0]["v"], B, n0, H, hd))
    for s in range(1, j):
        kc[:, :, n0 + s - 1].copy_(trace[s]["k"].view(B, H, hd))
        vc[:, :, n0 + s - 1].copy_(trace[s]["v"].view(B, H, hd))
    work = dec._rows_buffers(B, dev)
    h, u = work["h"], work["u"]
    op, ln = layer.self_attn.out_proj, layer.final_layer_norm
    x = t["x_in"].clone()
    o = t["o"].clone()
    split = dec._linear_split(lib, stream, o, op, x, work, B, D, D, ln=ln, ln_out=h)
    if not split:
        dec._linear(lib, stream, o, op, B, D, D, residual=x, out=x)
        dec._layernorm(lib, stream, x, ln, B, D, h)
    rep.cmp("out_proj + residual" + (" (split-K)" if split else ""), x, t["x_mid"], stages=3,
            also=t["x_in"].abs() + op.bias.abs().view(1, D),
            acc=(D, t["x_mid"].float() - t["x_in"].float()))
    rep.cmp("... LayerNorm 2", h, t["h2"], stages=2,
            also=ln_also(t["x_mid"], t["x_mid"].abs() + t["x_in"].abs() + op.bias.abs().view(1, D),
                         ln, 3))
    dec._linear(lib, stream, t["h2"].clone(), layer.fc1, B, F, D, relu=True, out=u)
    rep.cmp("fc1 + ReLU", u, t["u"], stages=2, also=layer.fc1.bias.view(1, F), acc=(D, t["u"]))
    x = t["x_mid"].clone()
    uu = t["u"].clone()
    split = dec._linear_split(lib, stream, uu, layer.fc2, x, work, B, D, F)
    if not split:
        dec._linear(lib, stream, uu, layer.fc2, B, D, F, residual=x, out=x)
    rep.cmp("fc2 + residual" + (" (split-K)" if split else ""), x, t["x_out"], stages=3,
            also=t["x_mid"].abs() + layer.fc2.bias.abs().view(1, D),
            acc=(F, t["x_out"].float() - t["x_mid"].float()))
    # chained, from the layer's input
    x = t["x_in"].clone()
    dec._rows_layer(lib, stream, layer, x, work, B, 1, S0, kc, vc, cap, None)
    rep.cmp_chained(x, t["x_out"], t["x_in"])
    torch.cuda.synchronize()
    return rep
