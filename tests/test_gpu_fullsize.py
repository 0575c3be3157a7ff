"""Parity at the benchmark's full sizes (BASELINE configs 2 to 5, at their real depth, batch and
prompt length).

The CPU oracle needs minutes to hours at these sizes, so the same oracle code runs on the GPU
through torch ops (it is device-agnostic; fp32 matmuls of fp16-representable values, rounded at
the reference's rounding points).  At 30B / 66B the oracle and the HIP model do not fit the
device together, so the phases run one after the other and each frees what it held:

  A. oracle: free-running greedy generation, every step's logits kept (fp16-exact values);
  B. HIP path: free-running generation through SequenceGenerator; teacher-forced prefill and
     decode steps along the ORACLE's tokens, logits within the benchmark's tolerance (max-abs
     2e-2, mean-abs 2e-3) at every step; and, if a row left the oracle's path, teacher-forced
     decode steps along the HIP path's OWN tokens, logits of those rows kept;
  C. oracle again, on the HIP path's own tokens of every row that diverged: logits within
     tolerance at every later position, and every later HIP choice is the oracle's arg-max or
     within 2 fp16 ulps of it (a numerical tie decided by the fp32 summation order).

Greedy tokens over the first 32 generated tokens must be identical, except that a row may
leave the oracle's path at such a tie; phase C then keeps checking it to the end.

At 30B / 66B depth and width two evaluations of the REFERENCE that differ only in the fp32
summation order inside their matrix products already lie further apart than the benchmark's
tolerance (rounding noise of the fp16 residual stream, decorrelated after a few layers).  Phase
A therefore also measures that floor (the oracle with fp32 products vs with torch's native fp16
products, the reference's own GPU arithmetic), and for those two configurations the bound is
the larger of the tolerance and the floor with a small margin.  Configurations 2 and 3 assert
the benchmark's tolerance as it stands."""
import gc

import pytest
import torch

from metaseq_amd import (Dictionary, SequenceGenerator, TransformerLanguageModel,
                         iter_random_state_dict, opt_config, random_prompts, random_state_dict)
from oracle.opt_oracle import dequantize_int8, greedy_generate, layer_norm, quantize_int8
from tests.common import make_oracle
from tests.layer_checks import (check_decode_layer, check_prefill_layer,
                                check_rows_decode_layer)

pytestmark = pytest.mark.gpu
DEV = "cuda"
# fp16 matrix products of the native-product oracle accumulate in fp32 throughout
torch.backends.cuda.matmul.allow_fp16_reduced_precision_reduction = False
MAX_ABS, MEAN_ABS = 2e-2, 2e-3
QUANTISED = ("qkv_proj.weight", "out_proj.weight", "fc1.weight", "fc2.weight")


def _diff(got, want):
    d = (got.float() - want.float().to(got.device)).abs()
    return float(d.max()), float(d.mean())


def _free():
    gc.collect()
    torch.cuda.empty_cache()


def _oracle_weights(cfg, int8):
    """The weights the reference runs on: the seeded fp16 draw; in the int8 configuration every
    matrix the reference quantises is replaced by its dequantised value, computed with the
    oracle's own quantiser (so the product's quantiser is checked against it as well)."""
    sd = {}
    for name, t in iter_random_state_dict(cfg, seed=1234, dtype=torch.float16, device=DEV):
        if int8 and name.endswith(QUANTISED):
            t = dequantize_int8(*quantize_int8(t))
        sd[name] = t
    return sd


def _build_model(cfg, int8):
    """The HIP model filled tensor by tensor (no second copy of the weights is ever held)."""
    model = TransformerLanguageModel.build_model(cfg, None, device=DEV)
    model.decoder.load_tensors(
        iter_random_state_dict(cfg, seed=1234, dtype=torch.float16, device=DEV),
        quantize_int8=int8)
    return model


def _masked_top(lg, pad=1, eos=2):
    """Oracle logits of one position with the ids the loop never selects before min_len removed:
    (top value, fp16 ulp at the top, gap between the two best)."""
    lg = lg.float().clone()
    lg[pad] = lg[eos] = float("-inf")
    top2 = lg.topk(2).values
    top = float(top2[0])
    ulp = 2.0 ** (torch.tensor(abs(top)).log2().floor().item() - 10) if top != 0 else 2.0 ** -24
    return lg, top, ulp, float(top2[0] - top2[1])


FULL_KEYS = None
DEPTH_ROWS = 32     # positions per batch row, from the end of the prompt, in the depth table


def _exit_logits(oracle, x_rows):
    """The logits a residual stream ``x_rows`` [rows, D] would give if the model ended there:
    final LayerNorm and vocabulary projection, evaluated in fp32 for every implementation alike
    (only the distance between residual streams is of interest)."""
    f = layer_norm(x_rows.float(), oracle.w["decoder.layer_norm.weight"],
                   oracle.w["decoder.layer_norm.bias"])
    return f @ oracle.w["decoder.embed_tokens.weight"].t()


def _run_config(size, B, P, G=32, max_pos=None, layers=None, int8=False, sequential=False,
                strict=True, check_layers=None, decode_checks=(1,)):
    """strict: the benchmark's tolerance (2e-2 / 2e-3) and the 2-ulp tie rule are asserted as
    they stand.  Otherwise (30B / 66B at full depth) the bound at every step is the larger of the
    benchmark's tolerance and the reference's own reproducibility floor, measured in the same
    run: the distance between two evaluations of the oracle that differ only in the summation
    order of their matrix products (fp32 products rounded afterwards vs torch's native fp16
    products, which is what the reference itself runs on a GPU), with 3 % of slack on the mean
    and 15 % on the maximum (a single element's statistic).

    Independently of how that floor is defined, every configuration is also held to a
    three-point check: with T = the same weights and tokens evaluated in fp32 THROUGHOUT (no
    fp16 rounding anywhere), the HIP path must be no further from T than the reference's own two
    fp16 evaluations are: x 1.05 on the mean-abs at the prefill and at every decode step; on the
    max-abs, the statistic of one element out of millions, x 1.5 at a single step and x 1.25 over
    all steps together.

    check_layers: indices of the layers whose ops are checked one by one against the oracle's
    own intermediate tensors (tests/layer_checks.py); default first, middle and last.  A table of
    the distances between the residual streams at several depths, expressed as logits, is
    printed (how the reference's own reproducibility floor grows with depth)."""
    over = {"max_target_positions": max_pos or 2048}
    if layers:
        over["decoder_layers"] = layers
    cfg = opt_config(size, **over)
    L = cfg.decoder_layers
    src = random_prompts(cfg, B, P, seed=4321, device=DEV)
    n0 = src.shape[1]
    max_len_b = n0 + G + 1
    tag = "%s%s B%d P%d L%d" % (size, "-int8" if int8 else "", B, P, L)
    if check_layers is None:
        check_layers = sorted({0, L // 2, L - 1})
    depth_layers = sorted({d - 1 for d in (2, 8, 16, 32, 48, 64) if d <= L} | {L - 1})
    n_depth = min(DEPTH_ROWS, n0)
    depth_idx = (torch.arange(B, device=DEV).unsqueeze(1) * n0
                 + torch.arange(n0 - n_depth, n0, device=DEV).unsqueeze(0)).flatten()

    # ---- phase A: the oracle's own generation, then its reproducibility floor -------------------
    print("%s: phase A (oracle generation)" % tag, flush=True)
    sd = _oracle_weights(cfg, int8)
    oracle = make_oracle(cfg, sd, torch.float16, device=DEV, lean=sequential)
    oracle.trace = {i: [] for i in sorted(set(check_layers) | set(depth_layers))}
    oracle.trace_keys = {i: (FULL_KEYS if i in check_layers else {"x_out"}) for i in oracle.trace}
    if sequential:
        oracle.trace_device = "cpu"  # tens of GB that phase A has no room for on the device
    want = greedy_generate(oracle, src, max_len_b=max_len_b, min_len=max_len_b - 1,
                           return_step_logits=True)
    traces, oracle.trace, oracle.trace_device = oracle.trace, None, None
    depth_x = {"oracle, fp32 products": {i: traces[i][0]["x_out"][depth_idx.cpu()].to(DEV)
                                         if sequential else traces[i][0]["x_out"][depth_idx]
                                         for i in depth_layers}}
    for i in depth_layers:
        if i not in check_layers:
            del traces[i]
    wt = want["tokens"][:, 0].clone()
    ref_logits = [l.half() for l in want["step_logits"]]  # values are fp16-exact already
    del want
    # the same tokens through the oracle with native fp16 matrix products
    oracle.native_matmul = True
    oracle.trace = {i: [] for i in depth_layers}
    oracle.trace_keys = {"x_out"}
    nat_logits, floor = [], []
    inc = {}
    for i in range(G + 1):
        logits = oracle(wt[:, :n0 + i], incremental_state=inc)[0]
        floor.append(_diff(logits, ref_logits[i]))
        nat_logits.append(logits.half())
        if i == 0:
            depth_x["oracle, native fp16 products"] = {
                l: oracle.trace[l][0]["x_out"][depth_idx] for l in depth_layers}
            oracle.trace = None
        del logits
    del inc
    oracle.native_matmul = False
    print("%s reference vs reference (fp32 vs native fp16 matrix products): prefill max-abs "
          "%.3e mean-abs %.3e; decode steps worst max-abs %.3e mean-abs %.3e"
          % (tag, floor[0][0], floor[0][1], max(f[0] for f in floor[1:]),
             max(f[1] for f in floor[1:])), flush=True)
    if strict:
        tol = [(MAX_ABS, MEAN_ABS)] * (G + 1)
    else:
        tol = [(max(MAX_ABS, 1.15 * f[0]), max(MEAN_ABS, 1.03 * f[1])) for f in floor]
    # the third point: fp32 throughout, one causal pass over the oracle's tokens (position p of
    # it is what the incremental evaluation produces for the history 0 .. p)
    print("%s: phase A2 (fp32-throughout evaluation of the same weights and tokens)" % tag,
          flush=True)
    truth_model = make_oracle(cfg, sd, torch.float32, device=DEV, lean=True,
                              store_dtype=torch.float16)
    truth_model.attn_chunk_bytes = oracle.attn_chunk_bytes
    truth_model.trace = {i: [] for i in depth_layers}
    truth_model.trace_keys = {"x_out"}
    full = truth_model(wt[:, :n0 + G])[0]                       # [B, n0 + G, V] fp32
    nT = n0 + G
    depth_truth = {}
    for l in depth_layers:
        xo = truth_model.trace[l][0].pop("x_out")               # [B * nT, D] fp32
        depth_truth[l] = xo.view(B, nT, -1)[:, n0 - n_depth:n0].reshape(B * n_depth, -1).clone()
        del xo
    truth_model.trace = None
    truth = [full[:, :n0]] + [full[:, n0 + i - 1:n0 + i] for i in range(1, G + 1)]
    # how far each of the reference's two fp16 evaluations is from it
    e_ref = [_diff(ref_logits[i], truth[i]) for i in range(G + 1)]
    e_nat = [_diff(nat_logits[i], truth[i]) for i in range(G + 1)]
    del nat_logits
    print("%s distance from the fp32-throughout evaluation, prefill (max-abs / mean-abs): oracle "
          "fp32 products %.3e / %.3e, oracle native fp16 products %.3e / %.3e"
          % (tag, e_ref[0][0], e_ref[0][1], e_nat[0][0], e_nat[0][1]), flush=True)
    # the depth table's logits are formed with the oracle's final LayerNorm and embedding
    depth_logits = {"truth": {l: _exit_logits(truth_model, depth_truth[l]) for l in depth_layers}}
    for name, xs in depth_x.items():
        depth_logits[name] = {l: _exit_logits(truth_model, xs[l]) for l in depth_layers}
    del depth_truth, depth_x
    if sequential:
        exit_w = {k: truth_model.w.raw(k).clone() for k in (
            "decoder.layer_norm.weight", "decoder.layer_norm.bias", "decoder.embed_tokens.weight")}
        del oracle, truth_model, sd
        _free()

    # ---- phase B: the HIP path ----------------------------------------------------------------
    print("%s: phase B (HIP path)" % tag, flush=True)
    model = _build_model(cfg, int8)
    dec = model.decoder
    # kernel-local parity first: every op of the chosen layers on the oracle's own inputs
    for i in check_layers:
        passes = [{k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in t.items()}
                  for t in traces.pop(i)[:max(decode_checks) + 1]]
        check_prefill_layer(dec, i, passes[0], B, n0, tag)
        for j in decode_checks:
            if j < len(passes):   # the packed decode path up to 128 rows, row-major above
                (check_decode_layer if B <= 128 else check_rows_decode_layer)(
                    dec, i, passes, j, B, n0, tag)
        del passes
    _free()
    gen = SequenceGenerator([model], Dictionary(cfg.vocab_size), max_len_b=max_len_b,
                            min_len=max_len_b - 1)
    got = gen.generate([model], {"net_input": {"src_tokens": src}})
    gt = got["tokens"][:, 0].clone()
    del got
    dec.kv_cache_capacity = max_len_b
    same_rows = (wt == gt).all(dim=1)
    rows = (~same_rows).nonzero().flatten().tolist()
    first = {r: int((wt[r] != gt[r]).nonzero()[0]) for r in rows}

    def teacher_forced(toks):
        """Prefill + G decode steps along `toks`; yields (position, logits[B, T, V]) where the
        last row of the logits at position p predicts the token at p + 1."""
        inc = {}
        logits = model(toks[:, :n0], incremental_state=inc)[0]
        yield n0 - 1, logits
        for t in range(n0, n0 + G):
            yield t, dec(toks[:, :t + 1], incremental_state=inc)[0]

    # teacher-forced along the oracle's tokens: within tolerance at every step, and no further
    # from the fp32-throughout evaluation than the reference's own fp16 evaluations are
    hip_x = {}
    dec.layer_probe = lambda i, x: hip_x.update({i: x[depth_idx].clone()}) \
        if i in depth_layers else None
    worst = (0.0, 0.0)
    worst_three = (0.0, 0.0)
    worst_hip_T = worst_ref_T = 0.0
    agree = 0
    at_divergence = {}
    for i, (p, logits) in enumerate(teacher_forced(wt)):
        dec.layer_probe = None
        mx, mean = _diff(logits, ref_logits[i])
        t_mx, t_mean = _diff(logits, truth[i])
        b_mx, b_mean = max(e_ref[i][0], e_nat[i][0]), max(e_ref[i][1], e_nat[i][1])
        worst_three = (max(worst_three[0], t_mx / b_mx), max(worst_three[1], t_mean / b_mean))
        worst_hip_T, worst_ref_T = max(worst_hip_T, t_mx), max(worst_ref_T, b_mx)
        if i == 0:
            print("%s prefill: max-abs %.3e mean-abs %.3e; from the fp32-throughout evaluation "
                  "%.3e / %.3e (the reference's two: %.3e / %.3e and %.3e / %.3e)"
                  % (tag, mx, mean, t_mx, t_mean, e_ref[0][0], e_ref[0][1], e_nat[0][0],
                     e_nat[0][1]), flush=True)
        else:
            worst = (max(worst[0], mx), max(worst[1], mean))
            agree += int((logits[:, -1].float().argmax(-1)
                          == ref_logits[i][:, -1].float().argmax(-1).to(DEV)).sum())
        assert mx <= tol[i][0] and mean <= tol[i][1], (tag, p, mx, mean, tol[i])
        assert t_mean <= 1.05 * b_mean and t_mx <= 1.5 * b_mx, (
            "%s step %d: further from the fp32-throughout evaluation (%.3e / %.3e) than the "
            "reference's own fp16 evaluations (%.3e / %.3e)" % (tag, i, t_mx, t_mean, b_mx,
                                                               b_mean))
        for r in rows:
            if first[r] == p + 1:  # the step at which row r leaves: both saw the same tokens
                at_divergence[r] = (logits[r, -1].clone(), ref_logits[i][r, -1].clone())
        del logits
    print("%s decode steps: worst max-abs %.3e mean-abs %.3e; teacher-forced arg-max agreement "
          "%d / %d" % (tag, worst[0], worst[1], agree, B * G), flush=True)
    print("%s three-point check: the HIP path's distance from the fp32-throughout evaluation is "
          "at most %.3f (max-abs) / %.3f (mean-abs) of the larger of the reference's own two at "
          "any single step; largest max-abs over the prefill and %d decode steps %.3e against "
          "the reference's %.3e" % (tag, worst_three[0], worst_three[1], G, worst_hip_T,
                                    worst_ref_T), flush=True)
    assert worst_hip_T <= 1.25 * worst_ref_T, (tag, worst_hip_T, worst_ref_T)
    del truth, full

    # the residual streams at several depths, as the logits they would give
    class _W:   # the three tensors _exit_logits reads, kept past the oracle's lifetime
        def __init__(self, t):
            self.w = {k: v.float() for k, v in t.items()}
    exit_model = _W(exit_w) if sequential else truth_model
    depth_logits["HIP"] = {l: _exit_logits(exit_model, hip_x[l]) for l in depth_layers}
    print("%s distances between residual streams after n layers, as the logits they would give "
          "(mean-abs, last %d prompt positions of every row):" % (tag, n_depth), flush=True)
    print("  layers | reference vs reference | HIP vs oracle fp32 products | HIP vs oracle native "
          "| from fp32-throughout: oracle fp32 prod. / oracle native / HIP", flush=True)
    a, b = "oracle, fp32 products", "oracle, native fp16 products"
    for l in depth_layers:
        d = lambda u, v: float((depth_logits[u][l] - depth_logits[v][l]).abs().mean())
        print("  %6d | %.3e | %.3e | %.3e | %.3e / %.3e / %.3e"
              % (l + 1, d(a, b), d("HIP", a), d("HIP", b), d(a, "truth"), d(b, "truth"),
                 d("HIP", "truth")), flush=True)
        assert d("HIP", "truth") <= 1.05 * max(d(a, "truth"), d(b, "truth")), (tag, l)
    del depth_logits, hip_x, exit_model

    # free-running greedy tokens over the first G generated tokens
    print("%s free-running greedy: %d / %d rows identical over %d generated tokens"
          % (tag, int(same_rows.sum()), B, G), flush=True)
    for r in rows:
        # A row may leave the oracle's path only at a numerical tie.  The HIP path must have
        # chosen the arg-max of its own logits (which the loop above holds within tolerance of
        # the oracle's), and the oracle's own two best must be closer than twice the distance
        # between the two logit vectors - strict: within 2 fp16 ulps of each other.
        hip, ref = at_divergence[r]
        lg, top, ulp, gap = _masked_top(ref)
        hl, htop, hulp, _ = _masked_top(hip)
        c = int(gt[r, first[r]])
        dev = float((hip.float() - ref.float()).abs().max())
        print("  row %d leaves the oracle path at position %d: oracle top-2 gap %.4f = %.1f ulp, "
              "its logits differ from the oracle's by at most %.4f there"
              % (r, first[r], gap, gap / ulp, dev), flush=True)
        # (the fused selection and the stored logits may come from two kernels: 1 ulp of slack)
        assert htop - float(hl[c]) <= hulp + 1e-6, "the HIP choice is not its own arg-max"
        assert top - float(lg[c]) <= (2 * ulp if strict else max(2 * ulp, 2 * dev)) + 1e-6, \
            "divergence at a clear decision: a real mismatch"
    own = {}
    if rows:
        # the HIP path's logits along its own tokens, for the rows that diverged
        ridx = torch.tensor(rows, device=DEV)
        for p, logits in teacher_forced(gt):
            own[p] = logits[ridx, -1].clone()
            del logits
    del ref_logits, at_divergence
    if not rows and not sequential:
        return model, cfg, src
    if sequential:
        del model, gen
        _free()
    if not rows:
        return None

    # ---- phase C: the oracle along the HIP path's own tokens, rows that diverged ---------------
    print("%s: phase C (oracle on the HIP path's own tokens, %d rows)" % (tag, len(rows)),
          flush=True)
    if sequential:
        oracle = make_oracle(cfg, _oracle_weights(cfg, int8), torch.float16, device=DEV, lean=True)
    full = oracle(gt[ridx][:, :n0 + G])[0]  # [rows, n0 + G, V]: every position at once
    # one row's mean deviation scatters around the batch's: half as much slack again
    row_tol = (max(t[0] for t in tol), 1.5 * max(t[1] for t in tol))
    for j, r in enumerate(rows):
        w_abs = w_mean = w_short = 0.0
        checked = 0
        for p in range(first[r] - 1, n0 + G - 1):
            mx, mean = _diff(own[p][j], full[j, p])
            lg, top, ulp, _ = _masked_top(full[j, p])
            short = top - float(lg[int(gt[r, p + 1])])  # 0 = the oracle's own arg-max
            w_abs, w_mean, w_short = max(w_abs, mx), max(w_mean, mean), max(w_short, short / ulp)
            checked += 1
            assert mx <= row_tol[0] and mean <= row_tol[1], (tag, r, p, mx, mean, row_tol)
            assert short <= (2 * ulp if strict else max(2 * ulp, 2 * mx)) + 1e-6, (
                "row %d position %d: the HIP choice is %.1f ulp below the oracle's best on the "
                "same tokens" % (r, p + 1, short / ulp))
        print("  row %d after leaving: %d positions, logits max-abs %.3e mean-abs %.3e, HIP "
              "choices at most %.1f ulp below the oracle's best" % (r, checked, w_abs, w_mean,
                                                                    w_short), flush=True)
    del full, oracle
    if sequential:
        _free()
        return None
    return model, cfg, src


def test_config2_opt1p3b_batch8_prompt512():
    """BASELINE config 2: OPT-1.3B shape (head_dim 64), batch 8, prompt EOS + 512 ids."""
    model, cfg, src = _run_config("1.3b", 8, 512)
    # size-independent properties on the same model
    inc = {}
    a = model(src, incremental_state=inc)[0]
    inc2 = {}
    b = model(src, incremental_state=inc2)[0]
    assert torch.equal(a, b), "prefill is not run-to-run deterministic"
    nxt = torch.cat([src, torch.full((8, 1), 77, device=DEV)], 1)
    step = model.decoder(nxt, incremental_state=inc)[0]
    step2 = model.decoder(nxt, incremental_state=inc2)[0]
    assert torch.equal(step, step2), "decode step is not run-to-run deterministic"
    full = model(nxt)[0][:, -1:]
    mx, mean = _diff(step, full)
    print("incremental vs full recompute: max-abs %.3e mean-abs %.3e" % (mx, mean), flush=True)
    assert mx <= MAX_ABS and mean <= MEAN_ABS


def _need_memory(gb):
    free, total = torch.cuda.mem_get_info()
    if total < gb * 1e9:
        pytest.skip("needs ~%d GB of device memory" % gb)


def test_config3_opt6p7b_batch32_prompt1024():
    """BASELINE config 3 (the headline): OPT-6.7B shape, batch 32, prompt EOS + 1024 ids."""
    _need_memory(120)
    _run_config("6.7b", 32, 1024)
    _free()


@pytest.mark.timeout(900)
def test_config4_opt30b_batch16_prompt2048():
    """BASELINE config 4 at full depth: OPT-30B shape (48 layers, d_model 7168, 56 heads of 128,
    FFN 28672), batch 16, prompt EOS + 2048 ids (long-context prefill attention, 46 GB cache),
    first 32 generated tokens."""
    _need_memory(250)
    _run_config("30b", 16, 2048, max_pos=4096, sequential=True, strict=False)


@pytest.mark.timeout(900)
def test_config5_opt66b_int8_batch64_prompt512():
    """BASELINE config 5 at full depth: OPT-66B shape (64 layers, d_model 9216, 72 heads, FFN
    36864), int8 weight-only, batch 64, prompt EOS + 512 ids; the oracle runs on the dequantised
    fp16 weights."""
    _need_memory(250)
    _run_config("66b", 64, 512, int8=True, sequential=True, strict=False)


def test_config4_shape_opt30b_two_layers():
    """Config 4's shape with two layers and a short prompt (a quick check of the shape)."""
    _run_config("30b", 16, 96, G=16, layers=2)
    _free()


def test_config5_shape_opt66b_int8_two_layers():
    """Config 5's shape with two layers; the oracle runs on the dequantised fp16 weights."""
    _run_config("66b", 64, 48, G=16, layers=2, int8=True)
    _free()


@pytest.mark.parametrize("rows", [70, 128, 200])
def test_wide_decode_batches_at_the_6p7b_layer_shapes(rows):
    """Service-sized decode batches (replicas, many short requests) at OPT-6.7B's real layer
    shapes, two layers deep: 70 and 128 rows decode on the packed path with eight row blocks
    (checked op by op against the oracle's own intermediates, then end to end), 200 rows on
    row-major activations through the tiled kernels."""
    _run_config("6.7b", rows, 40, G=8, layers=2)
    _free()


def test_kv_cache_grows_when_no_capacity_is_given():
    cfg = opt_config("125m", max_target_positions=1024)
    sd = random_state_dict(cfg, seed=3, dtype=torch.float16, device=DEV)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    toks = random_prompts(cfg, 2, 700, seed=5, device=DEV)
    inc_small, inc_big = {}, {}
    model.decoder.kv_cache_capacity = None      # 300 + 256 positions, then geometric growth
    model(toks[:, :300], incremental_state=inc_small)
    model.decoder.kv_cache_capacity = 1024
    model(toks[:, :300], incremental_state=inc_big)
    model.decoder.kv_cache_capacity = None
    cache = model.decoder.get_cache(inc_small)
    cap0 = cache.capacity
    for t in range(300, 600):
        a = model.decoder(toks[:, :t + 1], incremental_state=inc_small)[0]
        b = model.decoder(toks[:, :t + 1], incremental_state=inc_big)[0]
        assert torch.equal(a, b), t
    assert cache.capacity > cap0 and cache.length == 600


def test_state_dict_round_trips_through_the_packed_layout():
    cfg = opt_config("125m", max_target_positions=64)
    sd = random_state_dict(cfg, seed=9, dtype=torch.float16, device=DEV)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    model(random_prompts(cfg, 1, 8, device=DEV))     # packs the weights
    assert model.decoder.layers[0].fc1.packed
    back = model.state_dict()
    assert set(back) == set(sd)
    for k, v in sd.items():
        assert torch.equal(back[k].cpu(), v.cpu()), k
    model2 = TransformerLanguageModel.build_model(cfg, back, device=DEV)
    toks = random_prompts(cfg, 2, 12, device=DEV)
    assert torch.equal(model(toks)[0], model2(toks)[0])
