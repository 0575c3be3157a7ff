"""The GEMM entry points at the REAL reduction lengths of the two largest benchmark
configurations: OPT-30B's fc2 sums over 28 672 products per output, OPT-66B's over 36 864 (the
shapes of tests/test_gpu_kernels.py stop at K = 4096).  A long reduction is where a summation
scheme shows: fp32 partial sums of a K range, split-K slices added in slice order, the int8
weights dequantised on the way.  Inputs are drawn and the expected values computed on the
device (the oracle's ``linear`` is device-agnostic; it is handed float64 copies of the fp16
values here, so the expected sums are exact and rounded at the reference's rounding points, and
what is measured is the kernels' own fp32 summation); everything goes through the C ABI.

Bound: one fp16 ulp per rounding point the op passes through (an fp32 sum in another order
straddles a rounding boundary more often the longer the sum: a fraction of a per cent of the
elements here), or the same step at the magnitude of an intermediate result (bias, residual)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import opt_oracle as O
from tests.fp16util import fp16_stats
from tests.layer_checks import acc_floor, pack_rows, unpack_rows

pytestmark = pytest.mark.gpu
DEV = "cuda"
IN_PACKED, OUT_PACKED, RELU = 2, 4, 1


@pytest.fixture(scope="module")
def lib():
    from metaseq_amd import _capi
    return _capi.load()


def P(t):
    return None if t is None else t.data_ptr()


def ok(rc, lib):
    assert rc == 0, lib.msa_last_error().decode()


def r16(t):
    return t.to(torch.float16).float()


def draw(*shape, seed, std=1.0, mean=0.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    t = torch.empty(*shape, dtype=torch.float32, device=DEV).normal_(mean, std, generator=g)
    return t.half()


def close(got, want, what, stages=1, also=None, max_frac=1e-2, acc=None):
    """``stages`` fp16 rounding points: one ulp per stage, or that step at the magnitude of an
    intermediate result (``also``); ``acc`` = (K, products): plus the fp32 rounding error of a
    K-term sum of that size, which exceeds an fp16 ulp of the results that nearly cancel."""
    mag = want.abs().half()
    if also is not None:
        mag = mag + also.abs().half()
    floor = stages * 2.0 ** -24 + (acc_floor(*acc) if acc is not None else 0.0)
    worst, frac, n_bad, worst_abs, worst_rel = fp16_stats(
        got, want, max_ulp=stages, mag=mag, rel=stages * 1.01 * 2.0 ** -10, floor=floor)
    print("  %-40s %.3f %% of elements differ, the worst by %.2f of its allowance"
          % (what, 100 * frac, worst_rel), flush=True)
    assert n_bad == 0, "%s: %d elements beyond %d ulp (worst %.3g abs)" % (what, n_bad, stages,
                                                                          worst_abs)
    assert frac <= max_frac, "%s: %.4f of the elements differ" % (what, frac)


def _weights(lib, N, K, w8):
    """(packed weight, scales or None, the fp16 matrix the reference multiplies by)."""
    W = draw(N, K, seed=8, std=0.02)
    if not w8:
        Wp = torch.empty_like(W)
        ok(lib.msa_pack_weight_f16(P(W), P(Wp), N, K, None), lib)
        return Wp, None, W
    q, s = O.quantize_int8(W)
    del W
    qp = torch.empty_like(q)
    ok(lib.msa_pack_weight_i8(P(q.contiguous()), P(qp), N, K, None), lib)
    return qp, s.contiguous(), O.dequantize_int8(q, s)


def _linear(lib, x, Wp, s, b, res, y, M, N, K, flags):
    if s is None:
        ok(lib.msa_linear_f16(P(x), P(Wp), P(b), P(res), P(y), M, N, K, flags, None), lib)
    else:
        ok(lib.msa_linear_w8a16(P(x), P(Wp), P(s), P(b), P(res), P(y), M, N, K, flags, None), lib)


# (N, K): fc2 and fc1 of OPT-30B, fc2 and fc1 of OPT-66B
SHAPES = [(7168, 28672), (28672, 7168), (9216, 36864), (36864, 9216)]


@pytest.mark.parametrize("w8", [False, True])
@pytest.mark.parametrize("N,K", SHAPES)
def test_decode_rows_at_real_reduction_lengths(lib, N, K, w8):
    """1, 16 and 64 packed rows: the weight-streaming kernels, with bias + ReLU (fc1's epilogue)
    and as split-K partial sums followed by the fused bias + residual + LayerNorm tail (fc2's)."""
    Wp, s, Wref = _weights(lib, N, K, w8)
    b = draw(N, seed=9, std=0.02)
    g, be = draw(N, seed=11, std=0.02, mean=1.0), draw(N, seed=12, std=0.02)
    for M in (1, 16, 64):
        print("decode rows", M, N, K, "int8" if w8 else "fp16", flush=True)
        # activations as the layer sees them: LayerNorm output (fc1), ReLU output (fc2)
        x = draw(M, K, seed=7 + M)
        if K > N:
            x = F.relu(x)
        res = draw(M, N, seed=10, std=4.0)
        lin = O.linear(x.double(), Wref.double(), b.double(), r16)  # exact products and sums
        want = F.relu(lin).half()
        xp = pack_rows(x)
        y = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
        _linear(lib, xp, Wp, s, b, None, y, M, N, K, IN_PACKED | RELU)
        close(y, want, "bias + ReLU, %d rows" % M, stages=2, also=b.view(1, N), acc=(K, lin))
        MB = (M + 15) // 16
        yp = torch.zeros(MB * 16 * N, dtype=torch.float16, device=DEV)
        _linear(lib, xp, Wp, s, b, None, yp, M, N, K, IN_PACKED | OUT_PACKED | RELU)
        assert torch.equal(unpack_rows(yp, M, N), y)
        if N > 16384:
            continue  # the fused tail normalises rows of d_model elements, never of the FFN's
        # split-K with the library's own choice of slices, then the fused tail
        splits = lib.msa_linear_default_splits_w8a16 if w8 else lib.msa_linear_default_splits
        S = splits(M, N, K)
        part = torch.full((S, M, N), float("nan"), dtype=torch.float32, device=DEV)
        if w8:
            ok(lib.msa_linear_partial_w8a16(P(xp), P(Wp), P(s), P(part), M, N, K, S, IN_PACKED,
                                            None), lib)
        else:
            ok(lib.msa_linear_partial_f16(P(xp), P(Wp), P(part), M, N, K, S, IN_PACKED, None), lib)
        xo = r16(lin + res.float())
        want_h = O.layer_norm(xo, g, be).half()
        xd = res.clone()
        hp = torch.zeros(MB * 16 * N, dtype=torch.float16, device=DEV)
        ok(lib.msa_residual_layernorm_f16(P(part), S, P(b), P(xd), P(g), P(be), P(hp), M, N, 1e-5,
                                          OUT_PACKED, None), lib)
        torch.cuda.synchronize()
        exact = x.double() @ Wref.double().t()
        assert float((part.sum(0) - exact).abs().max()) < 4 * acc_floor(K, exact)
        close(xd, xo.half(), "split-K (%d slices) + residual, %d rows" % (S, M), stages=3,
              also=res, acc=(K, lin))
        # where x is up to 3 ulp off, the normalised value moves by that step over the row's
        # standard deviation, whatever its own size
        sigma = xo.var(dim=-1, unbiased=False, keepdim=True).add(1e-5).sqrt()
        close(unpack_rows(hp, M, N), want_h, "... fused LayerNorm", stages=2,
              also=(xo.abs() + res.float().abs()) / sigma * g.float().abs().view(1, N) * 3)


@pytest.mark.parametrize("w8", [False, True])
@pytest.mark.parametrize("N,K", [(7168, 28672), (9216, 36864), (36864, 9216)])
def test_prefill_rows_at_real_reduction_lengths(lib, N, K, w8):
    """4096 + 77 row-major rows (whole 256-row tiles plus a ragged bottom): the MFMA tile
    kernels, with bias + residual in place (fc2, out_proj) and bias + ReLU (fc1); for int8 also
    through the matrix expanded once to fp16, as the decoder runs products of this many rows."""
    M = 4096 + 77
    print("prefill rows", M, N, K, "int8" if w8 else "fp16", flush=True)
    Wp, s, Wref = _weights(lib, N, K, w8)
    b = draw(N, seed=9, std=0.02)
    x = draw(M, K, seed=7)
    if K > N:
        x = F.relu(x)
    res = draw(M, N, seed=10, std=4.0)
    plain = O.linear(x.double(), Wref.double(), b.double(), r16)  # exact products and sums
    want_res = r16(plain + res.float()).half()
    want_relu = F.relu(plain).half()
    acc = (K, plain)
    y = res.clone()
    _linear(lib, x, Wp, s, b, y, y, M, N, K, 0)
    close(y, want_res, "bias + residual (in place)", stages=3, also=res, acc=acc)
    y.fill_(float("nan"))
    _linear(lib, x, Wp, s, b, None, y, M, N, K, RELU)
    close(y, want_relu, "bias + ReLU", stages=2, also=b.view(1, N), acc=acc)
    if w8:
        We = torch.empty(N * K, dtype=torch.float16, device=DEV)
        ok(lib.msa_expand_weight_w8_f16(P(Wp), P(s), P(We), N, K, None), lib)
        back = torch.empty(N, K, dtype=torch.float16, device=DEV)
        ok(lib.msa_unpack_weight_f16(P(We), P(back), N, K, None), lib)
        assert torch.equal(back, Wref), "the expanded matrix is not round(q * scale)"
        y.copy_(res)
        ok(lib.msa_linear_f16(P(x), P(We), P(b), P(y), P(y), M, N, K, 0, None), lib)
        close(y, want_res, "expanded to fp16: bias + residual", stages=3, also=res, acc=acc)
    torch.cuda.synchronize()
