"""Per-kernel parity through the C ABI: every entry point of libmetaseq_amd.so against the
oracle's restatement of the same reference op on identical seeded inputs.

Tolerance: both sides accumulate in fp32 and round to fp16 at the same points, so results
may differ only where a different fp32 summation order straddles an fp16 rounding boundary:
at most 1 fp16 ulp on a small fraction of elements (integer outputs: bit-exact)."""
import ctypes
import sys

import pytest
import torch
import torch.nn.functional as F

from oracle import opt_oracle as O
from tests.fp16util import assert_fp16_close

pytestmark = pytest.mark.gpu

DEV = "cuda"


def r16(t):
    return t.to(torch.float16).float()


@pytest.fixture(scope="module")
def lib():
    from metaseq_amd import _capi
    return _capi.load()


_KEEP = []


def P(t):
    return None if t is None else t.data_ptr()


def G(t):
    """Device copy that stays alive until the end of the test (a temporary's memory would be
    recycled by the caching allocator before the kernel reads it)."""
    if t is None:
        return None
    d = t.to(DEV)
    _KEEP.append(d)
    return d


@pytest.fixture(autouse=True)
def _drop_keepalive():
    yield
    torch.cuda.synchronize()
    _KEEP.clear()


def ok(rc, lib):
    assert rc == 0, lib.msa_last_error().decode()


IN_PACKED, OUT_PACKED = 2, 4


def pack_w(lib, w):
    """row-major [N, K] fp16 device tensor -> tile-packed copy (through the C ABI)."""
    out = torch.empty_like(w)
    ok(lib.msa_pack_weight_f16(P(w), P(out), w.shape[0], w.shape[1], None), lib)
    _KEEP.append(out)
    return out


def pack_w8(lib, q):
    out = torch.empty_like(q)
    ok(lib.msa_pack_weight_i8(P(q), P(out), q.shape[0], q.shape[1], None), lib)
    _KEEP.append(out)
    return out


def pack_act(x):
    """[M, K] -> packed activation layout (host-side restatement of the documented formula)."""
    M, K = x.shape
    MB = (M + 15) // 16 if M <= 64 else 8   # 65 .. 128 rows: always eight row blocks
    xp = torch.zeros(MB * 16, K, dtype=x.dtype)
    xp[:M] = x
    return xp.view(MB, 16, K // 32, 4, 8).permute(2, 0, 3, 1, 4).contiguous().view(-1)


def unpack_act(xp, M, K):
    MB = (M + 15) // 16 if M <= 64 else 8   # 65 .. 128 rows: always eight row blocks
    x = xp.view(K // 32, MB, 4, 16, 8).permute(1, 3, 0, 2, 4).contiguous().view(MB * 16, K)
    return x[:M]


def rnd(*shape, seed=0, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).half()


@pytest.mark.parametrize("rows,D", [(1, 64), (32, 768), (7, 2048), (32, 4096), (33, 7168),
                                    (32, 9216), (300, 1024),
                                    # many rows: 128-, 256- and 512-thread workgroups
                                    (100, 4096), (200, 768), (70, 7168), (65, 9216),
                                    # more rows than workgroups: every workgroup walks several rows
                                    (9001, 1024), (4500, 7168), (3000, 9216)])
def test_layernorm(lib, rows, D):
    print("layernorm", rows, D, flush=True)
    x = rnd(rows, D, seed=1)
    g = (1 + rnd(D, seed=2, std=0.1).float()).half()
    b = rnd(D, seed=3, std=0.1)
    want = O.layer_norm(x, g, b).half()
    y = torch.empty(rows, D, dtype=torch.float16, device=DEV)
    ok(lib.msa_layernorm_f16(P(G(x)), P(G(g)), P(G(b)), P(y), rows, D, 1e-5, 0, None),
       lib)
    torch.cuda.synchronize()
    assert_fp16_close(y, want, what="layernorm")
    if rows <= 128 and D % 32 == 0:
        MB = (rows + 15) // 16 if rows <= 64 else 8
        yp = torch.zeros(MB * 16 * D, dtype=torch.float16, device=DEV)
        ok(lib.msa_layernorm_f16(P(G(x)), P(G(g)), P(G(b)), P(yp), rows, D, 1e-5, OUT_PACKED,
                                 None), lib)
        torch.cuda.synchronize()
        assert torch.equal(unpack_act(yp.cpu(), rows, D), y.cpu())


def test_layernorm_rejects_bad_dim(lib):
    x = torch.zeros(4, 12, dtype=torch.float16, device=DEV)
    assert lib.msa_layernorm_f16(P(x), P(x), P(x), P(x), 4, 12, 1e-5, 0, None) == -1
    assert b"multiple of 8" in lib.msa_last_error()


@pytest.mark.parametrize("T_out", [1, 9])
def test_embed_positions_and_sum(lib, T_out):
    print("embed", T_out, flush=True)
    V, D, n, B, pad = 50, 64, 9, 4, 1
    E, Ptab = rnd(V, D, seed=4), rnd(n + 8, D, seed=5)
    g = torch.Generator().manual_seed(6)
    toks = torch.randint(4, V, (B, 12), generator=g)
    toks[:, 0] = 2
    toks[1, 3:5] = pad
    toks[2, 6:9] = pad        # right padded row (last token is pad)
    toks[3, 0:2] = pad        # left padded row
    view = toks[:, :n]        # strided view, as the generator passes tokens[:, :step + 1]
    pos = O.make_positions(view, pad)
    want_pos = pos[:, n - T_out:]
    want = r16(F.embedding(view[:, n - T_out:], E.float()) + F.embedding(want_pos, Ptab.float()))
    td = toks.to(DEV)
    x = torch.empty(B * T_out, D, dtype=torch.float16, device=DEV)
    po = torch.empty(B, T_out, dtype=torch.long, device=DEV)
    st = torch.zeros(1, dtype=torch.int32, device=DEV)
    ok(lib.msa_embed_f16(P(td), td.stride(0), B, n, T_out, P(G(E)), V, P(G(Ptab)),
                         Ptab.shape[0], pad, D, P(x), P(po), P(st), None, None, 0, None), lib)
    torch.cuda.synchronize()
    assert torch.equal(po.cpu(), want_pos)
    assert torch.equal(x.cpu().float().view(B, T_out, D), want)
    assert int(st) == 0


def test_embed_flags_out_of_range_ids(lib):
    V, D = 20, 64
    E, Ptab = rnd(V, D), rnd(6, D)
    toks = torch.tensor([[2, 5, 25]], device=DEV)
    x = torch.empty(1, D, dtype=torch.float16, device=DEV)
    st = torch.zeros(1, dtype=torch.int32, device=DEV)
    ok(lib.msa_embed_f16(P(toks), 3, 1, 3, 1, P(G(E)), V, P(G(Ptab)), 6, 1, D, P(x),
                         None, P(st), None, None, 0, None), lib)
    torch.cuda.synchronize()
    assert int(st) == 1


COL_FROM_LEN = 8


def test_device_side_length_matches_host_arguments(lib):
    """embed / qkv append / attention / select with the history length read from device memory
    (one entry per row, all equal here) give the results of the host-argument form, and
    msa_advance_len increments every entry."""
    B, H, hd, V, S_cap = 4, 2, 64, 64, 24
    D = H * hd
    E, Ptab = rnd(V, D, seed=4), rnd(40, D, seed=5)
    toks = torch.randint(4, V, (B, 20), generator=torch.Generator().manual_seed(1))
    td = G(toks)
    W, bq = rnd(3 * D, D, seed=2, std=0.05), rnd(3 * D, seed=3, std=0.1)
    Wp = pack_w(lib, G(W))
    Kc0, Vc0 = G(rnd(B, H, S_cap, hd, seed=6)), G(rnd(B, H, S_cap, hd, seed=7))
    ln = torch.full((B,), 11, dtype=torch.int32, device=DEV)
    outs = []
    for len_dev, n, S0 in ((None, 12, 11), (ln, 20, 0)):
        Kc, Vc = Kc0.clone(), Vc0.clone()
        x = torch.empty(B, D, dtype=torch.float16, device=DEV)
        ok(lib.msa_embed_f16(P(td), 20, B, n, 1, P(G(E)), V, P(G(Ptab)), 40, 1, D, P(x), None,
                             None, P(len_dev), None, COL_FROM_LEN if len_dev is not None else 0,
                             None), lib)
        q = torch.empty(B, D, dtype=torch.float16, device=DEV)
        xp = G(pack_act(x.cpu()))
        ok(lib.msa_qkv_proj_f16(P(xp), P(Wp), P(G(bq)), P(q), P(Kc), P(Vc), B, 1, H, hd, S0, S_cap,
                                D, IN_PACKED, P(len_dev), None), lib)
        o = torch.empty(B, D, dtype=torch.float16, device=DEV)
        ok(lib.msa_attention_f16(P(q), P(Kc), P(Vc), None, 0, P(o), B, H, hd, 1, S0, S_cap, 0,
                                 P(len_dev), None), lib)
        tok = torch.zeros(B, 20, dtype=torch.long, device=DEV)
        sc = torch.zeros(B, 20, dtype=torch.float32, device=DEV)
        ba = (ctypes.c_int32 * 1)(1)
        col = 0 if len_dev is not None else 11
        ok(lib.msa_greedy_select_f16(P(o), D, B, D, 1.0, ba, 1, ba, 0, None, None, 0, 2,
                                     P(tok[:, col]), 20, P(sc[:, col]), 20, P(len_dev), None), lib)
        torch.cuda.synchronize()
        outs.append((x.clone(), q.clone(), Kc.clone(), Vc.clone(), o.clone(), tok.clone(),
                     sc.clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert int(outs[0][5][:, 11].abs().sum()) > 0
    ok(lib.msa_advance_len(P(ln), None, B, 1, None), lib)
    torch.cuda.synchronize()
    assert ln.tolist() == [12] * B


@pytest.mark.parametrize("hd,H", [(64, 3), (128, 2)])
def test_per_row_lengths_append_and_attend_each_row_at_its_own_length(lib, hd, H):
    """A decode step over rows of different lengths (and one inactive row, length -1): every row
    gets the position embedding of its own length, appends its key and value at its own slot
    and attends exactly its own history.  Checked against the oracle's attention arithmetic
    row by row on that row's history; slots past a row's length hold NaN, so a key read beyond
    the length would poison the result."""
    print("per-row lengths", hd, H, flush=True)
    V, S_cap, pad = 64, 40, 1
    D = H * hd
    lens = [0, 7, 19, -1, 38, 3, 5]
    B = len(lens)
    E, Ptab = rnd(V, D, seed=4), rnd(S_cap + 4, D, seed=5)
    toks = torch.randint(4, V, (B, 1), generator=torch.Generator().manual_seed(1))
    toks[6, 0] = pad  # a pad as the new token: the row sits the step out
    W, bq = rnd(3 * D, D, seed=2, std=0.05), rnd(3 * D, seed=3, std=0.1)
    Wp = pack_w(lib, G(W))
    Kc, Vc = rnd(B, H, S_cap, hd, seed=6), rnd(B, H, S_cap, hd, seed=7)
    for b, n in enumerate(lens):
        Kc[b, :, max(n, 0):] = float("nan")
        Vc[b, :, max(n, 0):] = float("nan")
    Kd, Vd = G(Kc.clone()), G(Vc.clone())
    ln = torch.tensor(lens, dtype=torch.int32, device=DEV)
    x = torch.empty(B, D, dtype=torch.float16, device=DEV)
    po = torch.empty(B, 1, dtype=torch.long, device=DEV)
    sl = torch.full((B,), 99, dtype=torch.int32, device=DEV)
    ok(lib.msa_embed_f16(P(G(toks)), 1, B, 1, 1, P(G(E)), V, P(G(Ptab)), Ptab.shape[0], pad, D,
                         P(x), P(po), None, P(ln), P(sl), 0, None), lib)
    q = torch.zeros(B, D, dtype=torch.float16, device=DEV)
    ok(lib.msa_qkv_proj_f16(P(G(pack_act(x.cpu()))), P(Wp), P(G(bq)), P(q), P(Kd), P(Vd), B, 1, H,
                            hd, 0, S_cap, D, IN_PACKED, P(sl), None), lib)
    o = torch.full((B, D), 7.0, dtype=torch.float16, device=DEV)
    ok(lib.msa_attention_f16(P(q), P(Kd), P(Vd), None, 0, P(o), B, H, hd, 1, max(lens), S_cap, 0,
                             P(sl), None), lib)
    ok(lib.msa_advance_len(P(ln), P(sl), B, 1, None), lib)
    torch.cuda.synchronize()
    assert sl.tolist() == [0, 7, 19, -1, 38, 3, -1]
    assert ln.tolist() == [1, 8, 20, -1, 39, 4, 5]
    lens[6] = -1  # from here on row 6 is checked like the inactive row
    dec = O.OracleDecoder(O.OracleConfig(1, D, H, 4 * D, V, S_cap), {}, dtype=torch.float16)
    for b, n in enumerate(lens):
        if n < 0:  # inactive: nothing appended, output row untouched
            assert torch.equal(o[b].cpu(), torch.full((D,), 7.0, dtype=torch.float16))
            assert torch.equal(torch.isnan(Kd[b].cpu()), torch.isnan(Kc[b]))
            continue
        assert int(po[b]) == pad + 1 + n
        xb = r16(E[toks[b, 0]].float() + Ptab[pad + 1 + n].float())
        assert torch.equal(x[b].cpu().float(), xb)
        kvq = O.linear(xb.unsqueeze(0), W.float(), bq.float(), r16)[0]
        k, v, qq = kvq.split(D)
        qq = r16(qq * hd ** -0.5)
        assert_fp16_close(q[b], qq, atol=2e-3, max_frac=0.05, what="q")
        # the new key / value sit at slot n; slots before keep the history, slots after NaN
        kb, vb = Kd[b].cpu(), Vd[b].cpu()
        assert_fp16_close(kb[:, n].reshape(-1), k, atol=2e-3, max_frac=0.05, what="appended k")
        assert_fp16_close(vb[:, n].reshape(-1), v, atol=2e-3, max_frac=0.05, what="appended v")
        assert torch.equal(kb[:, :n], Kc[b, :, :n]) and bool(torch.isnan(kb[:, n + 1:]).all())
        want = dec.attention_core(q[b].cpu().float().view(H, 1, hd), kb[:, :n + 1].float(),
                                  vb[:, :n + 1].float(), 1)
        assert_fp16_close(o[b], want.reshape(-1), atol=2e-3, max_frac=0.05, what="attention row %d" % b)


def test_selection_with_per_row_modes(lib):
    """row_mode gives every row its own regime: MSA_ROW_BAN_EARLY removes eos and the stop ids,
    MSA_ROW_ONLY_EOS leaves only eos.  Both selection entry points, against masked arg-max."""
    M, V, K, eos = 12, 4000, 128, 2
    x, E = rnd(M, K, seed=3, std=1.0), rnd(V, K, seed=4, std=0.3)
    Ep = pack_w(lib, G(E))
    xp = G(pack_act(x))
    logits = torch.empty(M, V, dtype=torch.float16, device=DEV)
    ok(lib.msa_linear_f16(P(xp), P(Ep), None, None, P(logits), M, V, K, IN_PACKED, None), lib)
    # make eos or a stop id the plain arg-max of some rows, so the bans change the outcome
    lg = logits.float().cpu()
    stop = [int(lg[1].argmax()), int(lg[4].argmax())]
    modes = torch.tensor([0, 1, 2, 0, 1, 3, 0, 1, 2, 0, 1, 0], dtype=torch.uint8)
    want = []
    for m in range(M):
        z = lg[m].clone()
        z[1] = float("-inf")  # pad is always banned
        if modes[m] & 1:
            z[[eos] + stop] = float("-inf")
        if modes[m] & 2:
            keep = z[eos].clone()
            z[:] = float("-inf")
            z[eos] = keep
        want.append(int(z.argmax()) if bool(torch.isfinite(z).any()) else 0)
    ba = (ctypes.c_int32 * 1)(1)
    sa = (ctypes.c_int32 * 2)(*stop)
    ws = torch.empty(lib.msa_lm_head_select_workspace_bytes(M), dtype=torch.uint8, device=DEV)
    md = G(modes)
    for fused in (True, False):
        tok = torch.full((M,), -7, dtype=torch.long, device=DEV)
        sc = torch.zeros(M, dtype=torch.float32, device=DEV)
        fin = torch.zeros(M, dtype=torch.uint8, device=DEV)
        if fused:
            ok(lib.msa_lm_head_greedy_select_f16(P(xp), P(Ep), None, P(ws), M, V, K, 1.0, ba, 1, sa,
                                                 2, P(fin), P(md), 0, eos, P(tok), 1, P(sc), 1,
                                                 None, None), lib)
        else:
            ok(lib.msa_greedy_select_f16(P(logits), V, M, V, 1.0, ba, 1, sa, 2, P(fin), P(md), 0,
                                         eos, P(tok), 1, P(sc), 1, None, None), lib)
        torch.cuda.synchronize()
        assert tok.tolist() == want, (fused, tok.tolist(), want)
        assert fin.tolist() == [int(t == eos or t in stop) for t in want]
        lp = torch.log_softmax(lg, -1)
        for m in range(M):  # mode 3: eos banned and alone eligible -> (0, -inf)
            if modes[m] == 3:
                assert float(sc[m]) == float("-inf")
            else:
                assert abs(float(sc[m]) - float(lp[m, want[m]])) < 2e-5


def test_pack_roundtrip_and_layout(lib):
    """pack/unpack are inverse, and the packed layout is the documented one."""
    N, K = 48, 96
    w = rnd(N, K, seed=1)
    wp = pack_w(lib, G(w))
    back = torch.empty_like(wp)
    ok(lib.msa_unpack_weight_f16(P(wp), P(back), N, K, None), lib)
    torch.cuda.synchronize()
    assert torch.equal(back.cpu(), w)
    want = w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    assert torch.equal(wp.cpu().view(-1), want.view(-1))
    q = torch.randint(-127, 128, (32, 128), dtype=torch.int8)
    qp = pack_w8(lib, G(q))
    qb = torch.empty_like(qp)
    ok(lib.msa_unpack_weight_i8(P(qp), P(qb), 32, 128, None), lib)
    torch.cuda.synchronize()
    assert torch.equal(qb.cpu(), q)
    # block (t, ks8): lane 16g+r holds [k = 64ks8+8g..+7 | k = 64ks8+32+8g..+7] of row 16t+r,
    # every byte stored as q + 128 (i.e. with the sign bit flipped)
    want = q.view(2, 16, 2, 2, 4, 8).permute(0, 2, 4, 1, 3, 5).contiguous()
    want = (want.view(-1).to(torch.int16) + 128).to(torch.uint8)
    assert torch.equal(qp.cpu().view(-1).view(torch.uint8), want)
    x = torch.zeros(4, 40, dtype=torch.float16, device=DEV)
    assert lib.msa_pack_weight_f16(P(x), P(x), 16, 32, None) == -1      # aliased
    assert lib.msa_pack_weight_f16(P(x), P(back), 24, 32, None) == -1   # N % 16


LINEAR_SHAPES = [
    # M, N, K
    (1, 96, 64), (8, 768, 768), (32, 3072, 768), (32, 768, 3072), (33, 2048, 2048),
    (64, 4096, 4096), (17, 50272, 768), (65, 768, 768), (200, 2304, 768), (513, 4096, 1024),
    (129, 1008, 96),
    # 33 .. 64 rows: the shared-activation kernel with 1, 2 and 3 tiles per wave, a K range
    # shorter than one stage, and two passes over the workgroup's tiles
    (64, 1008, 96), (50, 24576, 256), (40, 73728, 128),
    # enough 256 x 256 tiles to take the large tiled kernel, with ragged M and N edges; a bottom
    # block of at most 128 rows goes through the streaming kernel on row-major activations
    (1000, 16400, 128), (4099, 4096, 256), (1124, 16400, 128),
    # 8 tiles across: the tiles of a full round of 256 are regrouped per XCD, those of the last,
    # partial round (with a ragged bottom tile) are not
    (9160, 2048, 128),
    # few rows under a wide output: one row tile of the four-wave kernel plus a bottom block for
    # the streaming kernel; two row tiles, the second moved up over most of the first
    (300, 32768, 128), (420, 32768, 128),
    # 65 .. 128 packed rows: the shared-activation kernel with eight row blocks and 1, 2 and 3
    # tiles per wave, several passes over a workgroup's tiles, a K range of one stage
    (128, 4096, 128), (70, 8192, 256), (96, 24576, 128), (128, 50272, 128), (127, 1008, 96),
    # 64 and 44 bottom rows with few tiles per workgroup: the streaming kernel's four-tile groups
    (4160, 4096, 256), (4140, 8192, 128),
    # exactly one full round of 256 x 256 tiles, also with a moved-up bottom tile
    (2048, 8192, 128), (2000, 8192, 192),
    # few enough tiles that the 256 x 128 ones all run at once: one row over four row tiles (moved-up
    # tile in the same round), a moved-up tile over most of its neighbour, a ragged right tile
    (1025, 4096, 256), (700, 6144, 128), (512, 16016, 192),
    # the 256 x 64 form: fewer than 256 rows (the last row repeated in the loads), a ragged right
    # tile, more than 256 rows with a ragged bottom that is not moved up
    (128, 4096, 256), (100, 2304, 128), (65, 2064, 192), (255, 6144, 64), (300, 4096, 128),
]


def _linear_want(x, W, b, res, relu):
    want = O.linear(x.float(), W.float(), None if b is None else b.float(), r16)
    if relu:
        want = F.relu(want)
    if res is not None:
        want = r16(want + res.float())
    return want


def test_linear_f16_residual_in_place_ragged_rows(lib):
    """y aliasing the residual on the large tiled kernel with a ragged bottom tile: the rows that
    the moved-up last tile shares with its neighbour must be added to exactly once."""
    M, N, K = 1000, 16384, 128
    x, W, res = rnd(M, K, seed=7), rnd(N, K, seed=8, std=0.05), rnd(M, N, seed=10)
    want = _linear_want(x, W, None, res, False).half()
    y = G(res).clone()
    ok(lib.msa_linear_f16(P(G(x)), P(pack_w(lib, G(W))), None, P(y), P(y), M, N, K, 0, None), lib)
    torch.cuda.synchronize()
    assert_fp16_close(y, want, atol=float(want.abs().max()) * 2 ** -10, what="in-place residual")


@pytest.mark.parametrize("M,N,K", LINEAR_SHAPES)
@pytest.mark.parametrize("epi", ["plain", "bias", "bias_relu", "bias_res"])
def test_linear_f16(lib, M, N, K, epi):
    """Row-major activations (tiled kernel) and, for M <= 64, packed activations (streaming
    kernel, row-major and packed outputs) against the oracle's linear."""
    print("linear", M, N, K, epi, flush=True)
    x, W = rnd(M, K, seed=7), rnd(N, K, seed=8, std=0.05)
    b = rnd(N, seed=9, std=0.1) if epi != "plain" else None
    res = rnd(M, N, seed=10) if epi == "bias_res" else None
    relu = epi == "bias_relu"
    want = _linear_want(x, W, b, res, relu).half()
    # with a second rounding point (bias / residual add) a 1-ulp difference of the intermediate
    # survives at the intermediate's magnitude even where the final value cancels to ~0
    atol = 2e-5 if epi == "plain" else float(want.abs().max()) * 2 ** -10
    Wp = pack_w(lib, G(W))
    flags = 1 if relu else 0
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
    ok(lib.msa_linear_f16(P(G(x)), P(Wp), P(G(b)), P(G(res)), P(y), M, N, K, flags, None), lib)
    torch.cuda.synchronize()
    assert_fp16_close(y, want, atol=atol, what="linear %s (tiled)" % epi)
    if M <= 128:
        xp = G(pack_act(x))
        y2 = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
        ok(lib.msa_linear_f16(P(xp), P(Wp), P(G(b)), P(G(res)), P(y2), M, N, K,
                              flags | IN_PACKED, None), lib)
        torch.cuda.synchronize()
        assert_fp16_close(y2, want, atol=atol, what="linear %s (stream)" % epi)
        if N % 32 == 0:
            MB = (M + 15) // 16 if M <= 64 else 8
            y3 = torch.zeros(MB * 16 * N, dtype=torch.float16, device=DEV)
            ok(lib.msa_linear_f16(P(xp), P(Wp), P(G(b)), P(G(res)), P(y3), M, N, K,
                                  flags | IN_PACKED | OUT_PACKED, None), lib)
            torch.cuda.synchronize()
            assert torch.equal(unpack_act(y3.cpu(), M, N), y2.cpu())


def test_linear_in_place_residual(lib):
    for M, flags in ((32, IN_PACKED), (200, 0)):
        N, K = 768, 3072
        x, W, b = rnd(M, K, seed=1), rnd(N, K, seed=2, std=0.05), rnd(N, seed=3)
        res = rnd(M, N, seed=4)
        want = _linear_want(x, W, b, res, False)
        y = G(res).clone()
        xin = G(pack_act(x)) if flags else G(x)
        ok(lib.msa_linear_f16(P(xin), P(pack_w(lib, G(W))), P(G(b)), P(y), P(y), M, N, K, flags,
                              None), lib)
        torch.cuda.synchronize()
        assert_fp16_close(y, want.half(), atol=float(want.abs().max()) * 2 ** -10,
                          what="in-place residual")


def test_linear_rejects_bad_shapes(lib):
    x = torch.zeros(64, 64, dtype=torch.float16, device=DEV)
    y = torch.zeros(64, 64, dtype=torch.float16, device=DEV)
    assert lib.msa_linear_f16(P(x), P(x), None, None, P(y), 4, 16, 40, 0, None) == -1   # K % 32
    assert lib.msa_linear_f16(P(x), P(x), None, None, P(y), 4, 8, 32, 0, None) == -1    # N % 16
    assert lib.msa_linear_f16(None, P(x), None, None, P(y), 4, 16, 32, 0, None) == -1
    assert lib.msa_linear_f16(P(x), P(x), None, None, P(y), 4, 16, 32, 64, None) == -1  # flags
    assert lib.msa_linear_f16(P(x), P(x), None, None, P(y), 129, 16, 32, IN_PACKED, None) == -1
    assert lib.msa_linear_partial_f16(P(x), P(x), P(y), 4, 16, 64, 1, 0, None) == -1    # not packed
    assert lib.msa_linear_partial_f16(P(x), P(x), P(y), 4, 16, 64, 3, IN_PACKED, None) == -1


@pytest.mark.parametrize("M,N,K", [(8, 768, 768), (64, 3072, 768), (32, 768, 3072),
                                   (200, 2304, 768), (48, 4096, 4096), (64, 24576, 256),
                                   (40, 73728, 128),
                                   # 9 tiles per workgroup (12 waves as 4 x 3), the last
                                   # workgroup short of tiles and a K range of 1.5 stages
                                   (64, 36864, 256), (50, 36784, 192), (40, 36864, 256),
                                   # 65 .. 128 packed rows
                                   (100, 3072, 768), (128, 36864, 256), (70, 1008, 192),
                                   (1000, 16400, 128), (1124, 16400, 128)])   # large tiled kernel
def test_linear_w8a16(lib, M, N, K):
    print("w8a16", M, N, K, flush=True)
    x, W, b = rnd(M, K, seed=7), rnd(N, K, seed=8, std=0.02), rnd(N, seed=9, std=0.1)
    q, s = O.quantize_int8(W)
    Wd = O.dequantize_int8(q, s)
    want = O.linear(x.float(), Wd.float(), b.float(), r16).half()
    atol = float(want.abs().max()) * 2 ** -10
    qp = pack_w8(lib, G(q))
    y = torch.empty(M, N, dtype=torch.float16, device=DEV)
    ok(lib.msa_linear_w8a16(P(G(x)), P(qp), P(G(s)), P(G(b)), None, P(y), M, N, K, 0, None), lib)
    torch.cuda.synchronize()
    assert_fp16_close(y, want, atol=atol, what="w8a16 (tiled)")
    if M <= 128:
        y2 = torch.empty(M, N, dtype=torch.float16, device=DEV)
        ok(lib.msa_linear_w8a16(P(G(pack_act(x))), P(qp), P(G(s)), P(G(b)), None, P(y2), M, N, K,
                                IN_PACKED, None), lib)
        torch.cuda.synchronize()
        assert_fp16_close(y2, want, atol=atol, what="w8a16 (stream)")


@pytest.mark.parametrize("M,N,K,S", [(32, 768, 768, 1), (32, 768, 3072, 4), (8, 4096, 4096, 4),
                                     (33, 2048, 8192, 8), (64, 768, 3072, 3),
                                     (48, 4608, 2048, 4),
                                     # int8: 18 and 9 tiles per workgroup (12 waves as 2 x 6
                                     # and 4 x 3), the second with a ragged last K slice
                                     (64, 9216, 1024, 8), (64, 9216, 1152, 4),
                                     # 65 .. 128 rows
                                     (70, 4096, 4096, 4), (128, 768, 3072, 4), (100, 2048, 1024, 2)])
@pytest.mark.parametrize("w8", [False, True])
def test_split_k_partials_and_fused_layernorm(lib, M, N, K, S, w8):
    """msa_linear_partial_* followed by msa_residual_layernorm_f16 equals the oracle's
    linear + bias, residual add and LayerNorm."""
    print("splitk", M, N, K, S, w8, flush=True)
    x, W, b = rnd(M, K, seed=7), rnd(N, K, seed=8, std=0.03), rnd(N, seed=9, std=0.1)
    res, g, be = rnd(M, N, seed=10), (1 + rnd(N, seed=11, std=0.1).float()).half(), rnd(N, seed=12)
    if w8:
        q, sc = O.quantize_int8(W)
        Wuse = O.dequantize_int8(q, sc)
    else:
        Wuse = W
    xo = r16(O.linear(x.float(), Wuse.float(), b.float(), r16) + res.float())
    want_h = O.layer_norm(xo, g, be).half()
    part = torch.full((S, M, N), float("nan"), dtype=torch.float32, device=DEV)
    xp = G(pack_act(x))
    if w8:
        ok(lib.msa_linear_partial_w8a16(P(xp), P(pack_w8(lib, G(q))), P(G(sc)), P(part), M, N, K,
                                        S, IN_PACKED, None), lib)
    else:
        ok(lib.msa_linear_partial_f16(P(xp), P(pack_w(lib, G(W))), P(part), M, N, K, S, IN_PACKED,
                                      None), lib)
    xd = G(res).clone()
    MB = (M + 15) // 16 if M <= 64 else 8   # 65 .. 128 rows: always eight row blocks
    hp = torch.zeros(MB * 16 * N, dtype=torch.float16, device=DEV)
    ok(lib.msa_residual_layernorm_f16(P(part), S, P(G(b)), P(xd), P(G(g)), P(G(be)), P(hp), M, N,
                                      1e-5, OUT_PACKED, None), lib)
    torch.cuda.synchronize()
    # the partials are exact fp32 sums of their K range
    tot = part.sum(0).cpu()
    assert (tot - x.float() @ Wuse.float().t()).abs().max() < 1e-3
    atol = float(xo.abs().max()) * 2 ** -10
    assert_fp16_close(xd, xo.half(), atol=atol, what="residual stream")
    got_h = unpack_act(hp.cpu(), M, N)
    # a 1-ulp difference in x moves the normalised value by about one ulp of x / sigma
    assert_fp16_close(got_h, want_h, max_ulp=2, max_frac=2e-2, atol=4 * atol, what="fused LN")
    # without LayerNorm outputs only the residual stream is updated
    xd2 = G(res).clone()
    ok(lib.msa_residual_layernorm_f16(P(part), S, P(G(b)), P(xd2), None, None, None, M, N, 1e-5, 0,
                                      None), lib)
    torch.cuda.synchronize()
    assert torch.equal(xd2, xd)


@pytest.mark.parametrize("M,N,K,S", [(129, 4096, 4096, 4), (200, 1024, 8192, 8),
                                     (256, 4096, 1024, 2), (256, 2064, 512, 4),
                                     (300, 768, 3072, 1), (1, 64, 128, 1), (77, 4096, 2048, 4),
                                     # more slices than 256 x 64 tiles fit at once: 256 x 128
                                     # tiles (a ragged second row tile moved up, a ragged last
                                     # column tile)
                                     (256, 4096, 4096, 8), (300, 2064, 1024, 8),
                                     # the same form below 256 rows and with a ragged last row
                                     # tile: the last row repeated in the loads, rows past it
                                     # dropped
                                     (129, 4096, 16384, 8), (200, 4096, 4096, 8), (1, 4096, 2048, 8),
                                     (513, 4096, 1024, 2)])
def test_split_k_partials_of_row_major_rows(lib, M, N, K, S):
    """msa_linear_partial_f16 without MSA_IN_PACKED (decode batches above 128 rows): slice s of
    the output holds the fp32 sums over K range s and nothing else, for row counts that are not
    multiples of the 256-row tile and an N that is not a multiple of the 64-wide tile; followed
    by msa_residual_layernorm_f16 on row-major rows it equals the oracle's linear + bias,
    residual add and LayerNorm."""
    print("row-major splitk", M, N, K, S, flush=True)
    x, W, b = rnd(M, K, seed=7), rnd(N, K, seed=8, std=0.03), rnd(N, seed=9, std=0.1)
    res, g, be = rnd(M, N, seed=10), (1 + rnd(N, seed=11, std=0.1).float()).half(), rnd(N, seed=12)
    part = torch.full((S + 1, M, N), float("nan"), dtype=torch.float32, device=DEV)
    ok(lib.msa_linear_partial_f16(P(G(x)), P(pack_w(lib, G(W))), P(part), M, N, K, S, 0, None), lib)
    torch.cuda.synchronize()
    assert bool(torch.isnan(part[S]).all()), "wrote past the last slice"
    per = K // S
    for s_ in range(S):
        want = x[:, s_ * per:(s_ + 1) * per].double() @ W[:, s_ * per:(s_ + 1) * per].double().t()
        err = float((part[s_].cpu().double() - want).abs().max())
        assert err < 2e-4, "slice %d off by %.3g" % (s_, err)
    xo = r16(O.linear(x.float(), W.float(), b.float(), r16) + res.float())
    want_h = O.layer_norm(xo, g, be).half()
    xd = G(res).clone()
    h = torch.zeros(M, N, dtype=torch.float16, device=DEV)
    ok(lib.msa_residual_layernorm_f16(P(part), S, P(G(b)), P(xd), P(G(g)), P(G(be)), P(h), M, N,
                                      1e-5, 0, None), lib)
    torch.cuda.synchronize()
    atol = float(xo.abs().max()) * 2 ** -10
    assert_fp16_close(xd, xo.half(), atol=atol, what="residual stream")
    assert_fp16_close(h, want_h, max_ulp=2, max_frac=2e-2, atol=4 * atol, what="fused LN")


def test_split_k_of_row_major_rows_rejects_and_suggestion(lib):
    x = torch.zeros(256, 4096, dtype=torch.float16, device=DEV)
    part = torch.zeros(8 * 256 * 64, dtype=torch.float32, device=DEV)
    f = lib.msa_linear_partial_f16
    assert f(P(x), P(x), P(part), 256, 64, 4096, 3, 0, None) == -1    # 4096 / 3 is no whole range
    assert f(P(x), P(x), P(part), 256, 64, 256, 4, 0, None) == -1     # ranges of one stage
    assert lib.msa_linear_partial_w8a16(P(x), P(x), P(x), P(part), 256, 64, 4096, 4, 0, None) == -1
    # a few hundred rows against d_model output features: split; enough tiles already: not
    assert lib.msa_linear_default_splits_rows(256, 4096, 16384) == 8   # over 256 x 128 tiles
    assert lib.msa_linear_default_splits_rows(200, 4096, 16384) == 8   # the same below 256 rows
    assert lib.msa_linear_default_splits_rows(100, 4096, 16384) == 4   # up to 128: 256 x 64 tiles
    assert lib.msa_linear_default_splits_rows(200, 4096, 4096) == 4
    assert lib.msa_linear_default_splits_rows(512, 4096, 4096) == 2
    assert lib.msa_linear_default_splits_rows(256, 16384, 4096) == 1
    assert lib.msa_linear_default_splits_rows(4096, 4096, 4096) == 1


def test_default_splits_are_valid(lib):
    for M, N, K in [(32, 4096, 4096), (32, 4096, 16384), (32, 12288, 4096), (1, 768, 768),
                    (8, 2048, 8192), (64, 9216, 36864), (200, 4096, 4096)]:
        S = lib.msa_linear_default_splits(M, N, K)
        assert 1 <= S <= 8 and K // 64 >= S, (M, N, K, S)
    assert lib.msa_linear_default_splits(32, 4096, 16384) > 1


@pytest.mark.parametrize("B,T,H,hd,S0", [(3, 1, 2, 64, 5), (2, 7, 4, 128, 0), (32, 1, 12, 64, 40),
                                         (2, 70, 2, 64, 0), (64, 1, 4, 128, 3),
                                         (100, 1, 4, 64, 9), (128, 1, 2, 128, 0)])
@pytest.mark.parametrize("w8", [False, True])
def test_qkv_proj_scatter(lib, B, T, H, hd, S0, w8):
    print("qkv", B, T, H, hd, S0, w8, flush=True)
    D = H * hd
    S_cap = S0 + T + 3
    x, W, b = rnd(B * T, D, seed=1), rnd(3 * D, D, seed=2, std=0.05), rnd(3 * D, seed=3, std=0.1)
    if w8:
        qw, sc = O.quantize_int8(W)
        Wuse = O.dequantize_int8(qw, sc)
    else:
        Wuse = W
    kvq = O.linear(x.float(), Wuse.float(), b.float(), r16)
    k, v, q = kvq.split(D, dim=-1)
    q = r16(q * (hd ** -0.5))
    want_k = k.view(B, T, H, hd).permute(0, 2, 1, 3)
    want_v = v.view(B, T, H, hd).permute(0, 2, 1, 3)
    atol = float(kvq.abs().max()) * 2 ** -10
    modes = [0] + ([IN_PACKED] if B * T <= 128 else [])
    for flags in modes:
        Kc = torch.zeros(B, H, S_cap, hd, dtype=torch.float16, device=DEV)
        Vc = torch.zeros_like(Kc)
        qo = torch.empty(B * T, D, dtype=torch.float16, device=DEV)
        xin = G(pack_act(x)) if flags else G(x)
        if w8:
            ok(lib.msa_qkv_proj_w8a16(P(xin), P(pack_w8(lib, G(qw))), P(G(sc)), P(G(b)), P(qo),
                                      P(Kc), P(Vc), B, T, H, hd, S0, S_cap, D, flags, None, None), lib)
        else:
            ok(lib.msa_qkv_proj_f16(P(xin), P(pack_w(lib, G(W))), P(G(b)), P(qo), P(Kc), P(Vc), B,
                                    T, H, hd, S0, S_cap, D, flags, None, None), lib)
        torch.cuda.synchronize()
        assert_fp16_close(qo, q.half(), atol=atol, what="q")
        assert_fp16_close(Kc[:, :, S0:S0 + T], want_k.half(), atol=atol, what="K cache")
        assert_fp16_close(Vc[:, :, S0:S0 + T], want_v.half(), atol=atol, what="V cache")
        # nothing outside the appended slice was touched
        assert float(Kc[:, :, :S0].abs().sum()) == 0 and float(Kc[:, :, S0 + T:].abs().sum()) == 0


@pytest.mark.parametrize("w8", [False, True])
def test_qkv_proj_scatter_large_tiled_kernel(lib, w8):
    """A prefill-sized QKV projection (enough 256 x 256 tiles for the large tiled kernel): the
    scatter into the cache and the q scaling, with an input width independent of H * hd."""
    B, T, H, hd, S0, K = 2, 1057, 20, 128, 3, 256   # 2114 rows = 8 * 256 + 66
    D, S_cap = H * hd, S0 + T + 2
    x, W, b = rnd(B * T, K, seed=1), rnd(3 * D, K, seed=2, std=0.05), rnd(3 * D, seed=3, std=0.1)
    if w8:
        qw, sc = O.quantize_int8(W)
        Wuse = O.dequantize_int8(qw, sc)
    else:
        Wuse = W
    kvq = O.linear(x.float(), Wuse.float(), b.float(), r16)
    k, v, q = kvq.split(D, dim=-1)
    q = r16(q * (hd ** -0.5))
    atol = float(kvq.abs().max()) * 2 ** -10
    Kc = torch.zeros(B, H, S_cap, hd, dtype=torch.float16, device=DEV)
    Vc = torch.zeros_like(Kc)
    qo = torch.empty(B * T, D, dtype=torch.float16, device=DEV)
    if w8:
        ok(lib.msa_qkv_proj_w8a16(P(G(x)), P(pack_w8(lib, G(qw))), P(G(sc)), P(G(b)), P(qo), P(Kc),
                                  P(Vc), B, T, H, hd, S0, S_cap, K, 0, None, None), lib)
    else:
        ok(lib.msa_qkv_proj_f16(P(G(x)), P(pack_w(lib, G(W))), P(G(b)), P(qo), P(Kc), P(Vc), B, T,
                                H, hd, S0, S_cap, K, 0, None, None), lib)
    torch.cuda.synchronize()
    assert_fp16_close(qo, q.half(), atol=atol, what="q")
    assert_fp16_close(Kc[:, :, S0:S0 + T], k.view(B, T, H, hd).permute(0, 2, 1, 3).half(),
                      atol=atol, what="K cache")
    assert_fp16_close(Vc[:, :, S0:S0 + T], v.view(B, T, H, hd).permute(0, 2, 1, 3).half(),
                      atol=atol, what="V cache")
    assert float(Kc[:, :, :S0].abs().sum()) == 0 and float(Kc[:, :, S0 + T:].abs().sum()) == 0


@pytest.mark.parametrize("N,K", [(16, 64), (48, 192), (1008, 4096)])
def test_expand_weight_w8_f16(lib, N, K):
    """Packed int8 + scales -> packed fp16: bit for bit the packed form of the dequantised matrix
    round(q * scale), including the extreme bytes and a zero scale."""
    g = torch.Generator().manual_seed(5)
    q = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    q[0, :4] = torch.tensor([-128, -127, 127, 0], dtype=torch.int8)
    sc = (torch.rand(N, generator=g) * 0.02 + 1e-4).half()
    sc[N - 1] = 0
    want = pack_w(lib, G(O.dequantize_int8(q, sc).half()))
    got = torch.full((N, K), float("nan"), dtype=torch.float16, device=DEV)
    ok(lib.msa_expand_weight_w8_f16(P(pack_w8(lib, G(q))), P(G(sc)), P(got), N, K, None), lib)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert lib.msa_expand_weight_w8_f16(P(got), P(G(sc)), P(got), N, K, None) == -1
    assert lib.msa_expand_weight_w8_f16(P(G(q)), P(G(sc)), P(got), N, 96, None) == -1


@pytest.mark.parametrize("B", [300, 130])
def test_qkv_proj_wide_decode_batch_with_row_lengths(lib, B):
    """300 (130) rows of one new position each (T = 1) with per-row cache lengths on the device,
    one row inactive: a row-major product for the four-wave tiled kernel (more and fewer rows than
    one of its tiles), whose QKV epilogue must append every row at its own length and leave the
    inactive row's cache alone."""
    H, hd, K, S_cap = 16, 128, 256, 40
    D = H * hd
    x, W, b = rnd(B, K, seed=1), rnd(3 * D, K, seed=2, std=0.05), rnd(3 * D, seed=3, std=0.1)
    g = torch.Generator().manual_seed(4)
    lens = torch.randint(0, S_cap, (B,), generator=g, dtype=torch.int32)
    lens[7] = -1
    kvq = O.linear(x.float(), W.float(), b.float(), r16)
    k, v, q = kvq.split(D, dim=-1)
    q = r16(q * (hd ** -0.5))
    atol = float(kvq.abs().max()) * 2 ** -10
    Kc = torch.zeros(B, H, S_cap, hd, dtype=torch.float16, device=DEV)
    Vc = torch.zeros_like(Kc)
    qo = torch.empty(B, D, dtype=torch.float16, device=DEV)
    ok(lib.msa_qkv_proj_f16(P(G(x)), P(pack_w(lib, G(W))), P(G(b)), P(qo), P(Kc), P(Vc), B, 1, H,
                            hd, 0, S_cap, K, 0, P(G(lens)), None), lib)
    torch.cuda.synchronize()
    assert_fp16_close(qo, q.half(), atol=atol, what="q")
    Kh, Vh = Kc.cpu(), Vc.cpu()
    wantK, wantV = torch.zeros_like(Kh), torch.zeros_like(Vh)
    for r in range(B):
        if lens[r] >= 0:
            wantK[r, :, lens[r]] = k[r].view(H, hd).half()
            wantV[r, :, lens[r]] = v[r].view(H, hd).half()
    assert_fp16_close(Kh, wantK, atol=atol, what="K cache")
    assert_fp16_close(Vh, wantV, atol=atol, what="V cache")
    assert float(Kh[7].abs().sum()) == 0 and float(Vh[7].abs().sum()) == 0


def test_qkv_proj_capacity_error(lib):
    x = torch.zeros(2, 128, dtype=torch.float16, device=DEV)
    rc = lib.msa_qkv_proj_f16(P(x), P(x), P(x), P(x), P(x), P(x), 2, 1, 2, 64, 10, 10, 128, 0,
                              None, None)
    assert rc == -2 and b"capacity" in lib.msa_last_error()


def _oracle_core(dtype=torch.float16):
    cfg = O.OracleConfig(1, 64, 1, 64, 8)
    return O.OracleDecoder(cfg, {}, dtype=dtype)


@pytest.mark.parametrize("B,H,hd,T,S0,masked", [
    (2, 2, 64, 1, 0, False), (3, 2, 64, 1, 37, False), (2, 3, 128, 1, 300, True),
    (32, 12, 64, 1, 65, False), (2, 2, 128, 9, 0, False), (2, 2, 64, 33, 0, True),
    (100, 3, 64, 1, 40, True), (128, 2, 128, 1, 17, False),     # 65 .. 128 rows, packed output
    (1, 4, 128, 130, 0, False), (8, 32, 64, 1, 513, False), (2, 2, 64, 5, 11, False),
    (2, 3, 128, 257, 0, True), (1, 2, 64, 200, 56, False), (3, 1, 128, 129, 127, True),
    # query tiles are aligned to the end: exact multiples, one query over, one query short
    (1, 2, 128, 128, 0, False), (1, 1, 128, 1025, 0, False), (2, 1, 64, 127, 3, True),
    (1, 2, 64, 384, 130, False),
    # enough K and V rows (> 64 MiB) for the XCD-grouped order of the query tiles, with a number of
    # (row, head) pairs that is no multiple of 8
    (2, 33, 128, 1990, 10, True),
])
def test_attention(lib, B, H, hd, T, S0, masked):
    print("attention", B, H, hd, T, S0, masked, flush=True)
    D, S = H * hd, S0 + T
    S_cap = S + 5
    q = rnd(B * T, D, seed=1, std=0.3)
    Kc = rnd(B, H, S_cap, hd, seed=2)
    Vc = rnd(B, H, S_cap, hd, seed=3)
    mask = None
    if masked:
        mask = torch.zeros(B, S, dtype=torch.bool)
        mask[0, 1:3] = True
        mask[B - 1, S // 2] = True
    core = _oracle_core()
    qq = q.float().view(B, T, H, hd).permute(0, 2, 1, 3).reshape(B * H, T, hd)
    kk = Kc[:, :, :S].float().reshape(B * H, S, hd)
    vv = Vc[:, :, :S].float().reshape(B * H, S, hd)
    causal = torch.full((T, S), float("-inf")).triu(S0 + 1)  # query t sees keys 0..S0+t
    want = core.attention_core(qq, kk, vv, B, causal, mask)
    want = want.view(B, H, T, hd).permute(0, 2, 1, 3).reshape(B * T, D)
    out = torch.empty(B * T, D, dtype=torch.float16, device=DEV)
    dm = None if mask is None else mask.to(torch.uint8).to(DEV)
    ok(lib.msa_attention_f16(P(G(q)), P(G(Kc)), P(G(Vc)), P(dm),
                             0 if dm is None else dm.stride(0), P(out), B, H, hd, T, S0, S_cap,
                             0, None, None), lib)
    torch.cuda.synchronize()
    if T == 1 and B <= 128:
        MB = (B + 15) // 16 if B <= 64 else 8
        op = torch.zeros(MB * 16 * D, dtype=torch.float16, device=DEV)
        ok(lib.msa_attention_f16(P(G(q)), P(G(Kc)), P(G(Vc)), P(dm),
                                 0 if dm is None else dm.stride(0), P(op), B, H, hd, T, S0, S_cap,
                                 OUT_PACKED, None, None), lib)
        torch.cuda.synchronize()
        assert torch.equal(unpack_act(op.cpu(), B, D), out.cpu())
    # scores and probabilities are intermediate fp16 roundings.  A 1-ulp flip of a score of
    # magnitude up to 16 (these inputs reach |s| ~ 15) scales its probability by e^(2^-7), so a
    # few outputs may move by 2^-7 of the largest output; everything else is within 1 ulp.
    assert_fp16_close(out, want.half(), max_frac=2e-2, atol=float(want.abs().max()) * 2 ** -7,
                      what="attention")


@pytest.mark.parametrize("B,H,hd,S0,mode", [
    (1, 12, 64, 1100, "plain"), (1, 12, 64, 37, "plain"), (2, 5, 128, 700, "mask"),
    (3, 7, 128, 2049, "lens"), (2, 9, 64, 1500, "lens"), (1, 32, 128, 4, "plain"),
    (1, 3, 128, 8191, "plain")])
def test_split_attention_gives_the_bits_of_the_one_launch_form(lib, B, H, hd, S0, mode):
    """msa_attention_split_f16 (scores of 8 key ranges, then one workgroup per 32-column slice)
    forms every sum in the order of msa_attention_f16 at B*H < 512: the outputs are equal bit for
    bit, row-major and packed, with a padding mask, with per-row lengths and an inactive row, for
    histories shorter than one round of loads and at the 8192-key limit."""
    print("split attention", B, H, hd, S0, mode, flush=True)
    D = H * hd
    S_cap = S0 + 1 + (0 if S0 + 1 == 8192 else 3)
    q = G(rnd(B, D, seed=1, std=0.3))
    Kc, Vc = G(rnd(B, H, S_cap, hd, seed=2)), G(rnd(B, H, S_cap, hd, seed=3))
    dm, stride, ln = None, 0, None
    if mode == "mask":
        m = torch.zeros(B, S0 + 1, dtype=torch.uint8)
        m[0, 1:40] = 1
        m[B - 1, S0 // 2] = 1
        dm, stride = m.to(DEV), S0 + 1
    if mode == "lens":
        lens = [S0, S0 // 3, -1][:B] if B >= 3 else [S0 // 2, S0]
        ln = torch.tensor(lens, dtype=torch.int32, device=DEV)
        for b, n in enumerate(lens):  # nothing past a row's own length may be read
            Kc[b, :, max(n, -1) + 1:] = float("nan")
            Vc[b, :, max(n, -1) + 1:] = float("nan")
    ws = torch.empty(lib.msa_attention_split_workspace_bytes(B, H, S_cap), dtype=torch.uint8,
                     device=DEV)
    MB = (B + 15) // 16
    for flags in (0, OUT_PACKED):
        n_out = MB * 16 * D if flags else B * D
        one = torch.full((n_out,), 7.0, dtype=torch.float16, device=DEV)
        two = torch.full((n_out,), 7.0, dtype=torch.float16, device=DEV)
        ok(lib.msa_attention_f16(P(q), P(Kc), P(Vc), P(dm), stride, P(one), B, H, hd, 1, S0, S_cap,
                                 flags, P(ln), None), lib)
        ok(lib.msa_attention_split_f16(P(q), P(Kc), P(Vc), P(dm), stride, P(two), P(ws), B, H, hd,
                                       S0, S_cap, flags, P(ln), None), lib)
        torch.cuda.synchronize()
        assert torch.equal(one.view(torch.int16), two.view(torch.int16)), (
            "split attention differs in %d of %d values"
            % (int((one.view(torch.int16) != two.view(torch.int16)).sum()), n_out))
        live = one.float()
        assert bool(torch.isfinite(live).all())


def test_split_attention_rejects_and_preference(lib):
    x = torch.zeros(64, 128, dtype=torch.float16, device=DEV)
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    bad = lib.msa_attention_split_f16
    assert bad(P(x), P(x), P(x), None, 0, P(x), None, 1, 1, 64, 0, 4, 0, None, None) == -1
    assert bad(P(x), P(x), P(x), None, 0, P(x), P(ws), 1, 1, 96, 0, 4, 0, None, None) == -1
    assert bad(P(x), P(x), P(x), None, 0, P(x), P(ws), 1, 1, 64, 4, 4, 0, None, None) == -2
    assert lib.msa_attention_split_workspace_bytes(2, 3, 100) == 2 * 3 * 100 * 4
    # very few pairs over a very long history: yes; a batch or OPT's 2048 positions: no
    assert lib.msa_attention_prefers_split(1, 32, 128, 4097) == 1
    assert lib.msa_attention_prefers_split(4, 32, 128, 8000) == 0
    assert lib.msa_attention_prefers_split(1, 32, 128, 2049) == 0


def test_attention_rejects(lib):
    x = torch.zeros(64, 96, dtype=torch.float16, device=DEV)
    assert lib.msa_attention_f16(P(x), P(x), P(x), None, 0, P(x), 1, 1, 96, 1, 0, 4, 0, None, None) == -1
    assert lib.msa_attention_f16(P(x), P(x), P(x), None, 0, P(x), 1, 1, 64, 1, 4, 4, 0, None, None) == -2


def _select(lib, logits, temperature=1.0, banned=(), stop=(), finished=None, force=0, eos=2):
    B, V = logits.shape
    tok = torch.zeros(B, 3, dtype=torch.long, device=DEV)
    sc = torch.zeros(B, 3, dtype=torch.float32, device=DEV)
    ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
    sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
    ok(lib.msa_greedy_select_f16(P(logits), logits.stride(0), B, V, temperature, ba, len(banned),
                                 sa, len(stop), P(finished), None, force, eos, P(tok[:, 1]), 3,
                                 P(sc[:, 1]), 3, None, None), lib)
    torch.cuda.synchronize()
    assert float(tok[:, 0].abs().sum()) == 0 and float(tok[:, 2].abs().sum()) == 0
    return tok[:, 1].cpu(), sc[:, 1].cpu()


@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_greedy_select_matches_reference_passes(lib, temperature):
    B, V = 5, 50272
    logits = rnd(B, V, seed=3, std=1.3)
    logits[1, 777] = logits[1].max() + 1       # clear winner
    logits[2, 1] = 30.0                        # pad would win: must never be selected
    logits[3, 100] = logits[3, 4000] = 20.0    # exact tie -> lowest index
    logits[4, 2] = 25.0                        # eos wins but is banned below
    lp = torch.log_softmax(logits.float() / temperature, -1)
    lp[:, 1] = float("-inf")
    lp[:, 2] = float("-inf")
    want_s, want_t = lp.max(-1)
    tok, sc = _select(lib, logits.to(DEV), temperature, banned=[1, 2])
    assert torch.equal(tok, want_t)
    assert torch.allclose(sc, want_s, atol=2e-5)
    assert tok[3] == 100


def test_greedy_select_finished_force_stop_nan(lib):
    B, V = 4, 1000
    logits = rnd(B, V, seed=5)
    logits[3, 5] = float("nan")
    fin = torch.tensor([1, 0, 0, 0], dtype=torch.uint8, device=DEV)
    logits[1, 77] = 50.0   # row 1 picks the stop token 77
    tok, sc = _select(lib, logits.to(DEV), banned=[1], stop=[77], finished=fin)
    lp = torch.log_softmax(logits.float(), -1)
    assert tok[0] == 2 and abs(float(sc[0]) - float(lp[0, 2])) < 2e-5   # finished row: eos only
    assert tok[1] == 77
    assert tok[3] == 0 and sc[3] == float("-inf")                         # NaN row: all -inf
    assert fin.cpu().tolist() == [1, 1, 0, 0]
    tok, sc = _select(lib, logits.to(DEV), banned=[1], force=1)
    assert tok[:3].tolist() == [2, 2, 2]


def test_target_logprob(lib):
    R, V = 37, 50272
    logits = rnd(R, V, seed=9, std=1.2)
    tgt = torch.randint(0, V, (R,), generator=torch.Generator().manual_seed(1))
    want = torch.log_softmax(logits.float(), -1).gather(1, tgt[:, None])[:, 0]
    out = torch.empty(R, dtype=torch.float32, device=DEV)
    d = logits.to(DEV)
    ok(lib.msa_target_logprob_f16(P(d), d.stride(0), R, V, 1.0, P(G(tgt)), P(out), None), lib)
    torch.cuda.synchronize()
    assert torch.allclose(out.cpu(), want, atol=2e-5)


@pytest.mark.parametrize("M,V,K", [(1, 96, 64), (17, 2048, 256), (32, 50272, 768), (64, 4000, 128),
                                   (48, 50272, 256)])
def test_lm_head_fused_selection_matches_projection_then_select(lib, M, V, K):
    """msa_lm_head_greedy_select_f16 against msa_linear_f16 followed by msa_greedy_select_f16
    (itself checked against the reference's passes above).  The stand-alone selection runs on
    the logits the fused call stored: identical tokens and finished flags, scores equal up to the
    fp32 summation order of the log-sum-exp.  The stored logits equal msa_linear_f16's up to the
    fp32 summation order over K (above 32 rows the two run different kernels)."""
    print("lm-head select", M, V, K, flush=True)
    x, E = rnd(M, K, seed=3, std=1.0), rnd(V, K, seed=4, std=0.3)
    Ep = pack_w(lib, G(E))
    xp = G(pack_act(x))
    logits = torch.empty(M, V, dtype=torch.float16, device=DEV)
    ok(lib.msa_linear_f16(P(xp), P(Ep), None, None, P(logits), M, V, K, IN_PACKED, None), lib)
    ws = torch.empty(lib.msa_lm_head_select_workspace_bytes(M), dtype=torch.uint8, device=DEV)
    top = logits.float().argmax(-1)
    cases = [
        dict(),                                                     # plain
        dict(temperature=0.7, banned=(1, 2)),                       # min-length regime
        dict(banned=tuple({1, int(top[0]), int(top[-1])}), stop=(int(logits[0].float().topk(2).indices[1]),)),
        dict(banned=(1,), force=1),                                 # last step: only eos
        dict(banned=(1,), finished=[i % 3 == 0 for i in range(M)]),
    ]
    for c in cases:
        banned, stop = list(c.get("banned", ())), list(c.get("stop", ()))
        temp, force = c.get("temperature", 1.0), c.get("force", 0)
        ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
        sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
        outs = []
        fused_logits = None
        for fused in (True, False):
            fin = None
            if "finished" in c:
                fin = torch.tensor(c["finished"], dtype=torch.uint8, device=DEV)
            elif stop:
                fin = torch.zeros(M, dtype=torch.uint8, device=DEV)
            tok = torch.full((M, 3), -7, dtype=torch.long, device=DEV)
            sc = torch.full((M, 3), 9.0, dtype=torch.float32, device=DEV)
            lg = torch.zeros(M, V, dtype=torch.float16, device=DEV)
            if fused:
                ok(lib.msa_lm_head_greedy_select_f16(
                    P(xp), P(Ep), P(lg), P(ws), M, V, K, temp, ba, len(banned), sa, len(stop),
                    P(fin), None, force, 2, P(tok[:, 1]), 3, P(sc[:, 1]), 3, None, None), lib)
                fused_logits = lg
            else:
                ok(lib.msa_greedy_select_f16(P(fused_logits), V, M, V, temp, ba, len(banned), sa,
                                             len(stop), P(fin), None, force, 2, P(tok[:, 1]), 3,
                                             P(sc[:, 1]), 3, None, None), lib)
            torch.cuda.synchronize()
            outs.append((tok.cpu(), sc.cpu(), None if fin is None else fin.cpu()))
        (t0, s0, f0), (t1, s1, f1) = outs
        assert torch.equal(t0, t1), c
        assert torch.allclose(s0, s1, atol=2e-5, rtol=1e-6), (c, (s0 - s1).abs().max())
        assert (f0 is None and f1 is None) or torch.equal(f0, f1), c
        if M <= 32:
            assert torch.equal(fused_logits, logits), c
        else:
            assert_fp16_close(fused_logits, logits.cpu(),
                              atol=float(logits.float().abs().max()) * 2 ** -10, what="logits")
    # logits are optional, the column may come from the device, and a NaN row yields (0, -inf)
    ln = torch.tensor([2], dtype=torch.int32, device=DEV)
    tok = torch.full((M, 3), -7, dtype=torch.long, device=DEV)
    sc = torch.zeros(M, 3, dtype=torch.float32, device=DEV)
    ba = (ctypes.c_int32 * 1)(1)
    ok(lib.msa_lm_head_greedy_select_f16(P(xp), P(Ep), None, P(ws), M, V, K, 1.0, ba, 1, ba, 0,
                                         None, None, 0, 2, P(tok), 3, P(sc), 3, P(ln), None), lib)
    xn = x.clone()
    xn[0, 0] = float("nan")
    tok2 = torch.full((M, 1), -7, dtype=torch.long, device=DEV)
    sc2 = torch.zeros(M, 1, dtype=torch.float32, device=DEV)
    ok(lib.msa_lm_head_greedy_select_f16(P(G(pack_act(xn))), P(Ep), None, P(ws), M, V, K, 1.0, ba,
                                         1, ba, 0, None, None, 0, 2, P(tok2), 1, P(sc2), 1, None,
                                         None), lib)
    torch.cuda.synchronize()
    lg = logits.float().clone()
    lg[:, 1] = float("-inf")
    assert torch.equal(tok[:, 2].cpu(), lg.argmax(-1).cpu()) and int((tok[:, :2] != -7).sum()) == 0
    assert int(tok2[0]) == 0 and float(sc2[0]) == float("-inf")
    if M > 1:
        assert torch.equal(tok2[1:, 0].cpu(), lg[1:].argmax(-1).cpu())
    # argument checks
    assert lib.msa_lm_head_greedy_select_f16(P(xp), P(Ep), None, None, M, V, K, 1.0, ba, 1, ba, 0,
                                             None, None, 0, 2, P(tok), 3, P(sc), 3, None,
                                             None) == -1
    assert lib.msa_lm_head_greedy_select_f16(P(xp), P(Ep), None, P(ws), 65, V, K, 1.0, ba, 1, ba,
                                             0, None, None, 0, 2, P(tok), 3, P(sc), 3, None,
                                             None) == -1


def test_stream_read_probe_runs_and_validates(lib):
    """The measurement aid reads a buffer once; bad sizes and addresses are rejected."""
    buf = torch.zeros(1 << 29, dtype=torch.float16, device=DEV)  # 1 GiB
    ok(lib.msa_probe_stream_read(P(buf), buf.numel() * 2, None), lib)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    ok(lib.msa_probe_stream_read(P(buf), buf.numel() * 2, None), lib)
    e1.record()
    torch.cuda.synchronize()
    rate = buf.numel() * 2 / (e0.elapsed_time(e1) * 1e-3)
    assert 1e12 < rate < 8.5e12, rate  # it really reads the buffer: bounded by the memory system
    assert lib.msa_probe_stream_read(P(buf), 24, None) == -1
    assert lib.msa_probe_stream_read(ctypes.c_void_p(buf.data_ptr() + 2), 32, None) == -1
    assert lib.msa_probe_stream_read(None, 32, None) == -1


# ---- nucleus sampling kernel ------------------------------------------------------------------
def _sample(lib, logits, *, temperature=1.0, banned=(1,), stop=(), finished=None, row_mode=None,
            force=0, eos=2, topp_rows=None, topp_all=0.0, noise=None, counts=None,
            counts_src=None, alphas=(0.0, 0.0, 0.0, 0.0), temperature_rows=None, lprobs=None,
            penalty_rows=None):
    B, V = logits.shape
    ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
    sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
    tok = torch.full((B,), -7, dtype=torch.long, device=DEV)
    sc = torch.zeros(B, dtype=torch.float32, device=DEV)
    ok(lib.msa_sample_topp_f16(P(logits), logits.stride(0), B, V, temperature, P(temperature_rows),
                               ba, len(banned), sa, len(stop), P(finished), P(row_mode), force,
                               eos, P(topp_rows), topp_all, P(noise), P(counts), P(counts_src),
                               alphas[0], alphas[1], alphas[2], alphas[3], P(penalty_rows),
                               P(lprobs),
                               0 if lprobs is None else lprobs.stride(0), P(tok), 1, P(sc), 1,
                               None), lib)
    torch.cuda.synchronize()
    return tok.cpu(), sc.cpu()


def _reference_lprobs(logits, temperature, banned, early, only_eos, eos, counts, counts_src,
                      alphas):
    """The masked, penalised fp32 log-probabilities of the reference's loop
    (sequence_generator.py:272-293, 478-523), in its order."""
    z = logits.float().cpu()
    if temperature != 1.0:
        z = z / temperature
    lp = torch.log_softmax(z, -1)
    for r in range(lp.shape[0]):
        lp[r, list(banned) + (list(early[r]) if early else [])] = float("-inf")
    lp = O.apply_repetition_penalties(lp, counts, counts_src, *alphas)
    for r in range(lp.shape[0]):
        if only_eos[r]:
            keep = lp[r, eos].clone()
            lp[r] = float("-inf")
            lp[r, eos] = keep
    return lp


@pytest.mark.parametrize("V,B", [(50272, 8), (4001, 5), (96, 16)])
def test_nucleus_sampling_kernel_matches_oracle_given_the_same_noise(lib, V, B):
    """Masks, per-row regimes, both repetition penalties, temperature, one top-p per row: the
    kernel's token must be the oracle's (arg-max of truncated probability / noise over the same
    nucleus), its score the log-probability among the eligible ids, and the generated-token
    counts go up by one."""
    print("sample_topp", V, B, flush=True)
    g = torch.Generator().manual_seed(V)
    logits = (torch.randn(B, V, generator=g) * 2.0).half()
    counts = torch.randint(0, 3, (B, V), generator=g)
    counts_src = torch.randint(0, 2, (B, V), generator=g)
    alphas = (0.7, 0.2, 0.4, 0.1)
    eos, stop = 2, [7, 11]
    modes = torch.tensor([(i % 4) for i in range(B)], dtype=torch.uint8)   # 0, early, only, both
    fin = torch.tensor([i == 5 for i in range(B)], dtype=torch.uint8)
    topp = torch.tensor([0.05 + 0.9 * i / max(1, B - 1) for i in range(B)])
    noise = torch.empty(B, V).exponential_(generator=g)
    early = [[eos] + stop if int(m) & 1 else [] for m in modes]
    only = [bool(int(m) & 2) or bool(f) for m, f in zip(modes, fin)]
    lp = _reference_lprobs(logits, 0.8, [1], early, only, eos, counts, counts_src, alphas)
    want_sc, want_tok, _, _ = O.sample_topp(lp, topp.unsqueeze(1), noise=noise)
    cd = G(counts.clone())
    # the step's distribution goes into rows of a wider buffer, as into all_lprobs[:, step]
    stored = torch.full((B, 2, V + 3), 7.0, dtype=torch.float32, device=DEV)
    tok, sc = _sample(lib, G(logits), temperature=0.8, banned=[1], stop=stop, finished=G(fin.clone()),
                      row_mode=G(modes), eos=eos, topp_rows=G(topp), noise=G(noise), counts=cd,
                      counts_src=G(counts_src), alphas=alphas, lprobs=stored[:, 1])
    dead = ~torch.isfinite(lp).any(-1)      # eos banned and alone eligible: (0, -inf)
    assert bool(dead[3]) and int(tok[3]) == 0 and float(sc[3]) == float("-inf")
    live = ~dead
    assert torch.equal(tok[live], want_tok[live]), (tok, want_tok)
    assert torch.allclose(sc[live], want_sc[live], atol=2e-5)
    bumped = counts.clone()
    bumped[torch.arange(B), tok] += 1
    assert torch.equal(cd.cpu(), bumped)
    # the stored rows are the reference's masked, penalised log-probabilities (-inf where they
    # are), and nothing around them was touched
    got_lp = stored[:, 1, :V].cpu()
    assert torch.equal(torch.isinf(got_lp), torch.isinf(lp))
    fin_ = torch.isfinite(lp)
    assert torch.allclose(got_lp[fin_], lp[fin_], atol=1e-5, rtol=1e-6)
    assert bool((stored[:, 0] == 7.0).all()) and bool((stored[:, 1, V:] == 7.0).all())


def test_sampling_kernel_per_row_temperature_and_skipped_rows(lib):
    """Rows of one call at their own temperature and top-p equal the same rows run one call
    each; a row marked MSA_ROW_SKIP keeps whatever its outputs held; top-p 0 or temperature 0 for
    a row makes that row greedy."""
    B, V = 6, 4001
    g = torch.Generator().manual_seed(11)
    logits = (torch.randn(B, V, generator=g) * 2.0).half()
    noise = torch.empty(B, V).exponential_(generator=g)
    temps = torch.tensor([1.0, 0.7, 1.3, 0.0, 0.5, 0.9])
    topp = torch.tensor([0.9, 0.5, 1.0, 0.8, 0.0, 0.3])
    modes = torch.tensor([0, 0, 4, 0, 0, 1], dtype=torch.uint8)          # row 2 is skipped
    ld, nd = G(logits), G(noise)
    ba = (ctypes.c_int32 * 1)(1)
    sa = (ctypes.c_int32 * 1)(9)
    tok = torch.full((B,), -7, dtype=torch.long, device=DEV)
    sc = torch.full((B,), 5.0, dtype=torch.float32, device=DEV)
    ok(lib.msa_sample_topp_f16(P(ld), V, B, V, 1.0, P(G(temps)), ba, 1, sa, 1, None, P(G(modes)),
                               0, 2, P(G(topp)), 0.0, P(nd), None, None, 0.0, 0.0, 0.0, 0.0, None,
                               None, 0, P(tok), 1, P(sc), 1, None), lib)
    torch.cuda.synchronize()
    assert int(tok[2]) == -7 and float(sc[2]) == 5.0
    for r in (0, 1, 3, 4, 5):
        t, p_ = float(temps[r]), float(topp[r])
        greedy = t == 0.0 or p_ == 0.0
        one_tok, one_sc = _sample(lib, ld[r:r + 1], temperature=t, banned=[1], stop=[9],
                                  row_mode=G(modes[r:r + 1]), topp_all=0.0 if greedy else p_,
                                  noise=None if greedy else nd[r:r + 1])
        assert int(tok[r]) == int(one_tok[0]) and float(sc[r]) == float(one_sc[0]), r
        if greedy:
            z = logits[r].float() / (t if t > 0 else 1.0)
            lp = torch.log_softmax(z, -1)
            lp[1] = float("-inf")
            assert int(tok[r]) == int(lp.argmax()) and abs(float(sc[r]) - float(lp.max())) < 2e-5


def test_log_softmax_rows_into_a_strided_buffer(lib):
    """msa_log_softmax_f16 against torch's fp32 log_softmax: rows (b, t), t < T - 1, of logits
    [B, T, V] land at out[b, t + 1], as the generator stores the prompt's distributions."""
    B, T, V, L = 3, 5, 4001, 9
    g = torch.Generator().manual_seed(5)
    logits = (torch.randn(B, T, V, generator=g) * 3.0).half()
    out = torch.full((B, L, V), 7.0, dtype=torch.float32, device=DEV)
    ld = G(logits)
    for temperature in (1.0, 0.6):
        ok(lib.msa_log_softmax_f16(P(ld), T * V, V, B, T - 1, V, temperature, P(out[:, 1]), L * V, V,
                                   None), lib)
        torch.cuda.synchronize()
        want = torch.log_softmax(logits.float() / temperature, -1)[:, :-1]
        assert torch.allclose(out[:, 1:T].cpu(), want, atol=2e-5, rtol=1e-6)
        assert bool((out[:, 0] == 7.0).all()) and bool((out[:, T:] == 7.0).all())
    assert lib.msa_log_softmax_f16(P(ld), T * V, V - 1, B, T, V, 1.0, P(out), L * V, V, None) == -1


def test_nucleus_sampling_kernel_closed_forms(lib):
    """Hand-made distributions.  (i) p = 1/2, 1/4, 1/8, ...: with top-p 0.6 the nucleus is the
    first two ids (the third has 0.75 before it) and the race picks them 2 : 1; (ii) eight equal
    ids with top-p 0.3: ties are cut by id, the first three belong (0, 0.125, 0.25 before them);
    (iii) top-p >= 1 keeps everything; (iv) without noise the choice is greedy and the score the
    penalised log-softmax value, as the reference's max() over lprobs gives."""
    V = 16
    pr = torch.tensor([2.0 ** -(i + 1) for i in range(V)])
    pr[-1] = pr[-2]
    order = torch.randperm(V, generator=torch.Generator().manual_seed(3))
    probs = torch.zeros(V)
    probs[order] = pr                          # the big ones are not the low ids
    N = 4096
    logits = probs.log().half().unsqueeze(0).repeat(N, 1)
    noise = torch.empty(N, V).exponential_(generator=torch.Generator().manual_seed(4))
    tok, sc = _sample(lib, G(logits), banned=[], topp_all=0.6, noise=G(noise))
    a, b2 = int(order[0]), int(order[1])
    assert set(tok.tolist()) == {a, b2}
    frac = float((tok == a).float().mean())
    assert abs(frac - 2 / 3) < 0.03, frac
    assert torch.allclose(sc[tok == a], torch.tensor(0.5).log(), atol=2e-3)
    # (ii) ties cut by id
    flat = torch.zeros(N, V, dtype=torch.float16)
    flat[:, 8:] = float("-inf")
    tok, _ = _sample(lib, G(flat), banned=[], topp_all=0.3, noise=G(noise))
    assert set(tok.tolist()) == {0, 1, 2}
    for t in (0, 1, 2):
        assert abs(float((tok == t).float().mean()) - 1 / 3) < 0.03
    # the same cut among tied ids for ties that lie in different rounds of the kernel's loop
    # (ids 5, 1100, 2500, 40000 and 51000 tied at the top, top-p 0.5: the first three), and in a
    # vocabulary beyond 65 536 ids, where the search among tied ids is a bisection
    for big in (51200, 70000):
        M = 256
        wide = torch.full((M, big), -20.0, dtype=torch.float16)
        tied = [5, 1100, 2500, 40000, big - 200]
        wide[:, tied] = 3.0
        nz = torch.empty(M, big).exponential_(generator=torch.Generator().manual_seed(6))
        tok, sc = _sample(lib, G(wide), banned=[], topp_all=0.5, noise=G(nz))
        assert set(tok.tolist()) == set(tied[:3]), (big, set(tok.tolist()))
        want = torch.log_softmax(wide[0].float(), -1)[5]
        assert torch.allclose(sc, want.expand(M), atol=1e-4)
    # (iii) the whole distribution
    tok, _ = _sample(lib, G(logits), banned=[], topp_all=1.0, noise=G(noise))
    freq = torch.bincount(tok, minlength=V).float() / N
    assert torch.allclose(freq, probs / probs.sum(), atol=0.03)
    # (iv) greedy with penalties: the arg-max of lprobs - penalties, score = that value
    counts = torch.zeros(N, V, dtype=torch.long)
    counts[:, a] = 5                           # pushes the best id below the second best
    cd = G(counts.clone())
    tok, sc = _sample(lib, G(logits), banned=[], counts=cd, alphas=(0.3, 0.2, 0.0, 0.0))
    lp = torch.log_softmax(logits[0].float(), -1)
    lp[a] -= 5 * 0.2 + 0.3
    assert int(tok[0]) == int(lp.argmax()) == b2 and bool((tok == b2).all())
    assert abs(float(sc[0]) - float(lp[b2])) < 2e-5
    assert int(cd[0, b2]) == 1
    # the same weights given per row (and none for the odd rows, which keep the best id), with
    # scalar arguments that must be ignored
    cd = G(counts.clone())
    rows = torch.zeros(N, 4)
    rows[0::2] = torch.tensor([0.3, 0.2, 0.0, 0.0])
    tok, sc = _sample(lib, G(logits), banned=[], counts=cd, alphas=(9.0, 9.0, 9.0, 9.0),
                      penalty_rows=G(rows))
    assert bool((tok[0::2] == b2).all()) and bool((tok[1::2] == a).all())
    assert abs(float(sc[0]) - float(lp[b2])) < 2e-5
    assert abs(float(sc[1]) - float(torch.log_softmax(logits[1].float(), -1)[a])) < 2e-5
    # prompt counts with per-row weights: frequency_src 0.5 on a count of 4 and presence_src 0.1
    cs = torch.zeros(N, V, dtype=torch.long)
    cs[:, a] = 4
    rows = torch.zeros(N, 4)
    rows[0] = torch.tensor([0.0, 0.0, 0.1, 0.5])
    tok, sc = _sample(lib, G(logits), banned=[], counts_src=G(cs), penalty_rows=G(rows))
    lp = torch.log_softmax(logits[0].float(), -1)
    lp[a] -= 4 * 0.5 + 0.1
    assert int(tok[0]) == int(lp.argmax()) and abs(float(sc[0]) - float(lp.max())) < 2e-5
    assert bool((tok[1:] == a).all())
    # a NaN logit: token 0 with score -inf, whatever the mode
    bad = logits[:2].clone()
    bad[0, 3] = float("nan")
    tok, sc = _sample(lib, G(bad), banned=[], topp_all=0.9, noise=G(noise[:2]))
    assert int(tok[0]) == 0 and float(sc[0]) == float("-inf") and float(sc[1]) > float("-inf")
