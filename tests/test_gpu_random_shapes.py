"""Seeded random shapes through the C ABI: the decode GEMM paths (1 .. 128 packed rows, fp16 and
int8 weights, with and without split-K), the prefill GEMM paths (hundreds to thousands of
row-major rows, enough 256 x 256 tiles for the large tiled kernels) and both attention kernels (one query per row over a
history; a block of queries, causal, optionally appended to a history, optionally with a key
padding mask), each against the same arithmetic written with torch ops on the device.  The fixed
shapes of test_gpu_kernels.py pin the layouts and rounding points; these cases sweep the launch
geometry (tiles per workgroup, K ranges shorter than a stage, ragged tiles, cache capacities)."""
import random

import pytest
import torch

from tests.test_gpu_kernels import pack_act

pytestmark = pytest.mark.gpu
DEV = "cuda"


def r16(t):
    return t.half().float()


@pytest.fixture(scope="module")
def lib():
    from metaseq_amd import _capi
    return _capi.load()


def test_decode_gemm_random_shapes(lib):
    rng = random.Random(7)
    ran = 0
    for it in range(90):
        # two thirds of the cases up to 64 rows (row blocks as needed), the rest 65 .. 128
        # (always eight row blocks, the kernel that shares activation fragments between waves)
        M = rng.randint(1, 64) if it % 3 else rng.randint(65, 128)
        N = 16 * rng.choice([1, 3, 7, 20, 63, 64, 100, 257, 500, 1000, 2304, 3142])
        w8 = rng.random() < 0.5
        K = (64 if w8 else 32) * rng.choice([1, 2, 3, 5, 8, 12, 17, 32, 48, 64])
        S = rng.choice([1, 1, 2, 3, 4, 8])
        print("gemm case", it, M, N, K, "int8" if w8 else "fp16", "S", S, flush=True)
        g = torch.Generator().manual_seed(it)
        x = (torch.randn(M, K, generator=g) * 0.5).half()
        xp = pack_act(x).to(DEV)
        if w8:
            q = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
            sc = (torch.rand(N, generator=g) * 0.01 + 0.001).half()
            Wd = (q.float() * sc.float()[:, None]).half()
            qd, scd = q.to(DEV), sc.to(DEV)
            Wp = torch.empty_like(qd)
            assert lib.msa_pack_weight_i8(qd.data_ptr(), Wp.data_ptr(), N, K, None) == 0
        else:
            Wd = (torch.randn(N, K, generator=g) * 0.05).half()
            wd = Wd.to(DEV)
            Wp = torch.empty_like(wd)
            assert lib.msa_pack_weight_f16(wd.data_ptr(), Wp.data_ptr(), N, K, None) == 0
        ref = x.to(DEV).float() @ Wd.to(DEV).float().t()
        if S == 1:
            b = (torch.randn(N, generator=g) * 0.1).half().to(DEV)
            y = torch.full((M, N), float("nan"), dtype=torch.float16, device=DEV)
            if w8:
                rc = lib.msa_linear_w8a16(xp.data_ptr(), Wp.data_ptr(), scd.data_ptr(),
                                          b.data_ptr(), None, y.data_ptr(), M, N, K, 2, None)
            else:
                rc = lib.msa_linear_f16(xp.data_ptr(), Wp.data_ptr(), b.data_ptr(), None,
                                        y.data_ptr(), M, N, K, 2, None)
            assert rc == 0, lib.msa_last_error()
            torch.cuda.synchronize()
            got, want = y.float(), r16(r16(ref) + b.float())
        else:
            part = torch.full((S, M, N), float("nan"), dtype=torch.float32, device=DEV)
            if w8:
                rc = lib.msa_linear_partial_w8a16(xp.data_ptr(), Wp.data_ptr(), scd.data_ptr(),
                                                  part.data_ptr(), M, N, K, S, 2, None)
            else:
                rc = lib.msa_linear_partial_f16(xp.data_ptr(), Wp.data_ptr(), part.data_ptr(), M,
                                                N, K, S, 2, None)
            if rc != 0:  # a split count the K range cannot be cut into: refused, nothing ran
                assert b"outside" in lib.msa_last_error() or b"empty" in lib.msa_last_error()
                continue
            torch.cuda.synchronize()
            got, want = part.sum(0), ref  # every slice written (no NaN left), sums exact in fp32
        ran += 1
        assert torch.isfinite(got).all(), (it, "unwritten or non-finite output")
        err = float((got - want).abs().max())
        assert err <= max(1e-3, float(want.abs().max()) * 2e-3), (it, err)
    assert ran >= 60


def test_prefill_gemm_random_shapes(lib):
    """Row-major activations with enough output tiles for the large tiled kernels: ragged bottom
    row tiles (moved up, or handed to the streaming kernel), ragged right tiles, 8 / 16 tiles
    across (regrouped per XCD), K a multiple of 64 but not of 128, every epilogue, y aliasing the
    residual."""
    rng = random.Random(23)
    for it in range(18):
        w8 = it % 3 == 2
        ncol = rng.choice([8, 16, 16, 33, 48, 65, 100])
        small = it % 6 == 1  # few tiles: the 256 x 128 form of the four-wave kernel
        N = 256 * ncol - 16 * rng.choice([0, 0, 1, 5, 15])
        nrow = max(1, 100 // ncol) if small else -(-256 // ncol) + rng.choice([0, 1, 3])
        M = max(256, 256 * nrow - rng.choice([0, 0, 1, 100, 128, 129, 200, 255]))
        if it % 6 == 4:
            M = rng.choice([65, 100, 128, 200, 255])  # fewer rows than a tile: the 256 x 64 form
        K = 64 * rng.choice([2, 3, 4, 5, 8, 12])
        relu, use_res = rng.random() < 0.4, rng.random() < 0.6
        in_place = use_res and rng.random() < 0.5
        print("prefill gemm case", it, M, N, K, "int8" if w8 else "fp16", relu, use_res, in_place,
              flush=True)
        g = torch.Generator(device=DEV).manual_seed(100 + it)
        x = (torch.randn(M, K, generator=g, device=DEV) * 0.5).half()
        b = (torch.randn(N, generator=g, device=DEV) * 0.1).half()
        res = torch.randn(M, N, generator=g, device=DEV).half() if use_res else None
        if w8:
            q = torch.randint(-127, 128, (N, K), generator=g, device=DEV, dtype=torch.int8)
            sc = (torch.rand(N, generator=g, device=DEV) * 0.01 + 0.001).half()
            Wd = (q.float() * sc.float()[:, None]).half()
            Wp = torch.empty_like(q)
            assert lib.msa_pack_weight_i8(q.data_ptr(), Wp.data_ptr(), N, K, None) == 0
        else:
            Wd = (torch.randn(N, K, generator=g, device=DEV) * 0.05).half()
            Wp = torch.empty_like(Wd)
            assert lib.msa_pack_weight_f16(Wd.data_ptr(), Wp.data_ptr(), N, K, None) == 0
        want = r16(r16(x.float() @ Wd.float().t()) + b.float())
        if relu:
            want = want.clamp_min(0)
        if use_res:
            want = r16(want + res.float())
        y = res.clone() if in_place else torch.full((M, N), float("nan"), dtype=torch.float16,
                                                    device=DEV)
        rp = None if res is None else (y.data_ptr() if in_place else res.data_ptr())
        flags = 1 if relu else 0
        if w8:
            rc = lib.msa_linear_w8a16(x.data_ptr(), Wp.data_ptr(), sc.data_ptr(), b.data_ptr(), rp,
                                      y.data_ptr(), M, N, K, flags, None)
        else:
            rc = lib.msa_linear_f16(x.data_ptr(), Wp.data_ptr(), b.data_ptr(), rp, y.data_ptr(), M,
                                    N, K, flags, None)
        assert rc == 0, lib.msa_last_error()
        torch.cuda.synchronize()
        got = y.float()
        assert torch.isfinite(got).all(), (it, "unwritten or non-finite output")
        err = float((got - want).abs().max())
        # one fp16 ulp of the largest intermediate (a 1-ulp difference of the rounded product
        # survives the bias / residual additions at the product's magnitude)
        assert err <= float(want.abs().max()) * 2 ** -9 + 2e-3, (it, err)


def test_few_row_major_rows_gemm_random_shapes(lib):
    """Row-major activations of 1 .. 64 rows (fp16 and int8: one sweep of the streaming kernel)
    and of 65 .. 256 rows over int8 weights (a sweep per 64 rows), with output widths that are
    not multiples of a workgroup's tiles, every epilogue, y aliasing the residual; and the
    split-K form on row-major rows with the slices the library suggests."""
    rng = random.Random(31)
    for it in range(24):
        w8 = it % 2 == 1
        M = rng.randint(65, 256) if (w8 and it % 4 == 3) else rng.randint(1, 64)
        N = 16 * rng.choice([1, 3, 7, 20, 63, 64, 100, 257, 500, 768, 2304])
        K = 64 * rng.choice([1, 2, 3, 5, 8, 12, 17, 32, 64])
        relu, use_res = rng.random() < 0.4, rng.random() < 0.6
        in_place = use_res and rng.random() < 0.5
        print("few rows gemm case", it, M, N, K, "int8" if w8 else "fp16", relu, use_res,
              in_place, flush=True)
        g = torch.Generator(device=DEV).manual_seed(300 + it)
        x = (torch.randn(M, K, generator=g, device=DEV) * 0.5).half()
        b = (torch.randn(N, generator=g, device=DEV) * 0.1).half()
        res = torch.randn(M, N, generator=g, device=DEV).half() if use_res else None
        if w8:
            q = torch.randint(-127, 128, (N, K), generator=g, device=DEV, dtype=torch.int8)
            sc = (torch.rand(N, generator=g, device=DEV) * 0.01 + 0.001).half()
            Wd = (q.float() * sc.float()[:, None]).half()
            Wp = torch.empty_like(q)
            assert lib.msa_pack_weight_i8(q.data_ptr(), Wp.data_ptr(), N, K, None) == 0
        else:
            Wd = (torch.randn(N, K, generator=g, device=DEV) * 0.05).half()
            Wp = torch.empty_like(Wd)
            assert lib.msa_pack_weight_f16(Wd.data_ptr(), Wp.data_ptr(), N, K, None) == 0
        prod = x.float() @ Wd.float().t()
        want = r16(r16(prod) + b.float())
        if relu:
            want = want.clamp_min(0)
        if use_res:
            want = r16(want + res.float())
        y = res.clone() if in_place else torch.full((M, N), float("nan"), dtype=torch.float16,
                                                    device=DEV)
        rp = None if res is None else (y.data_ptr() if in_place else res.data_ptr())
        flags = 1 if relu else 0
        if w8:
            rc = lib.msa_linear_w8a16(x.data_ptr(), Wp.data_ptr(), sc.data_ptr(), b.data_ptr(), rp,
                                      y.data_ptr(), M, N, K, flags, None)
        else:
            rc = lib.msa_linear_f16(x.data_ptr(), Wp.data_ptr(), b.data_ptr(), rp, y.data_ptr(), M,
                                    N, K, flags, None)
        assert rc == 0, lib.msa_last_error()
        torch.cuda.synchronize()
        got = y.float()
        assert torch.isfinite(got).all(), (it, "unwritten or non-finite output")
        err = float((got - want).abs().max())
        assert err <= float(want.abs().max()) * 2 ** -9 + 2e-3, (it, err)
        if w8 or K < 256:
            continue
        # split-K partial sums of the same product on row-major rows
        S = max(2, lib.msa_linear_default_splits_rows(M, N, K))
        while K % (64 * S) or K // S < 128:
            S //= 2
        if S < 2:
            continue
        part = torch.full((S, M, N), float("nan"), dtype=torch.float32, device=DEV)
        rc = lib.msa_linear_partial_f16(x.data_ptr(), Wp.data_ptr(), part.data_ptr(), M, N, K, S,
                                        0, None)
        assert rc == 0, lib.msa_last_error()
        torch.cuda.synchronize()
        assert float((part.sum(0) - prod).abs().max()) < 2e-3 * max(1.0, float(prod.abs().max()))


def test_attention_random_shapes(lib):
    rng = random.Random(11)
    for it in range(48):
        hd, H, B = rng.choice([64, 128]), rng.choice([1, 2, 3, 5]), rng.choice([1, 2, 3, 7, 33])
        T = rng.choice([1, 1, 1, 2, 17, 64, 65, 127, 128, 129, 200, 300])
        S0 = (rng.choice([0, 0, 1, 5, 63, 64, 100, 511, 700]) if T > 1
              else rng.choice([0, 1, 7, 63, 64, 255, 256, 1000, 2047]))
        if it >= 45:
            # more than 64 MiB of K and V rows: the prefill kernel gives all query tiles of a
            # (row, head) pair to one XCD; pair counts that are no multiple of 8, both head sizes
            hd, H, B, T, S0 = [(64, 33, 2, 4000, 9), (128, 11, 3, 4100, 0), (64, 9, 5, 6100, 70)][it - 45]
        S = S0 + T
        S_cap = S + rng.choice([0, 1, 9, 64])
        masked = rng.random() < 0.4
        print("attention case", it, "B", B, "H", H, "hd", hd, "T", T, "S0", S0, "cap", S_cap,
              "mask", masked, flush=True)
        g = torch.Generator(device=DEV).manual_seed(it)
        D = H * hd
        q = (torch.randn(B * T, D, device=DEV, generator=g) * 0.3).half()
        Kc = torch.randn(B, H, S_cap, hd, device=DEV, generator=g).half()
        Vc = torch.randn(B, H, S_cap, hd, device=DEV, generator=g).half()
        # rows past the history hold NaN: none of them may reach the result
        Kc[:, :, S:] = float("nan")
        Vc[:, :, S:] = float("nan")
        mask = None
        if masked:
            mask = torch.zeros(B, S, dtype=torch.bool, device=DEV)
            for b in range(B):
                for _ in range(rng.randint(0, 3)):
                    mask[b, rng.randint(1, S - 1) if S > 1 else 0] = True
            mask[:, 0] = False  # key 0 stays visible: no fully masked row
        qq = q.float().view(B, T, H, hd).permute(0, 2, 1, 3)
        s = r16(qq @ Kc[:, :, :S].float().transpose(-1, -2))
        s = s + torch.full((T, S), float("-inf"), device=DEV).triu(S0 + 1)
        if mask is not None:
            s = s.masked_fill(mask[:, None, None, :], float("-inf"))
        p = r16(torch.softmax(s, -1, dtype=torch.float32))
        want = r16(p @ Vc[:, :, :S].float()).permute(0, 2, 1, 3).reshape(B * T, D)
        out = torch.full((B * T, D), float("nan"), dtype=torch.float16, device=DEV)
        dm = None if mask is None else mask.to(torch.uint8)
        rc = lib.msa_attention_f16(q.data_ptr(), Kc.data_ptr(), Vc.data_ptr(),
                                   None if dm is None else dm.data_ptr(),
                                   0 if dm is None else dm.stride(0), out.data_ptr(), B, H, hd, T,
                                   S0, S_cap, 0, None, None)
        assert rc == 0, lib.msa_last_error()
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all(), it
        err = float((out.float() - want).abs().max())
        # a 1-ulp flip of an fp16 score scales its probability by up to e^(2^-7)
        assert err <= float(want.abs().max()) * 2 ** -6 + 1e-3, (it, err)
