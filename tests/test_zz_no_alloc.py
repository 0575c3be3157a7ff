"""The entry point that allocates nothing (msa_lm_head_greedy_select_noalloc_f16) against
msa_lm_head_greedy_select_f16 with a caller-provided workspace, through the C ABI.

Both run the same kernels; only the home of the selection partials differs (a fixed device array
inside the library instead of the workspace), so tokens, finished flags, scores and stored
logits must be bit-identical.  Two calls in a row, the second with fewer rows and a smaller
vocabulary, so that stale partials of the first call sit in the shared array while the second
runs.  The test also asserts that the call leaves torch's allocator statistics and the device's
own count of free memory untouched, and that sizes beyond the fixed array are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _pack_act(x):
    M, K = x.shape
    MB = (M + 15) // 16 if M <= 64 else 8   # 65 .. 128 rows: always eight row blocks
    xp = torch.zeros(MB * 16, K, dtype=x.dtype)
    xp[:M] = x
    return xp.view(MB, 16, K // 32, 4, 8).permute(2, 0, 3, 1, 4).contiguous().view(-1)


def _case(lib, M, V, K, seed, banned, stop, temperature, finished_rows, device_memory=False):
    P = lambda t: None if t is None else t.data_ptr()
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).half()
    E = (torch.randn(V, K, generator=g) * 0.3).half().to(DEV)
    Ep = torch.empty_like(E)
    assert lib.msa_pack_weight_f16(P(E), P(Ep), V, K, None) == 0, lib.msa_last_error()
    xp = _pack_act(x).to(DEV)
    ws = torch.empty(lib.msa_lm_head_select_workspace_bytes(M), dtype=torch.uint8, device=DEV)
    ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
    sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
    outs = []
    for noalloc in (False, True):
        fin = torch.tensor(finished_rows, dtype=torch.uint8, device=DEV)
        tok = torch.full((M, 3), -7, dtype=torch.long, device=DEV)
        sc = torch.full((M, 3), 9.0, dtype=torch.float32, device=DEV)
        lg = torch.zeros(M, V, dtype=torch.float16, device=DEV)
        torch.cuda.synchronize()
        if noalloc:
            before = torch.cuda.memory_stats()["allocation.all.allocated"]
            free_before = torch.cuda.mem_get_info()[0]
            rc = lib.msa_lm_head_greedy_select_noalloc_f16(
                P(xp), P(Ep), P(lg), M, V, K, temperature, ba, len(banned), sa, len(stop), P(fin),
                None, 0, 2, P(tok[:, 1]), 3, P(sc[:, 1]), 3, None, None)
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
            if device_memory:
                # torch's statistics cannot see a hipMalloc made inside the library; the
                # device's own count of free bytes can (asked for on a call after the first on
                # this device, which may load the code object)
                torch.cuda.synchronize()
                assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated"
        else:
            rc = lib.msa_lm_head_greedy_select_f16(
                P(xp), P(Ep), P(lg), P(ws), M, V, K, temperature, ba, len(banned), sa, len(stop),
                P(fin), None, 0, 2, P(tok[:, 1]), 3, P(sc[:, 1]), 3, None, None)
        assert rc == 0, lib.msa_last_error().decode()
        torch.cuda.synchronize()
        outs.append((tok.cpu(), sc.cpu(), fin.cpu(), lg.cpu()))
    (t0, s0, f0, l0), (t1, s1, f1, l1) = outs
    assert torch.equal(t0, t1), "tokens differ"
    assert torch.equal(s0, s1), "scores differ"
    assert torch.equal(f0, f1), "finished flags differ"
    assert torch.equal(l0, l1), "stored logits differ"
    # and the tokens are the masked arg-max of the stored logits
    z = l0.float()
    z[:, banned] = float("-inf")
    want = z.argmax(-1)
    # a finished row may only emit eos; if eos is banned too, nothing is eligible and the
    # lowest index wins, as the reference's max over an all -inf row does
    want[torch.tensor(finished_rows, dtype=torch.bool)] = 0 if 2 in banned else 2
    assert torch.equal(t0[:, 1], want)
    assert int((t0[:, 0] != -7).sum()) == 0 and int((t0[:, 2] != -7).sum()) == 0


def test_noalloc_entry_matches_workspace_entry_on_two_calls_in_a_row():
    from metaseq_amd import _capi
    lib = _capi.load()
    print("no-alloc: M=64 V=50272 K=256, then M=5 V=4000 K=128", flush=True)
    _case(lib, 64, 50272, 256, 11, banned=[1, 2], stop=[17], temperature=0.7,
          finished_rows=[i % 5 == 0 for i in range(64)])
    # second call: fewer rows, fewer workgroups; the array still holds the first call's partials
    _case(lib, 5, 4000, 128, 12, banned=[1], stop=[], temperature=1.0,
          finished_rows=[False] * 5, device_memory=True)


def test_noalloc_entry_rejects_sizes_beyond_the_fixed_array():
    from metaseq_amd import _capi
    lib = _capi.load()
    one = ctypes.c_void_p(256)
    ba = (ctypes.c_int32 * 1)(1)
    rc = lib.msa_lm_head_greedy_select_noalloc_f16(one, one, None, 65, 4000, 128, 1.0, ba, 1, ba,
                                                   0, None, None, 0, 2, one, 1, one, 1, None, None)
    assert rc == -2 and b"exceed" in lib.msa_last_error()
