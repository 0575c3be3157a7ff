"""Host logic of the streaming weight loader (no GPU needed: parameters are plain tensors until
the first forward packs them)."""
import pytest
import torch

from metaseq_amd import TransformerDecoder, iter_random_state_dict, random_state_dict
from tests.common import tiny_cfg


def test_load_tensors_equals_load_state_dict():
    cfg = tiny_cfg(layers=2, dim=64, heads=1, vocab=64, max_pos=32)
    streamed = TransformerDecoder(cfg, None, device="cpu")
    streamed.load_tensors(iter_random_state_dict(cfg, seed=3))
    whole = TransformerDecoder(cfg, random_state_dict(cfg, seed=3), device="cpu")
    a, b = streamed.state_dict(), whole.state_dict()
    assert set(a) == set(b)
    for k in a:
        assert torch.equal(a[k], b[k]), k


def test_load_tensors_reports_missing_repeated_and_misshapen_parameters():
    cfg = tiny_cfg(layers=1, dim=64, heads=1, vocab=64, max_pos=32)
    items = list(iter_random_state_dict(cfg, seed=3))
    with pytest.raises(KeyError, match="missing parameters: layer_norm.bias"):
        TransformerDecoder(cfg, None, device="cpu").load_tensors(items[:-1])
    with pytest.raises(KeyError, match="unexpected or repeated"):
        TransformerDecoder(cfg, None, device="cpu").load_tensors(items + items[-1:])
    bad = [(n, t[:-1] if n.endswith("fc1.bias") else t) for n, t in items]
    with pytest.raises(ValueError, match="shape of layers.0.fc1.bias"):
        TransformerDecoder(cfg, None, device="cpu").load_tensors(bad)


def test_unsupported_head_size_is_refused_before_anything_is_allocated():
    """OPT-2.7B's head_dim 80 has no attention kernel: building the decoder says so at once
    instead of failing at the first attention call."""
    from metaseq_amd import OPTConfig
    cfg = OPTConfig(32, 2560, 32)
    assert cfg.head_dim == 80
    with pytest.raises(NotImplementedError, match="head_dim 80"):
        TransformerDecoder(cfg, None, device="meta")


def test_kv_cache_row_views_follow_growth_and_keep_nothing_alive():
    """A view of rows b0 .. b1 - 1 reads the cache's current tensors (also after growth), is
    the same object for the same range (work buffers kept on it persist), and does not keep
    the cache alive: dropping the last outside reference frees it at once."""
    import gc
    import weakref

    import torch

    from metaseq_amd.kv_cache import KVCache
    cache = KVCache(2, 6, 2, 8, 16, "cpu")
    cache.layers[1][1].copy_(torch.arange(6).view(6, 1, 1, 1).expand(6, 2, 16, 8))
    view = cache.rows_view(2, 5)
    assert view is cache.rows_view(2, 5) and view is not cache.rows_view(0, 2)
    assert view.k(0).shape == (3, 2, 16, 8) and view.v(1).is_contiguous()
    assert view.v(1)[:, 0, 0, 0].tolist() == [2.0, 3.0, 4.0]
    cache.length = 16
    cache.grow(40)
    assert view.capacity == 40 and view.v(1).shape == (3, 2, 40, 8)
    assert view.v(1)[:, 1, 15, 7].tolist() == [2.0, 3.0, 4.0]
    gc.disable()
    try:
        ref = weakref.ref(cache)
        del cache, view
        assert ref() is None
    finally:
        gc.enable()
