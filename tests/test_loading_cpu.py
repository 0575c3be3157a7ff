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


def test_offline_quantisation_replaces_the_four_per_layer_matrices_and_nothing_else():
    """``quantize_state_dict`` against the oracle's quantiser: qkv_proj / out_proj / fc1 / fc2
    weights of every layer become (.qweight, .scales) with the oracle's values; embeddings,
    biases and LayerNorms pass through untouched, with or without the "decoder." prefix."""
    from metaseq_amd.checkpoint_utils import is_quantized_state, quantize_state_dict
    from oracle.opt_oracle import quantize_int8
    cfg = tiny_cfg(layers=2, dim=64, heads=1, vocab=64, max_pos=32)
    sd = random_state_dict(cfg, seed=5)
    sd["decoder.layers.1.fc1.weight"][3].zero_()  # an all-zero row: scale 0, q 0
    for prefix in ("decoder.", ""):
        src = {(k[len("decoder."):] if not prefix else k): v for k, v in sd.items()}
        out = quantize_state_dict(src)
        assert is_quantized_state(out) and not is_quantized_state(src)
        changed = {k for k in src if k not in out}
        want = {"%slayers.%d.%s.weight" % (prefix, i, m) for i in range(2)
                for m in ("self_attn.qkv_proj", "self_attn.out_proj", "fc1", "fc2")}
        assert changed == want
        for k in want:
            q, s = quantize_int8(src[k])
            stem = k[:-len("weight")]
            assert out[stem + "qweight"].dtype == torch.int8 and out[stem + "scales"].dtype == torch.float16
            assert torch.equal(out[stem + "qweight"], q) and torch.equal(out[stem + "scales"], s)
        for k in src:
            if k not in want:
                assert out[k] is src[k]
        assert out[prefix + "layers.1.fc1.scales"][3] == 0
        assert not out[prefix + "layers.1.fc1.qweight"][3].any()


def test_load_tensors_refuses_int8_names_it_does_not_know():
    from metaseq_amd.checkpoint_utils import quantize_state_dict
    cfg = tiny_cfg(layers=1, dim=64, heads=1, vocab=64, max_pos=32)
    items = list(quantize_state_dict(dict(iter_random_state_dict(cfg, seed=3))).items())
    odd = [("layer_norm.qweight", torch.zeros(64, dtype=torch.int8))] + items
    with pytest.raises(KeyError, match="unexpected parameter 'layer_norm.qweight'"):
        TransformerDecoder(cfg, None, device="cpu").load_tensors(odd)
    twice = [items[i] for i in range(len(items))]
    name = next(n for n, _ in items if n.endswith("fc1.scales"))
    twice.insert(0, (name, dict(items)[name]))
    twice.insert(0, (name, dict(items)[name]))
    with pytest.raises(KeyError, match="unexpected or repeated parameter"):
        TransformerDecoder(cfg, None, device="cpu").load_tensors(twice)


def test_configuration_is_read_off_a_state_dicts_shapes():
    """Layers, widths, vocabulary and position count come from tensor shapes (fp16 or
    quantised offline, with or without the "decoder." prefix); heads from the OPT size table,
    or from the caller where the shape pair is no OPT size."""
    from metaseq_amd import config_from_state_dict, opt_config
    from metaseq_amd.checkpoint_utils import quantize_state_dict
    cfg = tiny_cfg(layers=3, dim=64, heads=1, vocab=72, max_pos=40, ffn=96)
    sd = random_state_dict(cfg, seed=1)
    with pytest.raises(ValueError, match="pass heads="):
        config_from_state_dict(sd)
    for state in (sd, quantize_state_dict(sd), {k[len("decoder."):]: v for k, v in sd.items()}):
        got = config_from_state_dict(state, heads=1)
        assert got == cfg
        TransformerDecoder(got, None, device="meta")
    # an OPT size: shapes alone (meta tensors stand in for OPT-125M's weights)
    want = opt_config("125m")
    dec = TransformerDecoder(want, None, device="meta")
    assert config_from_state_dict(torch.nn.Module.state_dict(dec)) == want
    assert config_from_state_dict(torch.nn.Module.state_dict(dec), max_target_positions=512
                                  ).max_target_positions == 512
