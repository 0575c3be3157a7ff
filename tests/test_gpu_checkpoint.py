"""A model glued from tensor-parallel checkpoint parts, loaded into the HIP decoder, computes
what the parts compute together under the tensor-parallel oracle."""
import pytest
import torch

from metaseq_amd import OPTConfig, TransformerLanguageModel, checkpoint_utils as C
from oracle.tp_oracle import tp_forward

pytestmark = pytest.mark.gpu
L, D, H, FF, V, P = 2, 128, 2, 256, 64, 30


def _parts(mp, seed):
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, std=0.05):
        return (torch.randn(*shape, generator=g) * std).half()
    shared = {"decoder.embed_positions.weight": rnd(P + 2, D),
              "decoder.layer_norm.weight": (1 + rnd(D).float()).half(),
              "decoder.layer_norm.bias": rnd(D)}
    for i in range(L):
        p = "decoder.layers.%d." % i
        for ln in ("self_attn_layer_norm", "final_layer_norm"):
            shared[p + ln + ".weight"] = (1 + rnd(D).float()).half()
            shared[p + ln + ".bias"] = rnd(D)
        shared[p + "self_attn.out_proj.bias"] = rnd(D)
        shared[p + "fc2.bias"] = rnd(D)
    parts = []
    for r in range(mp):
        sd = {"decoder.version": torch.tensor([3.0]),
              "decoder.embed_tokens.weight": rnd(V // mp, D, std=0.1)}
        for i in range(L):
            p = "decoder.layers.%d." % i
            sd[p + "self_attn.qkv_proj.weight"] = rnd(3 * D // mp, D)
            sd[p + "self_attn.qkv_proj.bias"] = rnd(3 * D // mp)
            sd[p + "self_attn.out_proj.weight"] = rnd(D, D // mp)
            sd[p + "fc1.weight"] = rnd(FF // mp, D)
            sd[p + "fc1.bias"] = rnd(FF // mp)
            sd[p + "fc2.weight"] = rnd(D, FF // mp)
        sd.update({k: v.clone() for k, v in shared.items()})
        parts.append(sd)
    return parts


def test_glued_parts_load_into_the_decoder_and_match_the_tensor_parallel_oracle():
    parts = _parts(2, seed=11)
    tokens = torch.tensor([[2, 5, 9, 23, 12, 4, 17, 33], [2, 8, 8, 13, 40, 1, 1, 1]])
    want = tp_forward(parts, tokens, H)          # fp32 arithmetic on the fp16 weights
    state = C.normalize_state_dict(C.glue_model_parts(parts))
    cfg = OPTConfig(decoder_layers=L, decoder_embed_dim=D, decoder_attention_heads=H,
                    decoder_ffn_embed_dim=FF, vocab_size=V, max_target_positions=P)
    model = TransformerLanguageModel.build_model(cfg, state, device="cuda")
    got = model(tokens.cuda())[0].float().cpu()
    d = (got - want).abs()
    print("glued model vs tensor-parallel oracle: max-abs %.3e mean-abs %.3e"
          % (float(d.max()), float(d.mean())), flush=True)
    assert float(d.max()) <= 2e-2 and float(d.mean()) <= 2e-3
    # and a wrongly glued model (plain concatenation of the fused rows) is far off
    wrong = dict(state)
    k = "decoder.layers.0.self_attn.qkv_proj.weight"
    wrong[k] = torch.cat([p[k] for p in parts], 0)
    bad = TransformerLanguageModel.build_model(cfg, wrong, device="cuda")(tokens.cuda())[0]
    assert float((bad.float().cpu() - want).abs().max()) > 5e-2


def _int8_models(tmp_path):
    from metaseq_amd import random_state_dict
    from tests.common import tiny_cfg
    cfg = tiny_cfg(layers=2, dim=128, heads=2, vocab=96, max_pos=48)
    sd = random_state_dict(cfg, seed=21, dtype=torch.float16)
    online = TransformerLanguageModel.build_model(tiny_cfg(layers=2, dim=128, heads=2, vocab=96,
                                                           max_pos=48), sd, device="cuda:0")
    online.decoder.quantize_int8_()
    return cfg, sd, online


def _same_logits(a, b, cfg):
    g = torch.Generator().manual_seed(3)
    toks = torch.randint(4, cfg.vocab_size, (3, 17), generator=g).to("cuda:0")
    toks[:, 0] = 2
    ia, ib = {}, {}
    assert torch.equal(a(toks[:, :12], incremental_state=ia)[0],
                       b(toks[:, :12], incremental_state=ib)[0])
    for t in range(12, 17):
        assert torch.equal(a.decoder(toks[:, :t + 1], incremental_state=ia)[0],
                           b.decoder(toks[:, :t + 1], incremental_state=ib)[0])


def test_weights_quantised_offline_on_the_cpu_load_as_the_model_quantised_on_the_gpu(tmp_path):
    """The offline step (``quantize_state_dict`` on CPU tensors, saved and read back with the
    loader that executes nothing) gives, bit for bit, the model that ``quantize_int8_()`` makes
    from the fp16 weights on the GPU: same packed int8 bytes and scales, same logits through
    prefill and decode steps."""
    print("offline int8", flush=True)
    cfg, sd, online = _int8_models(tmp_path)
    path = str(tmp_path / "int8.pt")
    torch.save({"model": C.quantize_state_dict(sd)}, path)
    state = torch.load(path, map_location="cpu", weights_only=True)["model"]
    offline = TransformerLanguageModel.build_model(cfg, state, device="cuda:0")
    assert cfg.quantize_int8
    for (name, a), (_, b) in zip(online.decoder._linears(), offline.decoder._linears()):
        assert b.weight.numel() == 0 and not b.packed
        assert torch.equal(a.qweight, b.qweight) and torch.equal(a.scales, b.scales), name
    _same_logits(online, offline, cfg)


def test_quantised_state_dict_round_trip_and_streaming(tmp_path):
    """``quantized_state_dict()`` of an int8 model equals the offline step's output, loads
    again whole (``load_state_dict``, also over a model that already holds packed weights) and
    streamed (``load_tensors``), and fp16 matrices beside int8 ones are refused."""
    print("int8 state dict", flush=True)
    from tests.common import tiny_cfg
    cfg, sd, online = _int8_models(tmp_path)
    qsd = online.decoder.quantized_state_dict()
    want = C.quantize_state_dict(sd)
    assert set(qsd) - {"decoder.version"} == set(want) - {"decoder.version"}
    for k, v in want.items():
        if k != "decoder.version":
            assert torch.equal(qsd[k].cpu(), v), k
    new = lambda: tiny_cfg(layers=2, dim=128, heads=2, vocab=96, max_pos=48)
    again = TransformerLanguageModel.build_model(new(), sd, device="cuda:0")
    again.decoder.prepare_()                       # packed fp16 weights, replaced below
    again.load_state_dict(qsd)
    _same_logits(online, again, cfg)
    streamed = TransformerLanguageModel.build_model(new(), None, device="cuda:0")
    streamed.decoder.load_tensors((k, v.cpu()) for k, v in qsd.items())
    _same_logits(online, streamed, cfg)
    mixed = dict(want)
    k = "decoder.layers.1.fc2."
    del mixed[k + "qweight"], mixed[k + "scales"]
    mixed[k + "weight"] = sd[k + "weight"]
    with pytest.raises(KeyError, match="layers.1.fc2 arrived in fp16 beside int8 layers"):
        TransformerLanguageModel.build_model(new(), mixed, device="cuda:0")
    with pytest.raises(ValueError, match="int8 weight: expected"):
        bad = dict(want)
        bad[k + "qweight"] = bad[k + "qweight"][:-1]
        TransformerLanguageModel.build_model(new(), bad, device="cuda:0")
    fp16 = TransformerLanguageModel.build_model(new(), sd, device="cuda:0")
    with pytest.raises(RuntimeError, match="needs an int8 model"):
        fp16.decoder.quantized_state_dict()
