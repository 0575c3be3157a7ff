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
