"""Checkpoint gluing rules pinned by the invariant they exist for: a model glued from
tensor-parallel parts computes the logits the parts compute together.

The parts are drawn independently with the per-rank shapes (not cut from a glued model by the
inverse rule), evaluated by the tensor-parallel oracle, which writes the reference's Megatron
collectives out as sums and concatenations, and compared with the single-part oracle (pinned
against Hugging Face OPT) on the glued state dict.  A wrong concatenation axis, a plain
concatenation of the fused K|V|Q rows, or a summed replicated bias each change the logits."""
import os

import pytest
import torch

from metaseq_amd import checkpoint_utils as C
from oracle.opt_oracle import OracleConfig, OracleDecoder
from oracle.tp_oracle import tp_forward

L, D, H, FF, V, P = 2, 32, 4, 64, 24, 20


def _parts(mp, seed=0):
    g = torch.Generator().manual_seed(seed)
    def rnd(*shape, std=0.2):
        return torch.randn(*shape, generator=g) * std
    shared = {"decoder.embed_positions.weight": rnd(P + 2, D),
              "decoder.layer_norm.weight": 1 + rnd(D), "decoder.layer_norm.bias": rnd(D)}
    for i in range(L):
        p = "decoder.layers.%d." % i
        for ln in ("self_attn_layer_norm", "final_layer_norm"):
            shared[p + ln + ".weight"] = 1 + rnd(D)
            shared[p + ln + ".bias"] = rnd(D)
        shared[p + "self_attn.out_proj.bias"] = rnd(D)
        shared[p + "fc2.bias"] = rnd(D)
    parts = []
    for r in range(mp):
        sd = {"decoder.version": torch.tensor([3.0]),
              "decoder.embed_tokens.weight": rnd(V // mp, D)}
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


def _single_logits(state, tokens):
    cfg = OracleConfig(L, D, H, FF, V, max_target_positions=P)
    return OracleDecoder(cfg, state, torch.float32)(tokens)[0]


TOKENS = torch.tensor([[2, 5, 9, 23, 12, 4, 17], [2, 8, 8, 13, 1, 1, 1]])


def test_tp_oracle_at_one_rank_is_the_single_part_oracle():
    [sd] = _parts(1)
    got = tp_forward([sd], TOKENS, H)
    want = _single_logits(C.normalize_state_dict(sd), TOKENS)
    assert torch.allclose(got, want, atol=1e-5)


@pytest.mark.parametrize("mp", [2, 4])
def test_glued_model_computes_what_the_parts_compute(mp):
    parts = _parts(mp, seed=mp)
    want = tp_forward(parts, TOKENS, H)
    glued = C.normalize_state_dict(C.glue_model_parts(parts))
    got = _single_logits(glued, TOKENS)
    assert got.shape == want.shape == (2, 7, V)
    assert torch.allclose(got, want, atol=2e-5), float((got - want).abs().max())
    assert "decoder.output_projection.weight" not in glued
    # the fused rows are K | V | Q of all heads, not the parts' blocks one after another
    plain = torch.cat([p["decoder.layers.0.self_attn.qkv_proj.weight"] for p in parts], 0)
    assert not torch.equal(glued["decoder.layers.0.self_attn.qkv_proj.weight"], plain)


@pytest.mark.parametrize("mp", [2, 4])
def test_split_is_the_inverse_of_glue(mp):
    parts = _parts(mp, seed=7)
    glued = C.glue_model_parts(parts)
    again = C.split_model_parts(glued, mp)
    for a, b in zip(parts, again):
        assert list(a.keys()) == list(b.keys())
        for k in a:
            assert torch.equal(a[k], b[k]), k
    # resharding 4 -> 2 parts keeps the function
    if mp == 4:
        two = C.split_model_parts(glued, 2)
        assert torch.allclose(tp_forward(two, TOKENS, H), tp_forward(parts, TOKENS, H), atol=2e-5)


def test_replicated_parameters_that_drifted_are_taken_from_part_0_with_a_warning(caplog):
    """The reference only logs the largest discrepancy between the parts' copies of a
    replicated parameter and keeps part 0's (stitch_fsdp_ckpt.py:253-262); a shape mismatch or
    a difference above an explicit tolerance is an error."""
    parts = _parts(2)
    key = "decoder.layer_norm.bias"
    one_ulp = parts[1][key].half()
    one_ulp = (one_ulp.view(torch.int16) + 1).view(torch.float16).float()  # next fp16 up
    parts[1][key] = one_ulp
    parts[0][key] = parts[0][key].half().float()
    with caplog.at_level("WARNING", logger="metaseq_amd.checkpoint_utils"):
        glued = C.glue_model_parts(parts)
    assert torch.equal(glued[key], parts[0][key])
    assert any(key in r.getMessage() and "taking part 0" in r.getMessage()
               for r in caplog.records)
    with pytest.raises(ValueError, match="tolerance"):
        C.glue_model_parts(parts, replica_tolerance=1e-9)
    C.glue_model_parts(parts, replica_tolerance=1.0)
    parts[1][key] = parts[1][key][:-1]
    with pytest.raises(ValueError, match="shape"):
        C.glue_model_parts(parts)


def test_normalize_fuses_a_singleton_checkpoint_and_drops_tied_projection():
    [sd] = _parts(1)
    sd = C.normalize_state_dict(sd)
    single = {}
    for k, v in sd.items():
        if "qkv_proj" in k:
            kk, vv, qq = v.split(v.shape[0] // 3, 0)
            single[k.replace("qkv_proj", "q_proj")] = qq   # any order in the file
            single[k.replace("qkv_proj", "k_proj")] = kk
            single[k.replace("qkv_proj", "v_proj")] = vv
        else:
            single[k] = v
    single["decoder.output_projection.weight"] = sd["decoder.embed_tokens.weight"].clone()
    back = C.normalize_state_dict(single)
    assert set(back) == set(sd)
    for k in sd:
        assert torch.equal(back[k], sd[k]), k


def test_load_model_state_reads_parts_from_files(tmp_path):
    parts = _parts(2, seed=3)
    names = []
    for r, p in enumerate(parts):
        path = os.path.join(tmp_path, "reshard-model_part-%d.pt" % r)
        torch.save({"model": p} if r == 0 else p, path)   # both file shapes
        names.append(path)
    ordered = C.find_model_parts(list(reversed(names)))
    assert ordered == names
    state = C.load_model_state(ordered)
    want = C.normalize_state_dict(C.glue_model_parts(parts))
    assert set(state) == set(want) and all(torch.equal(state[k], want[k]) for k in want)
    with pytest.raises(ValueError):
        C.find_model_parts([names[1]])
    bad = os.path.join(tmp_path, "bad.pt")
    torch.save({"model": {"a": 1}}, bad)
    with pytest.raises(ValueError):
        C.load_model_state([bad])
