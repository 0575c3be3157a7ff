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


# --- raw training checkpoints: flat, padded FSDP shards ------------------------------------
#
# The reference has no test or fixture for this form ("parity unpinned" by the reference); what
# pins the consolidation is the sharding it undoes, written out here the way fairscale's FSDP
# defines it (flatten the wrapped module's parameters in order, `chunk` over the data-parallel
# ranks, pad every short or missing slice at the end to the first slice's length) and the
# requirement that undoing it returns every parameter bit for bit.

def _fsdp_shard(state, groups, world, buffers=(), shared=()):
    """state dict -> `world` shard dicts.  groups: [(fsdp_path, [names relative to it])]."""
    import torch.nn.functional as F
    shards = [{"model": {}, "shard_metadata": {"param_metadata": [], "buffer_names": list(buffers),
                                                "shared_param_info": list(shared)}}
              for _ in range(world)]
    for path, names in groups:
        full = [(path + "." + n) if path else n for n in names]
        flat = torch.cat([state[k].reshape(-1) for k in full])
        chunks = list(flat.chunk(world))
        size = chunks[0].numel()
        key = (path + "." if path else "") + "flat_param_0"
        for r in range(world):
            c = chunks[r] if r < len(chunks) else flat.new_empty(0)
            pad = size - c.numel()
            shards[r]["model"][key] = F.pad(c, [0, pad]).clone()
            shards[r]["shard_metadata"]["param_metadata"].append({
                "fsdp_path": path,
                "params": {"flat_param_0": {"names": list(names),
                                            "shapes": [state[k].shape for k in full],
                                            "numels": [state[k].numel() for k in full],
                                            "padding": pad}}})
    for r in range(world):
        for b in buffers:
            shards[r]["model"][b] = state[b].clone()
    return shards


def _fsdp_groups(state, shared=()):
    skip = {"decoder.version"} | {d for _, d in shared}
    groups = []
    for i in range(L):
        p = "decoder.layers.%d" % i
        groups.append((p, [k[len(p) + 1:] for k in state if k.startswith(p + ".")]))
    rest = [k for k in state if not k.startswith("decoder.layers.") and k not in skip]
    groups.append(("", rest))
    return groups


@pytest.mark.parametrize("world", [1, 2, 3, 7])
def test_flat_fsdp_shards_consolidate_to_the_sharded_state(world):
    [sd] = _parts(1, seed=5)
    sd["decoder.output_projection.weight"] = sd["decoder.embed_tokens.weight"]
    shared = [("decoder.embed_tokens.weight", "decoder.output_projection.weight")]
    shards = _fsdp_shard(sd, _fsdp_groups(sd, shared), world, buffers=["decoder.version"],
                         shared=shared)
    if world == 7:   # slices really are padded, and unevenly named parameters straddle them
        assert any(g["params"]["flat_param_0"]["padding"] > 0
                   for g in shards[-1]["shard_metadata"]["param_metadata"])
    back = C.unflatten_fsdp_shards(shards)
    assert set(back) == set(sd)
    for k in sd:
        assert back[k].shape == sd[k].shape and torch.equal(back[k], sd[k]), k


def test_flat_fsdp_more_ranks_than_elements_leaves_empty_all_padding_slices():
    sd = {"a.w": torch.arange(3.0), "a.b": torch.arange(2.0) + 10}
    shards = _fsdp_shard(sd, [("a", ["w", "b"])], 8)
    assert shards[7]["shard_metadata"]["param_metadata"][0]["params"]["flat_param_0"]["padding"] == 1
    back = C.unflatten_fsdp_shards(shards)
    assert torch.equal(back["a.w"], sd["a.w"]) and torch.equal(back["a.b"], sd["a.b"])


def test_flat_fsdp_refuses_lengths_that_do_not_add_up_and_missing_vectors():
    sd = {"a.w": torch.arange(6.0).view(2, 3)}
    shards = _fsdp_shard(sd, [("a", ["w"])], 2)
    shards[1]["shard_metadata"]["param_metadata"][0]["params"]["flat_param_0"]["padding"] = 1
    with pytest.raises(ValueError, match="join to 5 elements, metadata lists 6"):
        C.unflatten_fsdp_shards(shards)
    shards = _fsdp_shard(sd, [("a", ["w"])], 2)
    del shards[1]["model"]["a.flat_param_0"]
    with pytest.raises(KeyError, match="shard 1 holds no flat parameter"):
        C.unflatten_fsdp_shards(shards)


def test_wrapper_prefixes_are_dropped_from_names():
    sd = {"m.w": torch.arange(4.0)}
    shards = _fsdp_shard(sd, [("m", ["w"])], 2)
    for s in shards:
        s["shard_metadata"]["param_metadata"][0]["params"]["flat_param_0"]["names"] = [
            "_fsdp_wrapped_module._fpw_module.w"]
    assert list(C.unflatten_fsdp_shards(shards)) == ["m.w"]


def test_raw_checkpoint_files_two_parts_three_shards_give_the_glued_models_logits(tmp_path):
    """File level: `-model_part-{r}-shard{s}.pt` of two tensor-parallel parts, each cut into
    three data-parallel shards, listed out of order -> the state dict of the glued model."""
    parts = _parts(2, seed=9)
    names = []
    for r, sd in enumerate(parts):
        for s, shard in enumerate(_fsdp_shard(sd, _fsdp_groups(sd), 3, buffers=["decoder.version"])):
            f = tmp_path / ("checkpoint_last-model_part-%d-shard%d.pt" % (r, s))
            torch.save(shard, f)
            names.append(str(f))
    loaded = C.load_fsdp_checkpoint(names[::-1])
    glued = C.normalize_state_dict(C.glue_model_parts(parts))
    assert set(loaded) == set(glued)
    for k in glued:
        assert torch.equal(loaded[k], glued[k]), k
    assert torch.allclose(_single_logits(loaded, TOKENS), tp_forward(parts, TOKENS, H), atol=1e-5)


def test_raw_checkpoint_grouping_checks_numbering(tmp_path):
    assert C.group_fsdp_files(["c-shard1.pt", "c-shard0.pt", "c-shard10.pt"][:2]) == [
        ["c-shard0.pt", "c-shard1.pt"]]
    with pytest.raises(ValueError, match="does not hold shards"):
        C.group_fsdp_files(["c-model_part-0-shard0.pt", "c-model_part-0-shard1.pt",
                            "c-model_part-1-shard0.pt", "c-model_part-1-shard2.pt"])
    with pytest.raises(ValueError, match="not numbered"):
        C.group_fsdp_files(["c-model_part-1-shard0.pt"])
    with pytest.raises(ValueError, match="not named"):
        C.group_fsdp_files(["reshard-model_part-0.pt"])


def test_unflattened_training_files_are_taken_as_they_are(tmp_path):
    parts = _parts(2, seed=11)
    names = []
    for r, sd in enumerate(parts):
        f = tmp_path / ("checkpoint_last-model_part-%d-shard0.pt" % r)
        torch.save({"model": sd, "shard_metadata": {"param_metadata": []}}, f)
        names.append(str(f))
    loaded = C.load_fsdp_checkpoint(names)
    glued = C.normalize_state_dict(C.glue_model_parts(parts))
    assert all(torch.equal(loaded[k], glued[k]) for k in glued)
