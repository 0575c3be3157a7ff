"""State-dict level ingest of the reference's checkpoints: gluing the tensor-parallel parts of
a `reshard-model_part-{r}.pt` set into the single-part state dict this decoder loads, the
inverse split, key normalisation, and the raw training form: FSDP shards
(`checkpoint_last-model_part-{r}-shard{s}.pt`) whose parameters are flat, padded slices.

Gluing rules (metaseq/distributed/stitch_fsdp_ckpt.py:203-214, 246-339):
* `qkv_proj` weight and bias: every part holds its own heads as local thirds K_r | V_r | Q_r;
  the glued tensor is cat(K_r) | cat(V_r) | cat(Q_r).  (The reference's singleton form splits
  these into k_proj / v_proj / q_proj; this decoder keeps the fused K | V | Q rows.)
* column-parallel `fc1` (weight and bias) and the token embedding: concatenated along dim 0;
* row-parallel `fc2` / `out_proj` weights: concatenated along dim 1, their biases replicated;
* LayerNorms, positional table, everything else: replicated (taken from part 0; copies that
  drifted apart are reported, as the reference does, not refused).

Flat FSDP shards (metaseq/scripts/reshard_fsdp.py:142-209; the same data-parallel
consolidation metaseq/distributed/stitch_fsdp_ckpt.py:96-109 asks of fairscale): every wrapped
module's parameters were flattened in order into one vector, cut into equal slices, one per
data-parallel rank, the short ones padded at the end; a file's "shard_metadata" lists, per
wrapped module, the flat vector's name and the names / shapes / element counts inside it and
that file's padding.  Undoing it: drop each slice's padding, join the slices in shard order, cut at
the element counts, reshape; buffers come from shard 0; shared parameters are aliases.

Only tensors are read from files: `torch.load(..., weights_only=True)` executes nothing from the
pickle, so a file whose "cfg" entry holds arbitrary Python objects is refused by the loader;
re-save such a file as {"model": state_dict} with the reference's own tools first.
"""
import logging
import re
from collections import OrderedDict
from typing import Dict, List

import torch

logger = logging.getLogger(__name__)

_DROP = ("decoder.output_projection.weight",)


def _agree(parts, key, tolerance=None):
    """Replicated parameter: part 0's copy is taken.  Copies that drifted apart (tensor-parallel
    training does not keep them bit-identical) are reported with their largest absolute
    difference, as the reference does (metaseq/distributed/stitch_fsdp_ckpt.py:253-262, which
    only logs).  Only a shape mismatch, or a difference above an explicitly given ``tolerance``,
    is an error."""
    ref = parts[0][key]
    worst = 0.0
    for r, p in enumerate(parts[1:], start=1):
        if p[key].shape != ref.shape:
            raise ValueError("replicated parameter %s has shape %s in part %d but %s in part 0"
                             % (key, tuple(p[key].shape), r, tuple(ref.shape)))
        if not torch.equal(p[key], ref):
            worst = max(worst, float((p[key].float() - ref.float()).abs().max()))
    if worst > 0.0:
        if tolerance is not None and worst > tolerance:
            raise ValueError("replicated parameter %s differs between model parts by %g "
                             "(tolerance %g)" % (key, worst, tolerance))
        logger.warning("replicated parameter %s differs between model parts by up to %g; "
                       "taking part 0", key, worst)
    return ref.clone()


def glue_model_parts(parts: List[Dict[str, torch.Tensor]],
                     replica_tolerance=None) -> "OrderedDict[str, torch.Tensor]":
    """Tensor-parallel parts (rank order) -> one state dict with fused K | V | Q rows.
    ``replica_tolerance``: largest absolute difference accepted between the parts' copies of a
    replicated parameter (None: any difference is only reported)."""
    if not parts:
        raise ValueError("no model parts")
    keys = list(parts[0].keys())
    for p in parts[1:]:
        if list(p.keys()) != keys:
            raise ValueError("model parts hold different parameter names")
    out = OrderedDict()
    for key in keys:
        ts = [p[key] for p in parts]
        if "qkv" in key:
            thirds = [t.split(t.shape[0] // 3, dim=0) for t in ts]
            out[key] = torch.cat([torch.cat([th[j] for th in thirds], dim=0) for j in range(3)],
                                 dim=0)
        elif "layer_norm" in key:
            out[key] = _agree(parts, key, replica_tolerance)
        elif "fc1" in key or re.search(r"\.(k|v|q)_proj\.", key):
            out[key] = torch.cat(ts, dim=0)
        elif "fc2" in key or "out_proj" in key:
            out[key] = (_agree(parts, key, replica_tolerance) if key.endswith("bias")
                        else torch.cat(ts, dim=1))
        elif "embed_tokens.weight" in key:
            out[key] = torch.cat(ts, dim=0)
        elif "_float_tensor" in key or "version" in key:
            out[key] = ts[0].clone()
        else:
            out[key] = _agree(parts, key, replica_tolerance)
    return out


def split_model_parts(state: Dict[str, torch.Tensor], n: int) -> List["OrderedDict[str, torch.Tensor]"]:
    """Inverse of glue_model_parts: the parts `n` tensor-parallel ranks would hold."""
    parts = [OrderedDict() for _ in range(n)]
    for key, t in state.items():
        if "qkv" in key:
            thirds = [th.chunk(n, dim=0) for th in t.split(t.shape[0] // 3, dim=0)]
            for r in range(n):
                parts[r][key] = torch.cat([thirds[j][r] for j in range(3)], dim=0).clone()
        elif "layer_norm" in key:
            for r in range(n):
                parts[r][key] = t.clone()
        elif "fc1" in key or "embed_tokens.weight" in key or re.search(r"\.(k|v|q)_proj\.", key):
            for r, c in enumerate(t.chunk(n, dim=0)):
                parts[r][key] = c.clone()
        elif ("fc2" in key or "out_proj" in key) and key.endswith("weight"):
            for r, c in enumerate(t.chunk(n, dim=1)):
                parts[r][key] = c.clone()
        else:
            for r in range(n):
                parts[r][key] = t.clone()
    return parts


def normalize_state_dict(state: Dict[str, torch.Tensor]) -> "OrderedDict[str, torch.Tensor]":
    """Drops what the decoder re-creates itself (the tied `decoder.output_projection.weight`:
    metaseq/checkpoint_utils.py:599-602, scripts/convert_to_singleton.py:160-166; sinusoidal
    `_float_tensor` buffers) and fuses a
    singleton checkpoint's k_proj / v_proj / q_proj back into `qkv_proj` rows K | V | Q."""
    out = OrderedDict()
    for key, t in state.items():
        if key in _DROP or key.endswith("_float_tensor"):
            continue
        m = re.match(r"(.*\.self_attn\.)k_proj\.(weight|bias)$", key)
        if m:
            pre, kind = m.groups()
            out[pre + "qkv_proj." + kind] = torch.cat(
                [state[pre + "%s_proj.%s" % (n, kind)] for n in "kvq"], dim=0)
            continue
        if re.match(r".*\.self_attn\.(v|q)_proj\.(weight|bias)$", key):
            continue
        out[key] = t
    return out


def load_model_state(paths: List[str]) -> "OrderedDict[str, torch.Tensor]":
    """Reads the tensor-parallel parts of one checkpoint (paths in rank order, e.g.
    reshard-model_part-0.pt, reshard-model_part-1.pt), glues and normalises them.  Each file is
    either a bare state dict or {"model": state_dict, ...} (metaseq/checkpoint_utils.py:540-557)."""
    parts = []
    for path in paths:
        obj = torch.load(path, map_location="cpu", weights_only=True)
        if isinstance(obj, dict) and "model" in obj and isinstance(obj["model"], dict):
            obj = obj["model"]
        if not isinstance(obj, dict) or not all(torch.is_tensor(v) for v in obj.values()):
            raise ValueError("%s does not hold a state dict of tensors" % path)
        parts.append(obj)
    return normalize_state_dict(glue_model_parts(parts) if len(parts) > 1 else parts[0])


_WRAPPER_PREFIXES = ("_fsdp_wrapped_module.", "_fpw_module.")


def _join(path, name):
    full = path + "." + name if path else name
    for w in _WRAPPER_PREFIXES:
        full = full.replace(w, "")
    return full


def unflatten_fsdp_shards(shards: List[dict]) -> "OrderedDict[str, torch.Tensor]":
    """The data-parallel shards of one model part (shard order; each
    {"model": flat slices, "shard_metadata": ...}) -> that part's state dict with named, shaped
    parameters.  Refuses slices whose joined length does not match the recorded element counts."""
    if not shards:
        raise ValueError("no shards")
    for s in shards:
        if "model" not in s or "shard_metadata" not in s:
            raise ValueError("an FSDP shard holds 'model' and 'shard_metadata'")
    layout = shards[0]["shard_metadata"]
    out = OrderedDict()
    for idx, group in enumerate(layout["param_metadata"]):
        path = group["fsdp_path"]
        for flat_name, info in group["params"].items():
            key = path + "." + flat_name if path else flat_name
            pieces = []
            for r, s in enumerate(shards):
                if key not in s["model"]:
                    raise KeyError("shard %d holds no flat parameter %s" % (r, key))
                piece = s["model"][key].reshape(-1)
                pad = int(s["shard_metadata"]["param_metadata"][idx]["params"][flat_name]["padding"])
                if pad < 0 or pad > piece.numel():
                    raise ValueError("shard %d: padding %d of %s exceeds its %d elements"
                                     % (r, pad, key, piece.numel()))
                pieces.append(piece[:piece.numel() - pad])
            flat = torch.cat(pieces)
            numels = [int(n) for n in info["numels"]]
            if sum(numels) != flat.numel():
                raise ValueError("%s: shards join to %d elements, metadata lists %d"
                                 % (key, flat.numel(), sum(numels)))
            for name, shape, t in zip(info["names"], info["shapes"], flat.split(numels)):
                out[_join(path, name)] = t.view(tuple(shape)).clone()
    for src, dest in layout.get("shared_param_info", []) or []:
        out[_join("", dest)] = out[_join("", src)]
    for name in layout.get("buffer_names", []) or []:
        if name not in shards[0]["model"]:
            raise KeyError("shard 0 holds no buffer %s" % name)
        out[_join("", name)] = shards[0]["model"][name].clone()
    return out


def is_flat_fsdp_shard(obj) -> bool:
    """A raw training shard: has shard metadata and no named embedding table
    (metaseq/distributed/stitch_fsdp_ckpt.py:84-93 tells the two forms apart the same way)."""
    return (isinstance(obj, dict) and isinstance(obj.get("model"), dict)
            and "shard_metadata" in obj and "decoder.embed_tokens.weight" not in obj["model"])


def group_fsdp_files(names: List[str]) -> List[List[str]]:
    """File names of one raw checkpoint -> [model part][shard], both in numeric order
    (`...-model_part-{r}-shard{s}.pt`; no `model_part` in the names means one part).  Every part
    must hold the same shard numbers 0..n-1."""
    table = {}
    for n in names:
        s = re.search(r"shard(\d+)\.pt$", n)
        if s is None:
            raise ValueError("%s is not named ...shard<N>.pt" % n)
        p = re.search(r"-model_part-(\d+)", n)
        table.setdefault(int(p.group(1)) if p else 0, {})[int(s.group(1))] = n
    parts = sorted(table)
    if parts != list(range(len(parts))):
        raise ValueError("model parts are not numbered 0..%d" % (len(parts) - 1))
    width = len(table[0])
    grouped = []
    for r in parts:
        if sorted(table[r]) != list(range(width)):
            raise ValueError("model part %d does not hold shards 0..%d" % (r, width - 1))
        grouped.append([table[r][i] for i in range(width)])
    return grouped


def load_fsdp_checkpoint(paths: List[str]) -> "OrderedDict[str, torch.Tensor]":
    """Reads a raw training checkpoint (every `-model_part-{r}-shard{s}.pt` file of it, any
    order): consolidates each part's data-parallel shards, glues the parts, normalises.  Files
    that already hold named parameters (training without flattening) are taken as they are, one
    per part, as metaseq/distributed/stitch_fsdp_ckpt.py:84-93,114-115 does."""
    states = []
    for files in group_fsdp_files(list(paths)):
        shards = [torch.load(f, map_location="cpu", weights_only=True) for f in files]
        if is_flat_fsdp_shard(shards[0]):
            states.append(unflatten_fsdp_shards(shards))
        else:
            first = shards[0]
            states.append(first["model"] if "model" in first else first)
    return normalize_state_dict(glue_model_parts(states) if len(states) > 1 else states[0])


# ---------------------------------------------------------------- offline int8 weights
_QUANTIZED = re.compile(r"^(decoder\.)?layers\.\d+\.(self_attn\.qkv_proj|self_attn\.out_proj|fc1|fc2)"
                        r"\.weight$")


def quantize_rows(w: torch.Tensor):
    """Symmetric int8 per output row of a [out, in] matrix: scale_j = fp16(max_i |w_ji| / 127),
    q_ji = clamp(rint(w_ji / scale_j), -127, 127) in fp32 arithmetic - the weight-only form the
    reference asks of its serving backend for these matrices
    (metaseq/scripts/convert_metaseq_ft.py:99-133).  Runs wherever ``w`` lives, with the same
    result on the CPU and on the GPU (every step is one correctly rounded operation)."""
    wf = w.float()
    scales = (wf.abs().amax(dim=1) / 127.0).to(torch.float16)
    s = scales.float().clamp_min(1e-30).unsqueeze(1)
    q = torch.clamp(torch.round(wf / s), -127, 127).to(torch.int8)
    return q.contiguous(), scales.contiguous()


def quantize_state_dict(state: Dict[str, torch.Tensor]) -> "OrderedDict[str, torch.Tensor]":
    """The offline step of int8 serving: every per-layer qkv_proj / out_proj / fc1 / fc2
    ``<name>.weight`` of a reference-named state dict becomes ``<name>.qweight`` (int8 [out, in],
    row-major) and ``<name>.scales`` (fp16 [out]); everything else is passed through.  The
    result is what ``TransformerDecoder.load_state_dict`` / ``load_tensors`` take in place of
    fp16 weights, so a served model never has to hold (or read) the fp16 matrices; it needs no
    GPU and can be saved with ``torch.save``."""
    out = OrderedDict()
    for k, v in state.items():
        if _QUANTIZED.match(k):
            stem = k[:-len("weight")]
            out[stem + "qweight"], out[stem + "scales"] = quantize_rows(v)
        else:
            out[k] = v
    return out


def is_quantized_state(state) -> bool:
    return any(k.endswith(".qweight") for k in state)


def find_model_parts(names: List[str]) -> List[str]:
    """Sorts file names of one checkpoint by their `-model_part-{r}` number
    (metaseq/distributed/stitch_fsdp_ckpt.py:342-352) and checks that no rank is missing."""
    numbered = []
    for n in names:
        m = re.search(r"-model_part-(\d+)", n)
        if m is not None:
            numbered.append((int(m.group(1)), n))
    numbered.sort()
    if [r for r, _ in numbered] != list(range(len(numbered))):
        raise ValueError("model parts are not numbered 0..%d" % (len(numbered) - 1))
    return [n for _, n in numbered]
