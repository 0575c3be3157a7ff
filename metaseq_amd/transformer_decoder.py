"""OPT decoder forward on hand-written gfx950 kernels, behind the interface of the
reference's ``ModelParallelTransformerDecoder`` (metaseq/models/transformer_decoder.py:62-537)
at tensor-parallel size 1: same ``forward`` signature, same prefill/decode switch (an empty
``incremental_state`` dict means prefill, a non-empty one a single-token step), same
parameter names in ``state_dict()``.

All arithmetic runs in libmetaseq_amd.so through the C ABI; torch only owns the device
memory and the stream.  There is no eager fallback.
"""
import ctypes
import uuid
from typing import Any, Dict, Optional

import torch
from torch import nn

from . import _capi
from ._capi import (MSA_EMBED_COL_FROM_LEN, MSA_EMBED_ROWS_GIVEN, MSA_EPI_RELU, MSA_IN_PACKED,
                    MSA_OUT_PACKED, check, ptr)
from .checkpoint_utils import quantize_rows
from .config import OPTConfig
from .kv_cache import KVCache


def upload(values, dtype, device):
    """A short host list as a device tensor without a blocking copy: through pinned memory and
    stream-ordered.  (A copy from pageable memory makes the host wait for everything queued
    ahead of it - a whole decode step - and leaves the GPU idle while the host goes on.)"""
    t = torch.tensor(values, dtype=dtype)
    if torch.device(device).type != "cuda":
        return t.to(device)
    return t.pin_memory().to(device, non_blocking=True)


class _Affine(nn.Module):
    """weight + bias holder (Linear or LayerNorm parameters under the reference's names).

    For a linear layer, ``prepare_`` converts ``weight`` in place to the tile-packed layout the
    kernels stream (same shape and bytes, permuted), or to packed int8 + fp16 scales."""

    def __init__(self, w_shape, b_shape, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(w_shape, dtype=torch.float16, device=device),
                                   requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(b_shape, dtype=torch.float16, device=device),
                                 requires_grad=False)
        self.packed = False
        self.qweight: Optional[torch.Tensor] = None  # tile-packed int8
        self.scales: Optional[torch.Tensor] = None
        self.shape = tuple(w_shape)

    def prepare_(self, lib, int8=False):
        if self.packed or self.qweight is not None:
            return
        N, K = self.shape
        w = self.weight.data
        if int8:
            self.adopt_int8_(lib, *quantize_rows(w))
        else:
            wp = torch.empty_like(w)
            check(lib.msa_pack_weight_f16(ptr(w), ptr(wp), N, K, _capi.stream_ptr()))
            self.weight.data = wp
            self.packed = True

    def adopt_int8_(self, lib, q, scales):
        """Takes already quantised weights (int8 [N, K] row-major, fp16 [N] scales), packs them
        for the kernels and frees the fp16 matrix."""
        N, K = self.shape
        dev = self.bias.device
        if tuple(q.shape) != (N, K) or q.dtype != torch.int8:
            raise ValueError("int8 weight: expected int8 %s, got %s %s"
                             % ((N, K), q.dtype, tuple(q.shape)))
        if tuple(scales.shape) != (N,):
            raise ValueError("int8 scales: expected %s, got %s" % ((N,), tuple(scales.shape)))
        q = q.to(dev).contiguous()
        qp = torch.empty_like(q)
        check(lib.msa_pack_weight_i8(ptr(q), ptr(qp), N, K, _capi.stream_ptr()))
        self.qweight = qp
        self.scales = scales.to(device=dev, dtype=torch.float16).contiguous()
        self.weight.data = torch.empty(0, dtype=torch.float16, device=dev)
        self.packed = False

    def row_major_int8(self, lib):
        """(int8 [N, K] row-major, fp16 [N] scales) of a quantised matrix."""
        N, K = self.shape
        q = torch.empty_like(self.qweight)
        check(lib.msa_unpack_weight_i8(ptr(self.qweight), ptr(q), N, K, _capi.stream_ptr()))
        return q, self.scales

    def row_major_weight(self, lib):
        """fp16 [N, K] row-major weight (for int8: the dequantised round(q * scale))."""
        N, K = self.shape
        if self.qweight is not None:
            q, scales = self.row_major_int8(lib)
            return (q.float() * scales.float().unsqueeze(1)).to(torch.float16)
        if not self.packed:
            return self.weight.data
        w = torch.empty_like(self.weight.data)
        check(lib.msa_unpack_weight_f16(ptr(self.weight.data), ptr(w), N, K, _capi.stream_ptr()))
        return w


class _Table(nn.Module):
    def __init__(self, rows, dim, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(rows, dim, dtype=torch.float16, device=device),
                                   requires_grad=False)


class _SelfAttention(nn.Module):
    def __init__(self, D, device=None):
        super().__init__()
        self.qkv_proj = _Affine((3 * D, D), (3 * D,), device)  # rows K | V | Q
        self.out_proj = _Affine((D, D), (D,), device)


class _DecoderLayer(nn.Module):
    def __init__(self, D, F, device=None):
        super().__init__()
        self.self_attn_layer_norm = _Affine((D,), (D,), device)
        self.self_attn = _SelfAttention(D, device)
        self.final_layer_norm = _Affine((D,), (D,), device)
        self.fc1 = _Affine((F, D), (F,), device)
        self.fc2 = _Affine((D, F), (D,), device)


class TransformerDecoder(nn.Module):
    """Drop-in for the reference decoder on the generation path.

    ``forward(prev_output_tokens, incremental_state)`` returns ``(logits[B, T, V], extra)``
    with ``T = n`` for prefill (``incremental_state`` None or empty) and ``T = 1`` for a decode
    step, mutating the caller's dict in place so that it is non-empty after the prefill.
    """

    def __init__(self, cfg: OPTConfig, state_dict: Optional[Dict[str, torch.Tensor]] = None,
                 device="cuda"):
        super().__init__()
        cfg.require_supported_head_dim()
        self.cfg = cfg
        self.args = cfg  # the reference exposes its namespace as .args
        D, F = cfg.decoder_embed_dim, cfg.decoder_ffn_embed_dim
        self.padding_idx = cfg.padding_idx
        self.max_target_positions = cfg.max_target_positions
        self.share_input_output_embed = True
        self.embed_scale = 1.0
        self.register_buffer("version", torch.tensor([3.0]))
        self.embed_tokens = _Table(cfg.vocab_size, D, device)
        self.embed_positions = _Table(cfg.max_target_positions + cfg.padding_idx + 1, D, device)
        self.layers = nn.ModuleList([_DecoderLayer(D, F, device)
                                     for _ in range(cfg.decoder_layers)])
        self.layer_norm = _Affine((D,), (D,), device)
        self.inference = True
        self.return_inner_states = False
        # instrumentation: called as layer_probe(i, x) with the residual stream [B * T, D] after
        # layer i of a pass over row-major activations (prefill); the tensor is overwritten by
        # the next layer, so a probe that keeps it must copy
        self.layer_probe = None
        # decode steps of at most 128 rows go through msa_decoder_step (one C call per token);
        # False drives the same kernels entry point by entry point from Python
        self.native_step = True
        self._native = None  # (handle, keep-alive references)
        # capacity (positions) of the KV cache the next prefill allocates; None = grow on demand
        self.kv_cache_capacity: Optional[int] = None
        self._state_key = str(uuid.uuid4()) + ".kv_cache"
        self._lib = None
        self._lm_head: Optional[torch.Tensor] = None  # tile-packed copy of the tied embedding
        self._w8_scratch: Optional[torch.Tensor] = None  # one int8 matrix expanded to fp16
        self.to(device)
        if state_dict is not None:
            self.load_state_dict(state_dict)

    # ------------------------------------------------------------------ weights
    def _linears(self):
        for i, layer in enumerate(self.layers):
            yield f"layers.{i}.self_attn.qkv_proj", layer.self_attn.qkv_proj
            yield f"layers.{i}.self_attn.out_proj", layer.self_attn.out_proj
            yield f"layers.{i}.fc1", layer.fc1
            yield f"layers.{i}.fc2", layer.fc2

    def load_state_dict(self, state_dict, strict=True, **kw):
        sd = dict(state_dict)
        # accept a model-level dict ("decoder." prefix) and the tied duplicate key
        if any(k.startswith("decoder.") for k in sd):
            sd = {k[len("decoder."):]: v for k, v in sd.items() if k.startswith("decoder.")}
        sd.pop("output_projection.weight", None)
        # the format marker is optional, as in the reference's upgrade_state_dict_named
        # (metaseq/models/transformer_decoder.py:539-567)
        sd.setdefault("version", torch.tensor([3.0]))
        for _, lin in self._linears():  # back to plain row-major parameters before loading
            if lin.packed or lin.qweight is not None:
                lin.weight.data = torch.empty(lin.shape, dtype=torch.float16,
                                              device=lin.bias.device)
                lin.packed, lin.qweight, lin.scales = False, None, None
        self._lm_head = None
        self._drop_native()
        if any(k.endswith(".qweight") for k in sd):
            # weights quantised offline (checkpoint_utils.quantize_state_dict)
            return self.load_tensors(sd.items())
        return super().load_state_dict(sd, strict=strict, **kw)

    def load_tensors(self, named_tensors, quantize_int8=False):
        """Streaming form of ``load_state_dict`` for checkpoints that leave no room for a second
        copy: ``named_tensors`` yields (reference parameter name, tensor) pairs, each is copied
        into place and may be freed by the producer right away.  With ``quantize_int8`` every
        linear layer is quantised and packed as soon as its weight has arrived, so the fp16
        matrices never all exist at once.  A linear layer quantised offline arrives as
        ``<name>.qweight`` (int8 [out, in]) and ``<name>.scales`` (fp16 [out]) in place of
        ``<name>.weight`` (``checkpoint_utils.quantize_state_dict``) and is packed as it is.
        Every parameter must arrive exactly once."""
        lib = self._lib = self._lib or _capi.load()
        if quantize_int8:
            self.cfg.quantize_int8 = True
        own = dict(self.named_parameters())
        linears = dict(self._linears())
        for lin in linears.values():
            if lin.packed or lin.qweight is not None:
                raise RuntimeError("load_tensors needs a freshly constructed decoder")
        self._lm_head = None
        self._drop_native()
        seen = set()
        halves = {}  # linear name -> {"qweight": ..., "scales": ...} until both have arrived
        for name, t in named_tensors:
            if name.startswith("decoder."):
                name = name[len("decoder."):]
            if name in ("version", "output_projection.weight"):
                continue
            stem, _, kind = name.rpartition(".")
            if kind in ("qweight", "scales"):
                if stem not in linears:
                    raise KeyError("unexpected parameter %r" % name)
                got = halves.setdefault(stem, {})
                if kind in got or stem + ".weight" in seen:
                    raise KeyError("unexpected or repeated parameter %r" % name)
                got[kind] = t
                if len(got) == 2:
                    linears[stem].adopt_int8_(lib, got["qweight"], got["scales"])
                    halves[stem] = {"qweight": None, "scales": None}  # arrived; tensors released
                    seen.add(stem + ".weight")
                    self.cfg.quantize_int8 = True
                continue
            if name not in own or name in seen:
                raise KeyError("unexpected or repeated parameter %r" % name)
            if tuple(own[name].shape) != tuple(t.shape):
                raise ValueError("shape of %s: expected %s, got %s"
                                 % (name, tuple(own[name].shape), tuple(t.shape)))
            own[name].data.copy_(t)
            seen.add(name)
            if quantize_int8 and name.endswith(".weight") and name[:-len(".weight")] in linears:
                linears[name[:-len(".weight")]].prepare_(lib, int8=True)
        missing = sorted(set(own) - seen)
        if missing:
            raise KeyError("missing parameters: %s" % ", ".join(missing[:8]))
        if halves:
            for name, lin in linears.items():
                if lin.qweight is None:
                    raise KeyError("%s arrived in fp16 beside int8 layers; quantise all of the "
                                   "per-layer matrices or none" % name)
        return self

    def quantized_state_dict(self):
        """The int8 model as ``checkpoint_utils.quantize_state_dict`` writes it (reference
        names with a "decoder." prefix; ``.qweight`` int8 [out, in] row-major and ``.scales``
        in place of the four per-layer ``.weight``): saved with ``torch.save``, it is loaded
        again by ``load_state_dict`` / ``load_tensors`` without the fp16 matrices."""
        if not self.cfg.quantize_int8:
            raise RuntimeError("quantized_state_dict() needs an int8 model (quantize_int8_())")
        lib = self.prepare_()
        linears = dict(self._linears())
        out = {}
        for k, v in nn.Module.state_dict(self).items():
            stem = k[:-len(".weight")] if k.endswith(".weight") else None
            if stem in linears:
                out["decoder." + stem + ".qweight"], out["decoder." + stem + ".scales"] = \
                    linears[stem].row_major_int8(lib)
            else:
                out["decoder." + k] = v
        return out

    def state_dict(self, *args, **kwargs):
        """Reference-layout (row-major, fp16) state dict; quantised matrices come back as their
        dequantised values round(q * scale)."""
        sd = super().state_dict(*args, **kwargs)
        prefix = kwargs.get("prefix", args[1] if len(args) > 1 else "")
        if self._lib is not None:
            for name, lin in self._linears():
                if lin.packed or lin.qweight is not None:
                    sd[prefix + name + ".weight"] = lin.row_major_weight(self._lib)
        return sd

    def prepare_(self):
        """Packs every linear weight for the kernels (idempotent); with ``cfg.quantize_int8`` the
        four per-layer matrices become symmetric per-output-channel int8 first:
        scale_j = fp16(max_i |W_ji| / 127), q = clamp(rint(W / scale_j), -127, 127) - the
        matrices the reference quantises for serving
        (metaseq/scripts/convert_metaseq_ft.py:118-129)."""
        lib = self._lib or _capi.load()
        self._lib = lib
        if not self.embed_tokens.weight.is_cuda:
            raise RuntimeError("metaseq_amd: the model must live on the GPU (no CPU path exists)")
        for _, lin in self._linears():
            lin.prepare_(lib, int8=self.cfg.quantize_int8)
        if self._lm_head is None:
            e = self.embed_tokens.weight.data
            self._lm_head = torch.empty_like(e)
            check(lib.msa_pack_weight_f16(ptr(e), ptr(self._lm_head), e.shape[0], e.shape[1],
                                          _capi.stream_ptr()))
        return lib

    def quantize_int8_(self):
        self.cfg.quantize_int8 = True
        for _, lin in self._linears():
            if lin.packed:
                raise RuntimeError("quantize_int8_() must be called before the first forward")
        self.prepare_()
        return self

    def dequantized_state_dict(self):
        """Reference-named fp16 weights with quantised matrices replaced by round(q * scale):
        what a reference model must be loaded with to be compared against the int8 path."""
        self.prepare_()
        return {"decoder." + k: v for k, v in self.state_dict().items()}

    # ------------------------------------------------------------------ reference API
    def max_positions(self):
        """metaseq/models/transformer_decoder.py:430-434."""
        return min(self.max_target_positions,
                   self.embed_positions.weight.shape[0] - self.padding_idx - 1)

    def make_generation_fast_(self, **unused):
        self.inference = True

    def reorder_incremental_state(self, incremental_state, new_order):
        """No-op, as in the reference (metaseq/models/base_decoder.py:82-93)."""

    def get_normalized_probs(self, logits, log_probs: bool):
        """metaseq/models/base_decoder.py:95-100 (fp32 softmax over the last dimension)."""
        if isinstance(logits, (tuple, list)):
            logits = logits[0]
        if log_probs:
            return torch.log_softmax(logits, dim=-1, dtype=torch.float32)
        return torch.softmax(logits, dim=-1, dtype=torch.float32)

    def get_cache(self, incremental_state) -> Optional[KVCache]:
        if not incremental_state:
            return None
        return incremental_state.get(self._state_key)

    # ------------------------------------------------------------------ kernels
    # From this many activation rows on, an int8 weight matrix is expanded once into a scratch
    # fp16 matrix (3 bytes moved per weight) and multiplied by the fp16 kernel, which is faster
    # than dequantising every fragment in every workgroup; the values are the same.
    W8_EXPAND_ROWS = 4096

    def _expands(self, M, N):
        """Whether a product of M row-major rows with an int8 [N, K] matrix runs on the matrix
        expanded to fp16: from 4096 rows on (the expansion is small beside the product), and
        for the few hundred rows whose 256 x 256 int8 tiles would leave CUs idle, where only
        the slow 128 x 128 int8 kernel remains."""
        if M >= self.W8_EXPAND_ROWS:
            return True
        return M > self.PACKED_MAX_ROWS and ((M + 255) // 256) * ((N + 255) // 256) < 256
    # decode steps of int8 weights above 128 rows run in chunks of <= 128 rows up to here
    W8_CHUNKED_ROWS = 512

    def _expanded(self, lib, stream, lin):
        """Pointer to the scratch matrix holding ``lin``'s int8 weights expanded to packed fp16."""
        N, K = lin.shape
        if self._w8_scratch is None:
            need = max(l.shape[0] * l.shape[1] for _, l in self._linears())
            self._w8_scratch = torch.empty(need, dtype=torch.float16, device=lin.qweight.device)
        check(lib.msa_expand_weight_w8_f16(ptr(lin.qweight), ptr(lin.scales),
                                           ptr(self._w8_scratch), N, K, stream))
        return ptr(self._w8_scratch)

    def _linear(self, lib, stream, x, lin, M, N, K, bias=True, residual=None, relu=False,
                out=None, flags=0):
        y = out if out is not None else torch.empty(M, N, dtype=torch.float16, device=x.device)
        flags |= MSA_EPI_RELU if relu else 0
        b = lin.bias if bias else None
        if lin.qweight is not None and self._expands(M, N):
            check(lib.msa_linear_f16(ptr(x), self._expanded(lib, stream, lin), ptr(b),
                                     ptr(residual), ptr(y), M, N, K, flags, stream))
        elif lin.qweight is not None:
            check(lib.msa_linear_w8a16(ptr(x), ptr(lin.qweight), ptr(lin.scales), ptr(b),
                                       ptr(residual), ptr(y), M, N, K, flags, stream))
        else:
            check(lib.msa_linear_f16(ptr(x), ptr(lin.weight), ptr(b), ptr(residual), ptr(y), M, N,
                                     K, flags, stream))
        return y

    def _linear_partial(self, lib, stream, x, lin, part, M, N, K, S):
        if lin.qweight is not None:
            check(lib.msa_linear_partial_w8a16(ptr(x), ptr(lin.qweight), ptr(lin.scales),
                                               ptr(part), M, N, K, S, MSA_IN_PACKED, stream))
        else:
            check(lib.msa_linear_partial_f16(ptr(x), ptr(lin.weight), ptr(part), M, N, K, S,
                                             MSA_IN_PACKED, stream))

    def _qkv(self, lib, stream, h, qkv, q, kc, vc, B, T, H, hd, S0, cap, D, flags, len_dev=None):
        if qkv.qweight is not None and self._expands(B * T, 3 * D):
            check(lib.msa_qkv_proj_f16(ptr(h), self._expanded(lib, stream, qkv), ptr(qkv.bias),
                                       ptr(q), ptr(kc), ptr(vc), B, T, H, hd, S0, cap, D, flags,
                                       ptr(len_dev), stream))
        elif qkv.qweight is not None:
            check(lib.msa_qkv_proj_w8a16(ptr(h), ptr(qkv.qweight), ptr(qkv.scales), ptr(qkv.bias),
                                         ptr(q), ptr(kc), ptr(vc), B, T, H, hd, S0, cap, D, flags,
                                         ptr(len_dev), stream))
        else:
            check(lib.msa_qkv_proj_f16(ptr(h), ptr(qkv.weight), ptr(qkv.bias), ptr(q), ptr(kc),
                                       ptr(vc), B, T, H, hd, S0, cap, D, flags, ptr(len_dev),
                                       stream))

    def __del__(self):
        self._drop_native()

    def _apply(self, fn, *args, **kwargs):
        self._drop_native()  # .to() / .half() move the tensors the handle points at
        self.__dict__["_w8_scratch"] = None  # re-created on the device the weights end up on
        return super()._apply(fn, *args, **kwargs)

    def _drop_native(self):
        native = self.__dict__.get("_native")
        lib = self.__dict__.get("_lib")
        if native is not None and lib is not None:
            lib.msa_decoder_destroy(native[0])
        self.__dict__["_native"] = None

    def _native_handle(self, lib):
        """The msa_decoder handle over this model's packed weights (created on first use; the
        table holds raw device pointers, so it is rebuilt when the weights are reloaded)."""
        if self._native is None:
            cfg = self.cfg
            int8 = self.layers[0].fc2.qweight is not None
            conf = _capi.DecoderConfig(cfg.decoder_layers, cfg.decoder_embed_dim,
                                       cfg.decoder_attention_heads, cfg.decoder_ffn_embed_dim,
                                       cfg.vocab_size, self.embed_positions.weight.shape[0],
                                       self.padding_idx, int(int8))
            table = (_capi.LayerWeights * cfg.decoder_layers)()
            for i, layer in enumerate(self.layers):
                t = table[i]
                t.ln1_gamma = layer.self_attn_layer_norm.weight.data_ptr()
                t.ln1_beta = layer.self_attn_layer_norm.bias.data_ptr()
                t.ln2_gamma = layer.final_layer_norm.weight.data_ptr()
                t.ln2_beta = layer.final_layer_norm.bias.data_ptr()
                for name, lin in (("qkv", layer.self_attn.qkv_proj),
                                  ("out", layer.self_attn.out_proj), ("fc1", layer.fc1),
                                  ("fc2", layer.fc2)):
                    w = lin.qweight if int8 else lin.weight
                    setattr(t, name + "_weight", w.data_ptr())
                    setattr(t, name + "_scales", lin.scales.data_ptr() if int8 else None)
                    setattr(t, name + "_bias", lin.bias.data_ptr())
            handle = ctypes.c_void_p()
            check(lib.msa_decoder_create(ctypes.byref(conf), ptr(self.embed_tokens.weight),
                                         ptr(self.embed_positions.weight), ptr(self._lm_head),
                                         ptr(self.layer_norm.weight), ptr(self.layer_norm.bias),
                                         table, ctypes.byref(handle)))
            self._native = (handle, table)
        return self._native[0]

    def _native_step(self, lib, stream, tokens, n, B, cache, mask, len_dev, S0, out,
                     col_from_len=False, advance=True):
        """One decode step through msa_decoder_step.  ``out``: dict with ``logits`` ([B, V] fp16
        tensor or None) and / or ``select`` (the keyword arguments of ``_select_from``)."""
        handle = self._native_handle(lib)
        ws = getattr(cache, "native_ws", None)
        need = lib.msa_decoder_step_workspace_bytes(handle, B)
        if ws is None or ws.numel() < need:
            ws = cache.native_ws = torch.empty(need, dtype=torch.uint8, device=cache.device)
            L = self.cfg.decoder_layers
            cache.native_kv = ((ctypes.c_void_p * L)(*[cache.k(i).data_ptr() for i in range(L)]),
                               (ctypes.c_void_p * L)(*[cache.v(i).data_ptr() for i in range(L)]),
                               cache.capacity)
        if cache.native_kv[2] != cache.capacity:  # the cache was re-allocated (grown)
            L = self.cfg.decoder_layers
            cache.native_kv = ((ctypes.c_void_p * L)(*[cache.k(i).data_ptr() for i in range(L)]),
                               (ctypes.c_void_p * L)(*[cache.v(i).data_ptr() for i in range(L)]),
                               cache.capacity)
        a = _capi.StepArgs()
        a.tokens, a.tok_stride, a.n, a.B = tokens.data_ptr(), tokens.stride(0), n, B
        a.k_cache, a.v_cache = cache.native_kv[0], cache.native_kv[1]
        a.S0, a.S_cap = S0, cache.capacity
        a.len_dev = ptr(len_dev)
        a.key_pad_mask = ptr(mask)
        a.mask_stride = mask.stride(0) if mask is not None else 0
        a.flags = ((MSA_EMBED_COL_FROM_LEN if col_from_len else 0)
                   | (0 if advance else _capi.MSA_STEP_NO_ADVANCE))
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        a.logits = ptr(out.get("logits"))
        sel = out.get("select")
        keep = None
        if sel is not None:
            banned, stop = list(sel["banned"]), list(sel["stop"])
            ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
            sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
            keep = (ba, sa)
            a.tok, a.tok_stride_out = ptr(sel["tok_out"]), sel["tok_stride"]
            a.score, a.score_stride = ptr(sel["score_out"]), sel["score_stride"]
            a.temperature = float(sel["temperature"])
            a.banned, a.n_banned, a.stop, a.n_stop = ba, len(banned), sa, len(stop)
            a.finished, a.row_mode = ptr(sel.get("finished")), ptr(sel.get("row_mode"))
            a.force_eos_all, a.eos_idx = int(sel["force_eos"]), int(sel["eos"])
        check(lib.msa_decoder_step(handle, ctypes.byref(a), stream))
        del keep

    # most rows of a decode step on packed activations (the library's MSA_PACKED_MAX_ROWS)
    PACKED_MAX_ROWS = 128
    SLOT_MAX_ROWS = 256     # rows of a slot cache (continuous batching)

    @staticmethod
    def _packed_rows(B):
        """Rows the packed activation buffers of a B-row step hold: whole blocks of 16 up to 64
        rows, 128 beyond (one kernel shape serves 65 .. 128 rows)."""
        return ((B + 15) // 16) * 16 if B <= 64 else 128

    def _step_buffers(self, cache, B):
        """Work buffers of a decode step (<= 128 rows), allocated once per KV cache so that their
        addresses stay fixed (a captured graph replays against them)."""
        bufs = getattr(cache, "step_bufs", None)
        if bufs is None:
            cfg, dev = self.cfg, cache.device
            D, F = cfg.decoder_embed_dim, cfg.decoder_ffn_embed_dim
            MP = self._packed_rows(B)
            lib = self._lib
            int8 = self.layers[0].fc2.qweight is not None
            splits = lib.msa_linear_default_splits_w8a16 if int8 else lib.msa_linear_default_splits
            S_o, S_f = splits(B, D, D), splits(B, D, F)
            f16 = dict(dtype=torch.float16, device=dev)
            bufs = {
                "x": torch.empty(B, D, **f16), "q": torch.empty(B, D, **f16),
                "h": torch.empty(MP * D, **f16), "o": torch.empty(MP * D, **f16),
                "u": torch.empty(MP * F, **f16), "feat": torch.empty(B, D, **f16),
                "part": torch.empty(max(S_o, S_f) * B * D, dtype=torch.float32, device=dev),
                "positions": torch.empty(B, 1, dtype=torch.long, device=dev),
                "step_len": torch.empty(B, dtype=torch.int32, device=dev),
                "S_o": S_o, "S_f": S_f,
            }
            cache.step_bufs = bufs
        return bufs

    def _decode_core(self, lib, stream, tokens, n, B, cache, mask, bufs, len_dev, S0,
                     want_packed, col_from_len=False, token_embeddings=None):
        """One decode step for at most 128 rows: packed activations, weight-streaming kernels,
        split-K tails fused into the LayerNorm that follows.  With ``len_dev`` (int32 [B] device
        tensor: positions of each row already in the cache, negative = inactive row) every row
        appends at and attends up to its own length, and nothing in the launch arguments
        depends on the step, so the sequence can be captured once and replayed.  The new tokens
        are the last column of ``tokens`` (or column ``len_dev[b]`` with ``col_from_len``)."""
        cfg = self.cfg
        D, L, M = cfg.decoder_embed_dim, cfg.decoder_layers, B
        x, h = bufs["x"], bufs["h"]
        OUT = MSA_OUT_PACKED
        # a row whose new token is a pad sits this step out (step_len = -1), as does an
        # inactive row; under graph replay there are no pads and the lengths are used as is
        step_len = bufs["step_len"] if (len_dev is not None and not col_from_len) else None
        table = self.embed_tokens.weight if token_embeddings is None else token_embeddings
        check(lib.msa_embed_f16(ptr(tokens), tokens.stride(0), B, n, 1, ptr(table),
                                cfg.vocab_size, ptr(self.embed_positions.weight),
                                self.embed_positions.weight.shape[0], self.padding_idx, D,
                                ptr(x), ptr(bufs["positions"]), None, ptr(len_dev), ptr(step_len),
                                (MSA_EMBED_COL_FROM_LEN if col_from_len else 0)
                                | (MSA_EMBED_ROWS_GIVEN if token_embeddings is not None else 0),
                                stream))
        if step_len is not None:
            len_dev = step_len
        self._layernorm(lib, stream, x, self.layers[0].self_attn_layer_norm, M, D, h, OUT)
        x_last = None
        feat = h
        for i, layer in enumerate(self.layers):
            last = i + 1 == L
            ln = self.layer_norm if last else self.layers[i + 1].self_attn_layer_norm
            if last and self.return_inner_states:
                self._decode_layer(lib, stream, layer, cache.k(i), cache.v(i), cache.capacity,
                                   bufs, B, S0, mask, len_dev, None, None, 0)
                x_last = x.view(B, 1, D).transpose(0, 1).clone()
                feat = h if want_packed else torch.empty(M, D, dtype=torch.float16,
                                                         device=x.device)
                self._layernorm(lib, stream, x, ln, M, D, feat, OUT if want_packed else 0)
            elif last and not want_packed:
                feat = torch.empty(M, D, dtype=torch.float16, device=x.device)
                self._decode_layer(lib, stream, layer, cache.k(i), cache.v(i), cache.capacity,
                                   bufs, B, S0, mask, len_dev, ln, feat, 0)
            else:
                self._decode_layer(lib, stream, layer, cache.k(i), cache.v(i), cache.capacity,
                                   bufs, B, S0, mask, len_dev, ln, h, OUT)
        return feat, x_last

    def _decode_layer(self, lib, stream, layer, kc, vc, cap, bufs, B, S0, mask, len_dev, tail_ln,
                      tail_out, tail_flags):
        """One layer of a decode step of at most 128 rows (transformer_decoder_layer.py:233-284).
        In: the residual stream ``bufs["x"]`` (row-major) and its LayerNorm ``bufs["h"]``
        (packed).  Out: ``x`` updated in place and, through the tail fused behind fc2,
        ``tail_out = LayerNorm(x; tail_ln)`` - the next layer's input or the decoder's final
        LayerNorm (``tail_ln`` None: the residual stream only)."""
        cfg = self.cfg
        D, H, hd, F = (cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim,
                       cfg.decoder_ffn_embed_dim)
        x, q, h, o, u, part = (bufs[k] for k in ("x", "q", "h", "o", "u", "part"))
        S_o, S_f = bufs["S_o"], bufs["S_f"]
        IN, OUT = MSA_IN_PACKED, MSA_OUT_PACKED
        mask_stride = mask.stride(0) if mask is not None else 0
        self._qkv(lib, stream, h, layer.self_attn.qkv_proj, q, kc, vc, B, 1, H, hd, S0, cap, D,
                  IN, len_dev)
        check(lib.msa_attention_f16(ptr(q), ptr(kc), ptr(vc), ptr(mask), mask_stride, ptr(o), B,
                                    H, hd, 1, S0, cap, OUT, ptr(len_dev), stream))
        op = layer.self_attn.out_proj
        self._linear_partial(lib, stream, o, op, part, B, D, D, S_o)
        ln = layer.final_layer_norm
        check(lib.msa_residual_layernorm_f16(ptr(part), S_o, ptr(op.bias), ptr(x), ptr(ln.weight),
                                             ptr(ln.bias), ptr(h), B, D, 1e-5, OUT, stream))
        self._linear(lib, stream, h, layer.fc1, B, F, D, relu=True, out=u, flags=IN | OUT)
        self._linear_partial(lib, stream, u, layer.fc2, part, B, D, F, S_f)
        check(lib.msa_residual_layernorm_f16(
            ptr(part), S_f, ptr(layer.fc2.bias), ptr(x),
            ptr(tail_ln.weight) if tail_ln is not None else None,
            ptr(tail_ln.bias) if tail_ln is not None else None, ptr(tail_out), B, D, 1e-5,
            tail_flags, stream))

    def decode_step_static(self, tokens, cache, len_dev, logits_out):
        """Graph-capturable decode step: embeds column ``len_dev[b]`` of the full ``tokens``
        buffer, appends to ``cache`` at that position, attends ``len_dev[b] + 1`` positions and
        writes ``logits_out[B, V]``.  No allocation, no sync, no step-dependent launch argument.
        The caller advances ``len_dev`` (msa_advance_len) and ``cache.length``."""
        lib = self.prepare_()
        stream = _capi.stream_ptr()
        B = tokens.shape[0]
        if B > self.PACKED_MAX_ROWS or cache.has_pads:
            raise ValueError("static decode steps need at most 128 rows and no padding")
        if self.native_step and not self.return_inner_states:
            self._native_step(lib, stream, tokens, tokens.shape[1], B, cache, None, len_dev, 0,
                              {"logits": logits_out}, col_from_len=True, advance=False)
            return logits_out
        bufs = self._step_buffers(cache, B)
        feat, _ = self._decode_core(lib, stream, tokens, tokens.shape[1], B, cache, None, bufs,
                                    len_dev, 0, True, col_from_len=True)
        D, V = self.cfg.decoder_embed_dim, self.cfg.vocab_size
        check(lib.msa_linear_f16(ptr(feat), ptr(self._lm_head), None, None, ptr(logits_out), B, V,
                                 D, MSA_IN_PACKED, stream))
        return logits_out

    def _layernorm(self, lib, stream, x, ln, rows, D, out, flags=0):
        check(lib.msa_layernorm_f16(ptr(x), ptr(ln.weight), ptr(ln.bias), ptr(out), rows, D, 1e-5,
                                    flags, stream))
        return out

    # ------------------------------------------------------------------ forward
    def _forward_features(self, prev_output_tokens, incremental_state, token_embeddings,
                          self_attn_padding_mask, want_packed, native_out=None):
        """Embedding, L pre-LN layers and the final LayerNorm.  Returns (features, packed,
        extra): features are ``[B, T, D]`` row-major, or - for a decode step of at most 128 rows
        when ``want_packed`` - the packed activation buffer the vocabulary projection reads."""
        cfg = self.cfg
        tokens = prev_output_tokens
        if tokens.dim() != 2:
            raise AssertionError("prev_output_tokens must be [batch, tgt_len]")
        if not tokens.is_cuda:
            raise RuntimeError("metaseq_amd: tokens must live on the GPU (no CPU path exists)")
        if tokens.dtype != torch.long:
            tokens = tokens.long()
        if tokens.stride(1) != 1:
            tokens = tokens.contiguous()
        lib = self.prepare_()
        stream = _capi.stream_ptr()
        dev = tokens.device
        B, n = tokens.shape
        D, H, hd = cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim
        F, L = cfg.decoder_ffn_embed_dim, cfg.decoder_layers

        cache = self.get_cache(incremental_state)
        prefill = cache is None
        if prefill:
            T, S0 = n, 0
        else:
            T, S0 = 1, cache.length
            if n != S0 + 1 or cache.batch != B:
                raise AssertionError(
                    "decode step expects the full history [B=%d, %d], got [%d, %d]"
                    % (cache.batch, S0 + 1, B, n))
        if n > self.embed_positions.weight.shape[0] - self.padding_idx - 1:
            raise ValueError("sequence length %d exceeds the %d learned positions"
                             % (n, self.embed_positions.weight.shape[0] - self.padding_idx - 1))

        # key padding mask: the reference tests tokens.eq(pad).any() on every call (a
        # device-to-host sync, transformer_decoder.py:357-361); here only the prefill syncs.
        # Right-padded prompts (the only padding a serving batch has) make the cache "ragged":
        # every row's keys and values are stored without its pads, per-row lengths live on the
        # device, and decode steps neither mask nor stream pad positions.  Pads anywhere else
        # keep the reference's layout (pads stored, masked at every step).
        mask, ragged, lens = None, False, None
        if self_attn_padding_mask is not None:
            if not prefill and cache.ragged:
                raise AssertionError("a cache prefilled from right-padded prompts stores no "
                                     "pads: decode steps take no padding mask")
            mask = self_attn_padding_mask
        elif prefill:
            m = tokens.eq(self.padding_idx)
            counts = n - m.sum(dim=1)
            trailing = m == (torch.arange(n, device=dev).unsqueeze(0) >= counts.unsqueeze(1))
            any_pad, all_trailing = torch.stack([m.any(), trailing.all()]).tolist()
            if any_pad:
                mask = m
                # (a one-column prompt takes the single-token kernels, where per-row lengths
                # mean positions already in the cache: it keeps the masked layout)
                ragged = bool(all_trailing) and B <= self.PACKED_MAX_ROWS and n > 1
                lens = counts.to(torch.int32) if ragged else None
        elif cache.ragged:
            lens = cache.lens
        elif cache.has_pads:
            mask = tokens.eq(self.padding_idx)
        if mask is not None:
            if mask.shape != (B, n):
                raise AssertionError("padding mask must be [batch, src_len]")
            mask = mask.to(torch.uint8).contiguous()

        if prefill:
            cap = self.kv_cache_capacity
            if cap is None:
                cap = min(self.max_positions(), n + 256)
            cap = max(int(cap), n)
            cache = KVCache(L, B, H, hd, cap, dev)
            cache.has_pads = mask is not None
            cache.ragged = ragged
            cache.lens = lens if ragged else None
        elif S0 + 1 > cache.capacity:
            cache.grow(min(max(self.max_positions(), S0 + 1), int(cache.capacity * 1.5) + 64))

        M = B * T
        if token_embeddings is not None:
            # the reference adds the positions to whatever embedding it is handed, one row per
            # embedded column (the last column only on a decode step,
            # metaseq/models/transformer_decoder.py:324-335)
            if tuple(token_embeddings.shape) != (B, T, D) or not token_embeddings.is_cuda:
                raise AssertionError("token_embeddings must be a device tensor [%d, %d, %d]"
                                     % (B, T, D))
            token_embeddings = token_embeddings.to(torch.float16).contiguous()
        PM = self.PACKED_MAX_ROWS
        if (T == 1 and M <= PM and native_out is not None and self.native_step
                and not self.return_inner_states and token_embeddings is None):
            # the whole step (vocabulary projection / selection included) in one C call
            self._native_step(lib, stream, tokens, n, B, cache, mask, lens, S0, native_out)
            cache.length = S0 + T
            if incremental_state is not None:
                incremental_state[self._state_key] = cache
            return None, True, (B, T), {"inner_states": [{"tok": None, "pos": None, "emb": None},
                                                         None]}
        if T == 1 and M <= PM:
            bufs = self._step_buffers(cache, B)
            feat, x_last = self._decode_core(lib, stream, tokens, n, B, cache, mask, bufs, lens,
                                             S0, want_packed, token_embeddings=token_embeddings)
            if lens is not None:
                check(lib.msa_advance_len(ptr(lens), ptr(bufs["step_len"]), B, 1, stream))
            inner_states = [{"tok": None, "pos": bufs["positions"], "emb": None}, x_last]
            packed = want_packed
            features = feat if packed else feat.view(B, T, D)
            cache.length = S0 + T
            if incremental_state is not None:
                incremental_state[self._state_key] = cache
            return features, packed, (B, T), {"inner_states": inner_states}
        int8 = self.layers[0].fc2.qweight is not None
        if T == 1 and int8 and M <= self.W8_CHUNKED_ROWS:
            feat, x_last, positions = self._decode_chunks(lib, stream, tokens, n, B, cache, mask,
                                                          None, S0, token_embeddings)
            cache.length = S0 + T
            if incremental_state is not None:
                incremental_state[self._state_key] = cache
            inner = [{"tok": None, "pos": positions, "emb": None}, x_last]
            return feat.view(B, T, D), False, (B, T), {"inner_states": inner}
        h, inner_states = self._rows_core(lib, stream, tokens, B, n, T, S0, cache, mask,
                                          token_embeddings)
        packed = False
        features = h.view(B, T, D)
        cache.length = S0 + T
        if incremental_state is not None:
            incremental_state[self._state_key] = cache
        return features, packed, (B, T), {"inner_states": inner_states}

    def _rows_core(self, lib, stream, tokens, B, n, T, S0, kv, mask, token_embeddings=None,
                   len_dev=None, step_len=None):
        """Prefill (or a decode batch above 128 rows): the last T columns of ``tokens[B, n]``
        through embedding, L layers and the final LayerNorm on row-major activations and the
        tiled MFMA kernels, keys and values written at positions S0 .. S0 + T - 1 of ``kv``
        (anything with ``k(i)``, ``v(i)`` and ``capacity``).  Returns the normalised features
        [B * T, D] and the inner-states list.  With ``len_dev`` (T == 1; int32 [B] device
        tensor: positions each row already holds, negative = inactive row) every row appends at
        and attends up to its own length; ``step_len`` (int32 [B]) receives the lengths the
        step used (-1 for the rows that sat it out)."""
        cfg = self.cfg
        D = cfg.decoder_embed_dim
        dev = tokens.device
        M = B * T
        x = torch.empty(M, D, dtype=torch.float16, device=dev)
        positions = torch.empty(B, T, dtype=torch.long, device=dev)
        table = self.embed_tokens.weight if token_embeddings is None else token_embeddings
        check(lib.msa_embed_f16(ptr(tokens), tokens.stride(0), B, n, T, ptr(table),
                                cfg.vocab_size, ptr(self.embed_positions.weight),
                                self.embed_positions.weight.shape[0], self.padding_idx, D,
                                ptr(x), ptr(positions), None, ptr(len_dev), ptr(step_len),
                                MSA_EMBED_ROWS_GIVEN if token_embeddings is not None else 0,
                                stream))
        if step_len is not None:
            len_dev = step_len
        inner_states = [{"tok": None, "pos": positions, "emb": None}]
        if self.return_inner_states:
            inner_states[0]["emb"] = x.view(B, T, D).transpose(0, 1).clone()
        work = self._rows_buffers(M, dev)
        for i, layer in enumerate(self.layers):
            self._rows_layer(lib, stream, layer, x, work, B, T, S0, kv.k(i), kv.v(i),
                             kv.capacity, mask, len_dev)
            if self.layer_probe is not None:
                self.layer_probe(i, x)
        if self.return_inner_states:
            inner_states.append(x.view(B, T, D).transpose(0, 1).clone())
        else:
            inner_states.append(None)
        h = work["h"]
        self._layernorm(lib, stream, x, self.layer_norm, M, D, h)
        return h, inner_states

    def _decode_chunks(self, lib, stream, tokens, n, B, cache, mask, lens, S0,
                       token_embeddings=None):
        """A decode step of more than 128 rows over int8 weights, which have no MFMA tile kernel
        that fills the chip at a few hundred rows (66B shape, 200 rows: 162 ms per step): the
        batch runs as chunks of at most 128 rows through the packed path, one sweep over the
        weights per chunk.  ``lens``: per-row lengths (advanced here), or None.  Returns the
        features [B, D], the last layer's residual stream (if inner states are kept) and the
        positions."""
        PM = self.PACKED_MAX_ROWS
        D = self.cfg.decoder_embed_dim
        chunks = (B + PM - 1) // PM
        size = (B + chunks - 1) // chunks
        features = torch.empty(B, D, dtype=torch.float16, device=tokens.device)
        x_last, positions = [], []
        for b0 in range(0, B, size):
            b1 = min(B, b0 + size)
            view = cache.rows_view(b0, b1)
            bufs = self._step_buffers(view, b1 - b0)
            rows = None if lens is None else lens[b0:b1]
            feat, xl = self._decode_core(
                lib, stream, tokens[b0:b1], n, b1 - b0, view,
                None if mask is None else mask[b0:b1].contiguous(), bufs, rows, S0, False,
                token_embeddings=None if token_embeddings is None
                else token_embeddings[b0:b1].contiguous())
            if rows is not None:
                check(lib.msa_advance_len(ptr(rows), ptr(bufs["step_len"]), b1 - b0, 1, stream))
            features[b0:b1] = feat
            x_last.append(xl)
            positions.append(bufs["positions"])
        return (features, torch.cat(x_last, dim=1) if self.return_inner_states else None,
                torch.cat(positions))

    def _rows_buffers(self, M, dev):
        """Work buffers of ``_rows_layer`` for M row-major activation rows."""
        D, F = self.cfg.decoder_embed_dim, self.cfg.decoder_ffn_embed_dim
        f16 = dict(dtype=torch.float16, device=dev)
        return {"q": torch.empty(M, D, **f16), "h": torch.empty(M, D, **f16),
                "o": torch.empty(M, D, **f16), "u": torch.empty(M, F, **f16)}

    def _rows_layer(self, lib, stream, layer, x, work, B, T, S0, kc, vc, cap, mask, len_dev=None):
        """One layer over B * T row-major rows (transformer_decoder_layer.py:233-284): ``x`` is
        the residual stream, updated in place; keys and values of the T new positions of every
        row go to positions S0 .. S0 + T - 1 of ``kc`` / ``vc``."""
        cfg = self.cfg
        D, H, hd, F = (cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim,
                       cfg.decoder_ffn_embed_dim)
        M = B * T
        if M <= self.PACKED_MAX_ROWS:
            return self._rows_layer_short(lib, stream, layer, x, work, B, T, S0, kc, vc, cap, mask,
                                          len_dev)
        q, h, o, u = work["q"], work["h"], work["o"], work["u"]
        mask_stride = mask.stride(0) if mask is not None else 0
        self._layernorm(lib, stream, x, layer.self_attn_layer_norm, M, D, h)
        self._qkv(lib, stream, h, layer.self_attn.qkv_proj, q, kc, vc, B, T, H, hd, S0, cap, D, 0,
                  len_dev)
        check(lib.msa_attention_f16(ptr(q), ptr(kc), ptr(vc), ptr(mask), mask_stride, ptr(o), B,
                                    H, hd, T, S0, cap, 0, ptr(len_dev), stream))
        # x = round(round(o Wo^T + bo) + x)   (transformer_decoder_layer.py:222-230)
        ln2 = layer.final_layer_norm
        if not self._linear_split(lib, stream, o, layer.self_attn.out_proj, x, work, M, D, D,
                                  ln=ln2, ln_out=h):
            self._linear(lib, stream, o, layer.self_attn.out_proj, M, D, D, residual=x, out=x)
            self._layernorm(lib, stream, x, ln2, M, D, h)
        self._linear(lib, stream, h, layer.fc1, M, F, D, relu=True, out=u)
        if not self._linear_split(lib, stream, u, layer.fc2, x, work, M, D, F):
            self._linear(lib, stream, u, layer.fc2, M, D, F, residual=x, out=x)

    def _rows_layer_short(self, lib, stream, layer, x, work, B, T, S0, kc, vc, cap, mask,
                          len_dev=None):
        """``_rows_layer`` for at most 128 rows (a short prompt): the layer's GEMM inputs are
        produced in the packed activation layout by the kernels in front of them, so that qkv,
        fc1 and fc2 run on the weight-streaming kernels of the decode step (56 rows, OPT-6.7B
        shapes: 25 / 30 / 30 us against 32 / 45 / 52 on row-major rows).  The attention output
        stays row-major (the prefill attention kernel writes no packed rows), so out_proj runs
        as in ``_rows_layer``."""
        cfg = self.cfg
        D, H, hd, F = (cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim,
                       cfg.decoder_ffn_embed_dim)
        M = B * T
        IN, OUT = MSA_IN_PACKED, MSA_OUT_PACKED
        q, o = work["q"], work["o"]
        if "hp" not in work:
            MP = self._packed_rows(M)
            work["hp"] = torch.empty(MP * D, dtype=torch.float16, device=x.device)
            work["up"] = torch.empty(MP * F, dtype=torch.float16, device=x.device)
            int8 = layer.fc2.qweight is not None
            splits = lib.msa_linear_default_splits_w8a16 if int8 else lib.msa_linear_default_splits
            work["S_f"] = splits(M, D, F)
        hp, up, S_f = work["hp"], work["up"], work["S_f"]
        mask_stride = mask.stride(0) if mask is not None else 0
        self._layernorm(lib, stream, x, layer.self_attn_layer_norm, M, D, hp, OUT)
        self._qkv(lib, stream, hp, layer.self_attn.qkv_proj, q, kc, vc, B, T, H, hd, S0, cap, D, IN,
                  len_dev)
        check(lib.msa_attention_f16(ptr(q), ptr(kc), ptr(vc), ptr(mask), mask_stride, ptr(o), B,
                                    H, hd, T, S0, cap, 0, ptr(len_dev), stream))
        ln2 = layer.final_layer_norm
        if not self._linear_split(lib, stream, o, layer.self_attn.out_proj, x, work, M, D, D,
                                  ln=ln2, ln_out=hp, ln_flags=OUT):
            self._linear(lib, stream, o, layer.self_attn.out_proj, M, D, D, residual=x, out=x)
            self._layernorm(lib, stream, x, ln2, M, D, hp, OUT)
        self._linear(lib, stream, hp, layer.fc1, M, F, D, relu=True, out=up, flags=IN | OUT)
        part = self._part(work, S_f * M * D, x.device)
        self._linear_partial(lib, stream, up, layer.fc2, part, M, D, F, S_f)
        check(lib.msa_residual_layernorm_f16(ptr(part), S_f, ptr(layer.fc2.bias), ptr(x), None,
                                             None, None, M, D, 1e-5, 0, stream))

    @staticmethod
    def _part(work, n, dev):
        """The fp32 partial-sum buffer of a layer's work buffers, at least ``n`` elements."""
        part = work.get("part")
        if part is None or part.numel() < n:
            part = work["part"] = torch.empty(n, dtype=torch.float32, device=dev)
        return part

    def _linear_split(self, lib, stream, a, lin, x, work, M, N, K, ln=None, ln_out=None,
                      ln_flags=0):
        """``x = round(round(a W^T + b) + x)`` as split-K partial sums + the fused tail, where M
        row-major rows against N output features leave most of the chip without a tile (a decode
        batch above 128 rows: 64 workgroups for d_model 4096); with ``ln``, the LayerNorm of the
        new ``x`` goes to ``ln_out`` in the same launch.  False (nothing done) where one pass of
        the tile kernel is as good, or for int8 weights below the row count from which they run
        expanded to fp16."""
        if lin.qweight is not None and not self._expands(M, N):
            return False
        S = lib.msa_linear_default_splits_rows(M, N, K)
        if S <= 1:
            return False
        part = self._part(work, S * M * N, a.device)
        w = self._expanded(lib, stream, lin) if lin.qweight is not None else ptr(lin.weight)
        check(lib.msa_linear_partial_f16(ptr(a), w, ptr(part), M, N, K, S, 0, stream))
        g, b = (ln.weight, ln.bias) if ln is not None else (None, None)
        check(lib.msa_residual_layernorm_f16(ptr(part), S, ptr(lin.bias), ptr(x), ptr(g), ptr(b),
                                             ptr(ln_out), M, N, 1e-5, ln_flags, stream))
        return True

    # ------------------------------------------------------------------ slot interface
    # A running batch whose rows belong to different requests (continuous batching): a fixed
    # number of slots over one KV cache, each slot filled by its own prefill and advanced by
    # decode steps over all slots at once.  No reference counterpart: the reference's service
    # runs every batch to completion (metaseq/cli/interactive_hosted.py:66-175).
    def new_slot_cache(self, slots: int, capacity: int, device=None) -> KVCache:
        """An empty cache of ``slots`` rows (at most 256) and ``capacity`` positions each."""
        if not 1 <= slots <= self.SLOT_MAX_ROWS:
            raise ValueError("a slot cache holds 1..%d rows" % self.SLOT_MAX_ROWS)
        cfg = self.cfg
        capacity = int(capacity)
        if not 1 <= capacity <= self.max_positions():
            raise ValueError("capacity %d outside 1..%d" % (capacity, self.max_positions()))
        dev = device if device is not None else self.embed_tokens.weight.device
        cache = KVCache(cfg.decoder_layers, slots, cfg.decoder_attention_heads, cfg.head_dim,
                        capacity, dev)
        cache.ragged = True
        cache.lens = torch.full((slots,), -1, dtype=torch.int32, device=dev)
        return cache

    def prefill_slot(self, cache: KVCache, slot: int, tokens: torch.Tensor):
        """Runs the prompt ``tokens`` (1-D ids on the device, no pads, the leading
        end-of-sentence token included) through the model into row ``slot`` of ``cache`` and
        activates the slot.  Returns the logits of every prompt position, ``[T, V]`` fp16."""
        lib = self.prepare_()
        if tokens.dim() != 1 or tokens.numel() == 0 or not tokens.is_cuda:
            raise AssertionError("tokens must be a non-empty 1-D device tensor")
        T = tokens.numel()
        if T >= cache.capacity:
            raise ValueError("a prompt of %d tokens leaves no room in a cache of %d positions"
                             % (T, cache.capacity))
        if not (cache.ragged and 0 <= slot < cache.batch):
            raise ValueError("not a slot cache, or slot %d outside 0..%d" % (slot, cache.batch - 1))
        toks = tokens.long().contiguous().view(1, T)
        h, _ = self._rows_core(lib, _capi.stream_ptr(), toks, 1, T, T, 0, _SlotView(cache, slot),
                               None)
        cache.lens[slot:slot + 1].fill_(T)   # (an element assignment waits for the stream)
        return self._project(h, False, 1, T)[0]

    def prefill_slots(self, cache: KVCache, slots, prompts):
        """One prefill for several prompts (1-D id tensors on the device, as for
        ``prefill_slot``) into the rows ``slots`` of ``cache``: the prompts run as one
        right-padded batch, so the weights are read once for all of them - under the causal
        mask no real position sees a pad, and the pads' own rows are dropped - and every
        prompt's keys and values are then copied to its slot.  Returns the logits of every
        prompt's positions, a list of ``[T_i, V]`` fp16 tensors.  The products run on other
        tile shapes than a prompt's own prefill would, so results can differ from
        ``prefill_slot``'s in the last bit."""
        if len(slots) != len(prompts) or not prompts:
            raise AssertionError("one slot per prompt")
        if len(prompts) == 1:
            return [self.prefill_slot(cache, slots[0], prompts[0])]
        lib = self.prepare_()
        cfg = self.cfg
        lens = [int(t.numel()) for t in prompts]
        for slot, t, T in zip(slots, prompts, lens):
            if t.dim() != 1 or T == 0 or not t.is_cuda:
                raise AssertionError("tokens must be non-empty 1-D device tensors")
            if T >= cache.capacity:
                raise ValueError("a prompt of %d tokens leaves no room in a cache of %d "
                                 "positions" % (T, cache.capacity))
            if not (cache.ragged and 0 <= slot < cache.batch):
                raise ValueError("not a slot cache, or slot %d outside 0..%d"
                                 % (slot, cache.batch - 1))
        if len(set(slots)) != len(slots):
            raise ValueError("a slot is named twice")
        k, Tmax = len(prompts), max(lens)
        dev = prompts[0].device
        toks = torch.full((k, Tmax), self.padding_idx, dtype=torch.long, device=dev)
        for r, t in enumerate(prompts):
            toks[r, :lens[r]] = t
        tmp = KVCache(cfg.decoder_layers, k, cfg.decoder_attention_heads, cfg.head_dim, Tmax, dev)
        h, _ = self._rows_core(lib, _capi.stream_ptr(), toks, k, Tmax, Tmax, 0, tmp, None)
        # one copy per layer: whole padded rows (what lies past a prompt's length is never read)
        where = upload(slots, torch.long, dev)
        for mine, theirs in zip(cache.layers, tmp.layers):
            mine[:, :, :, :Tmax].index_copy_(1, where, theirs)
        cache.lens[where] = upload(lens, torch.int32, dev)
        logits = self._project(h, False, k, Tmax)
        return [logits[r, :lens[r]] for r in range(k)]

    # admit_slot / admit_slots take ``lazy=True``: the prompt scores come back as device tensors
    # (None for a one-token prompt) for the caller to read together with everything else
    lazy_admission = True

    def admit_slots(self, cache: KVCache, requests, lazy=False):
        """``admit_slot`` for several requests with one shared prefill (``prefill_slots``).
        ``requests``: dicts with ``slot``, ``tokens`` and the keyword arguments of
        ``admit_slot``; returns the list of their prompt scores (``lazy``: as fp32 device
        tensors without the leading 0.0, nothing read back yet)."""
        logits = self.prefill_slots(cache, [r["slot"] for r in requests],
                                    [r["tokens"] for r in requests])
        out = []
        for r, lg in zip(requests, logits):
            kw = {k: v for k, v in r.items() if k not in ("slot", "tokens")}
            out.append(self.admit_slot(cache, r["slot"], r["tokens"], _logits=lg, _lazy=True,
                                       **kw))
        if lazy:
            return out
        # every request's kernels are queued: one copy for all the scores
        flat = torch.cat([lp for lp in out if lp is not None]).tolist() if any(
            lp is not None for lp in out) else []
        scores, at = [], 0
        for lp in out:
            n = lp.numel() if lp is not None else 0
            scores.append([0.0] + flat[at:at + n])
            at += n
        return scores

    def admit_slot(self, cache: KVCache, slot: int, tokens: torch.Tensor, *, banned=(), stop=(),
                   eos=2, mode=0, tok_out=None, score_out=None, temperature=1.0, topp=0.0,
                   noise=None, replicas=(), penalties=None, lprobs_out=None, prompt_topk=0,
                   detail=None, lazy=False, _logits=None, _lazy=False):
        """``prefill_slot`` plus what a request needs from its prompt: the log-probability of
        every prompt token given its prefix (returned as a list, 0.0 for the first token) and
        the choice of the first new token from the last position, written to ``tok_out`` /
        ``score_out`` (int64 / fp32 device tensors, one element per replica) under the selection
        regime ``mode`` (MSA_ROW_* bits).

        With the defaults the choice is greedy on the unscaled logits.  ``temperature`` scales
        the logits (prompt scores included, as the reference's loop does); ``topp`` > 0 with
        ``noise`` (fp32 [1 + len(replicas), V], independent Exp(1) numbers) draws from the
        nucleus.  ``replicas``: further slots that receive a copy of the prompt's keys and values
        and make their own choice (row r of ``noise``, element r of the outputs).

        ``penalties``: dict with ``alphas`` (presence, frequency, presence_src, frequency_src),
        ``counts`` (int64 [R, V], updated with the chosen tokens) and ``counts_src`` (int64
        [R, V] prompt-token counts), R = 1 + len(replicas): the reference's repetition penalties
        on the first choice.  ``lprobs_out`` (fp32 [R, V]) receives the masked, penalised
        log-probabilities the choice was made from.  ``prompt_topk`` > 0 with a dict ``detail``:
        ``detail["prompt_top"]`` = (values, ids), CPU tensors [T - 1, k], the k most likely
        tokens at every prompt position after the first (log-softmax of logits / temperature,
        what the reference records for the prompt with ``need_logprobs``)."""
        lib = self.prepare_()
        _lazy = _lazy or lazy
        # (_logits: the prompt was already prefilled into the slot, by prefill_slots)
        logits = _logits if _logits is not None else self.prefill_slot(cache, slot, tokens)
        T, V = logits.shape
        stream = _capi.stream_ptr()
        scores, lp = [0.0] * T, None
        if T > 1:
            lp = torch.empty(T - 1, dtype=torch.float32, device=logits.device)
            target = tokens.long()[1:].contiguous()
            check(lib.msa_target_logprob_f16(ptr(logits), logits.stride(0), T - 1, V,
                                             float(temperature), ptr(target), ptr(lp), stream))
            if not _lazy:   # (_lazy: the caller reads the device tensor once all is queued)
                scores[1:] = lp.tolist()
            if prompt_topk > 0 and detail is not None:
                dist = torch.empty(T - 1, V, dtype=torch.float32, device=logits.device)
                check(lib.msa_log_softmax_f16(ptr(logits), 0, logits.stride(0), 1, T - 1, V,
                                              float(temperature), ptr(dist), 0, V, stream))
                values, ids = dist.topk(min(int(prompt_topk), V), dim=-1)
                detail["prompt_top"] = (values.cpu(), ids.cpu())
                del dist
        for dst in replicas:
            self.copy_slot(cache, slot, dst, length=T)
        R = 1 + len(replicas)
        plain = (float(temperature) == 1.0 and not topp > 0 and noise is None
                 and penalties is None and lprobs_out is None)
        banned, stop = list(banned), list(stop)
        ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
        sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
        row_mode = torch.full((R,), mode, dtype=torch.uint8, device=logits.device)
        last = logits[T - 1:T]
        if R > 1:  # every replica reads its own copy of the row (a few hundred KB)
            last = last.expand(R, V).contiguous()
        if plain:
            check(lib.msa_greedy_select_f16(ptr(last), last.stride(0), R, V, 1.0, ba, len(banned),
                                            sa, len(stop), None, ptr(row_mode), 0, int(eos),
                                            ptr(tok_out), 1, ptr(score_out), 1, None, stream))
        else:
            pen = penalties or {}
            alphas = [float(a) for a in pen.get("alphas", (0.0, 0.0, 0.0, 0.0))]
            for name in ("counts", "counts_src"):
                t = pen.get(name)
                if t is not None and (t.shape != (R, V) or t.dtype != torch.long
                                      or not t.is_contiguous()):
                    raise AssertionError("%s must be contiguous int64 [%d, %d]" % (name, R, V))
            if lprobs_out is not None and (lprobs_out.shape != (R, V)
                                           or lprobs_out.dtype != torch.float32
                                           or lprobs_out.stride(1) != 1):
                raise AssertionError("lprobs_out must be fp32 [%d, %d]" % (R, V))
            check(lib.msa_sample_topp_f16(
                ptr(last), last.stride(0), R, V, float(temperature), None, ba, len(banned), sa,
                len(stop), None, ptr(row_mode), 0, int(eos), None, float(topp), ptr(noise),
                ptr(pen.get("counts")), ptr(pen.get("counts_src")), alphas[0], alphas[1],
                alphas[2], alphas[3], None, ptr(lprobs_out),
                lprobs_out.stride(0) if lprobs_out is not None else 0, ptr(tok_out), 1,
                ptr(score_out), 1, stream))
        return lp if _lazy else scores

    def copy_slot(self, cache: KVCache, src: int, dst: int, length: Optional[int] = None):
        """Makes slot ``dst`` a copy of slot ``src``: keys, values and length (a replica of a
        request starts from the same prompt).  ``length``: the source's length where the caller
        knows it (reading it from the device waits for everything queued)."""
        n = int(cache.lens[src]) if length is None else int(length)
        for layer in cache.layers:
            layer[:, dst, :, :n].copy_(layer[:, src, :, :n])
        cache.lens[dst:dst + 1].fill_(n)

    def release_slot(self, cache: KVCache, slot: int):
        # a fill kernel on a one-element view: ``lens[slot] = -1`` copies a host scalar to the
        # device and makes the caller wait for the work queued ahead of it
        cache.lens[slot:slot + 1].fill_(-1)

    def decode_slots(self, cache: KVCache, last_tokens: torch.Tensor, *, temperature=1.0,
                     banned=(), stop=(), eos=2, row_mode=None, tok_out=None, score_out=None,
                     finished=None, logits_out=None, sampled=None):
        """One decode step over every active slot: ``last_tokens`` ([slots] ids on the device;
        what an inactive slot holds does not matter) are embedded at each row's own position,
        appended to its history and attended over it; the vocabulary projection selects the
        next token greedily into ``tok_out`` / ``score_out`` ([slots], int64 / fp32) under the
        per-row ``row_mode`` (uint8 [slots]: MSA_ROW_BAN_EARLY, MSA_ROW_ONLY_EOS).  Every active
        row's length advances by one.  Outputs of inactive slots are undefined.

        ``sampled``: rows that are not chosen that way (another temperature, nucleus sampling) -
        a dict with ``row_mode`` (uint8 [slots]: the regime bits of those rows, MSA_ROW_SKIP for
        all others), ``temperature`` and ``topp`` (fp32 [slots]; top-p 0 = greedy at that
        temperature) and ``noise`` (fp32 [slots, V] Exp(1) numbers, or None).  The step then
        also stores its logits (``logits_out``, [slots, V] fp16, required) and
        msa_sample_topp_f16 overwrites the outputs of those rows.  Optional entries:
        ``penalty_rows`` (fp32 [slots, 4]: presence, frequency, presence_src, frequency_src of
        every row) with ``counts`` / ``counts_src`` (int64 [slots, V]; the former is updated
        with the chosen tokens), and ``lprobs_out`` (fp32 [slots, V]): the masked, penalised
        log-probabilities of those rows."""
        lib = self.prepare_()
        stream = _capi.stream_ptr()
        B = cache.batch
        if last_tokens.shape != (B,) or last_tokens.dtype != torch.long:
            raise AssertionError("last_tokens must be int64 [%d]" % B)
        if sampled is not None and logits_out is None:
            raise AssertionError("sampled rows need logits_out")
        if B > self.PACKED_MAX_ROWS:
            # row-major activations through the tile kernels (int8 weights: chunks of <= 128
            # rows through the packed path), stored logits, stand-alone selection
            tokens = last_tokens.view(B, 1)
            if self.layers[0].fc2.qweight is not None:
                feat, _, _ = self._decode_chunks(lib, stream, tokens, 1, B, cache, None,
                                                 cache.lens, 0)
            else:
                step_len = getattr(cache, "step_len", None)
                if step_len is None:
                    step_len = cache.step_len = torch.empty(B, dtype=torch.int32,
                                                            device=cache.device)
                feat, _ = self._rows_core(lib, stream, tokens, B, 1, 1, 0, cache, None,
                                          len_dev=cache.lens, step_len=step_len)
                check(lib.msa_advance_len(ptr(cache.lens), ptr(step_len), B, 1, stream))
            self._select_from(lib, feat, B, temperature, banned, stop, finished, row_mode, False,
                              eos, tok_out, 1, score_out, 1, logits_out, packed=False)
        elif self.native_step and not self.return_inner_states:
            select = dict(temperature=temperature, banned=banned, stop=stop, finished=finished,
                          row_mode=row_mode, force_eos=False, eos=eos, tok_out=tok_out,
                          tok_stride=1, score_out=score_out, score_stride=1)
            self._native_step(lib, stream, last_tokens.view(B, 1), 1, B, cache, None, cache.lens,
                              0, {"logits": logits_out, "select": select})
        else:
            bufs = self._step_buffers(cache, B)
            feat, _ = self._decode_core(lib, stream, last_tokens.view(B, 1), 1, B, cache, None,
                                        bufs, cache.lens, 0, True)
            check(lib.msa_advance_len(ptr(cache.lens), ptr(bufs["step_len"]), B, 1, stream))
            self._select_from(lib, feat, B, temperature, banned, stop, finished, row_mode, False,
                              eos, tok_out, 1, score_out, 1, logits_out)
        if sampled is not None:
            banned, stop = list(banned), list(stop)
            ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
            sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
            V = self.cfg.vocab_size
            lp = sampled.get("lprobs_out")
            for name, dtype in (("counts", torch.long), ("counts_src", torch.long),
                                ("lprobs_out", torch.float32)):
                t = sampled.get(name)
                if t is not None and (t.shape != (B, V) or t.dtype != dtype
                                      or not t.is_contiguous()):
                    raise AssertionError("%s must be contiguous [%d, %d]" % (name, B, V))
            pr = sampled.get("penalty_rows")
            if pr is not None and (pr.shape != (B, 4) or pr.dtype != torch.float32
                                   or not pr.is_contiguous()):
                raise AssertionError("penalty_rows must be contiguous fp32 [%d, 4]" % B)
            check(lib.msa_sample_topp_f16(
                ptr(logits_out), logits_out.stride(0), B, V, 1.0, ptr(sampled["temperature"]), ba,
                len(banned), sa, len(stop), ptr(finished), ptr(sampled["row_mode"]), 0, int(eos),
                ptr(sampled["topp"]), 0.0, ptr(sampled.get("noise")),
                ptr(sampled.get("counts")) if pr is not None else None,
                ptr(sampled.get("counts_src")) if pr is not None else None, 0.0, 0.0, 0.0, 0.0,
                ptr(pr), ptr(lp), V if lp is not None else 0, ptr(tok_out), 1, ptr(score_out), 1,
                stream))

    def extract_features(self, prev_output_tokens, incremental_state=None,
                         token_embeddings=None, self_attn_padding_mask=None):
        """metaseq/models/transformer_decoder.py:348-396.  Returns features ``[B, T, D]`` (the
        reference returns the same values as ``[T, B, D]``)."""
        f, _, _, extra = self._forward_features(prev_output_tokens, incremental_state,
                                                token_embeddings, self_attn_padding_mask, False)
        return f, extra

    def _project(self, features, packed, B, T):
        lib = self._lib
        D, V = self.cfg.decoder_embed_dim, self.cfg.vocab_size
        y = torch.empty(B * T, V, dtype=torch.float16, device=features.device)
        check(lib.msa_linear_f16(ptr(features), ptr(self._lm_head), None, None, ptr(y), B * T, V,
                                 D, MSA_IN_PACKED if packed else 0, _capi.stream_ptr()))
        return y.view(B, T, V)

    def output_layer(self, features, **kwargs):
        """Tied vocabulary projection without bias
        (metaseq/models/transformer_decoder.py:398-428). features ``[B, T, D]`` row-major."""
        self.prepare_()
        B, T, D = features.shape
        return self._project(features.contiguous(), False, B, T)

    def forward(self, prev_output_tokens,
                incremental_state: Optional[Dict[str, Any]] = None,
                features_only: bool = False, src_lengths=None, token_embeddings=None,
                self_attn_padding_mask=None):
        """metaseq/models/transformer_decoder.py:494-537."""
        native_out = None
        if (not features_only and self.native_step and incremental_state
                and prev_output_tokens.dim() == 2
                and prev_output_tokens.shape[0] <= self.PACKED_MAX_ROWS
                and prev_output_tokens.is_cuda):
            native_out = {"logits": torch.empty(prev_output_tokens.shape[0], self.cfg.vocab_size,
                                                dtype=torch.float16,
                                                device=prev_output_tokens.device)}
        f, packed, (B, T), extra = self._forward_features(
            prev_output_tokens, incremental_state, token_embeddings, self_attn_padding_mask,
            want_packed=not features_only, native_out=native_out)
        if features_only:
            return f, extra
        if f is None:  # the native step wrote the logits
            return native_out["logits"].view(B, T, -1), extra
        return self._project(f, packed, B, T), extra

    def forward_select(self, prev_output_tokens, incremental_state, *, temperature, banned, stop,
                       finished, force_eos, eos, tok_out, tok_stride, score_out, score_stride,
                       logits_out=None, row_mode=None):
        """One decode step (at most 128 rows) whose vocabulary projection is fused with the greedy
        selection of the next token (metaseq/models/transformer_decoder.py:494-537 followed by
        metaseq/sequence_generator.py:272-308,319-323): the logits are reduced inside the
        projection's epilogue and never stored unless ``logits_out`` ([B, V] fp16) is given.
        ``tok_out`` / ``score_out`` are views of the first row's output element (column of the
        token being chosen) with the given row strides; ``banned`` / ``stop`` are id lists,
        ``finished`` the uint8 row flags the call updates."""
        if not incremental_state:
            raise AssertionError("forward_select is a decode step: prefill first")
        select = dict(temperature=temperature, banned=banned, stop=stop, finished=finished,
                      row_mode=row_mode, force_eos=force_eos, eos=eos, tok_out=tok_out,
                      tok_stride=tok_stride, score_out=score_out, score_stride=score_stride)
        f, packed, (B, T), _ = self._forward_features(
            prev_output_tokens, incremental_state, None, None, want_packed=True,
            native_out={"logits": logits_out, "select": select})
        if not packed:
            raise ValueError("forward_select needs at most 128 rows")
        if f is None:
            return  # the native step selected
        self._select_from(self._lib, f, B, temperature, banned, stop, finished, row_mode,
                          force_eos, eos, tok_out, tok_stride, score_out, score_stride, logits_out)

    def _select_from(self, lib, f, B, temperature, banned, stop, finished, row_mode, force_eos,
                     eos, tok_out, tok_stride, score_out, score_stride, logits_out, packed=True):
        """Vocabulary projection of the packed features ``f`` fused with the greedy selection
        (beyond 64 rows, or for row-major features: the projection stores its logits and a
        second kernel selects)."""
        D, V = self.cfg.decoder_embed_dim, self.cfg.vocab_size
        if B > 64 or not packed:
            banned, stop = list(banned), list(stop)
            ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
            sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
            logits = logits_out if logits_out is not None else torch.empty(
                B, V, dtype=torch.float16, device=f.device)
            stream = _capi.stream_ptr()
            check(lib.msa_linear_f16(ptr(f), ptr(self._lm_head), None, None, ptr(logits), B, V, D,
                                     MSA_IN_PACKED if packed else 0, stream))
            check(lib.msa_greedy_select_f16(
                ptr(logits), V, B, V, float(temperature), ba, len(banned), sa, len(stop),
                ptr(finished), ptr(row_mode), int(force_eos), int(eos), ptr(tok_out), tok_stride,
                ptr(score_out), score_stride, None, stream))
            return
        need = lib.msa_lm_head_select_workspace_bytes(B)
        ws = getattr(self, "_select_ws", None)
        if ws is None or ws.numel() < need or ws.device != f.device:
            ws = self._select_ws = torch.empty(need, dtype=torch.uint8, device=f.device)
        banned, stop = list(banned), list(stop)
        ba = (ctypes.c_int32 * max(1, len(banned)))(*banned)
        sa = (ctypes.c_int32 * max(1, len(stop)))(*stop)
        check(lib.msa_lm_head_greedy_select_f16(
            ptr(f), ptr(self._lm_head), ptr(logits_out), ptr(ws), B, V, D, float(temperature), ba,
            len(banned), sa, len(stop), ptr(finished), ptr(row_mode), int(force_eos), int(eos),
            ptr(tok_out), tok_stride, ptr(score_out), score_stride, None, _capi.stream_ptr()))


class _SlotView:
    """Row ``slot`` of a KV cache, with the interface the prefill path expects of a cache."""

    def __init__(self, cache: KVCache, slot: int):
        self._layers, self._slot, self.capacity = cache.layers, slot, cache.capacity

    def k(self, i):
        return self._layers[i][0][self._slot:self._slot + 1]

    def v(self, i):
        return self._layers[i][1][self._slot:self._slot + 1]


# the name the reference's model code uses for this class
ModelParallelTransformerDecoder = TransformerDecoder
