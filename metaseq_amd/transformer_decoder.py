"""OPT decoder forward on hand-written gfx950 kernels, behind the interface of the
reference's ``ModelParallelTransformerDecoder`` (metaseq/models/transformer_decoder.py:62-537)
at tensor-parallel size 1: same ``forward`` signature, same prefill/decode switch (an empty
``incremental_state`` dict means prefill, a non-empty one a single-token step), same
parameter names in ``state_dict()``.

All arithmetic runs in libmetaseq_amd.so through the C ABI; torch only owns the device
memory and the stream.  There is no eager fallback.
"""
import uuid
from typing import Any, Dict, Optional

import torch
from torch import nn

from . import _capi
from ._capi import MSA_EPI_RELU, check, ptr
from .config import OPTConfig
from .kv_cache import KVCache


class _Affine(nn.Module):
    """weight + bias holder (Linear or LayerNorm parameters under the reference's names)."""

    def __init__(self, w_shape, b_shape):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(w_shape, dtype=torch.float16), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(b_shape, dtype=torch.float16), requires_grad=False)
        # int8 weight-only form, filled by TransformerDecoder.quantize_int8_()
        self.qweight: Optional[torch.Tensor] = None
        self.scales: Optional[torch.Tensor] = None


class _Table(nn.Module):
    def __init__(self, rows, dim):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(rows, dim, dtype=torch.float16),
                                   requires_grad=False)


class _SelfAttention(nn.Module):
    def __init__(self, D):
        super().__init__()
        self.qkv_proj = _Affine((3 * D, D), (3 * D,))  # rows K | V | Q
        self.out_proj = _Affine((D, D), (D,))


class _DecoderLayer(nn.Module):
    def __init__(self, D, F):
        super().__init__()
        self.self_attn_layer_norm = _Affine((D,), (D,))
        self.self_attn = _SelfAttention(D)
        self.final_layer_norm = _Affine((D,), (D,))
        self.fc1 = _Affine((F, D), (F,))
        self.fc2 = _Affine((D, F), (D,))


class TransformerDecoder(nn.Module):
    """Drop-in for the reference decoder on the generation path.

    ``forward(prev_output_tokens, incremental_state)`` returns ``(logits[B, T, V], extra)``
    with ``T = n`` for prefill (``incremental_state`` None or empty) and ``T = 1`` for a decode
    step, mutating the caller's dict in place so that it is non-empty after the prefill.
    """

    def __init__(self, cfg: OPTConfig, state_dict: Optional[Dict[str, torch.Tensor]] = None,
                 device="cuda"):
        super().__init__()
        self.cfg = cfg
        self.args = cfg  # the reference exposes its namespace as .args
        D, F = cfg.decoder_embed_dim, cfg.decoder_ffn_embed_dim
        self.padding_idx = cfg.padding_idx
        self.max_target_positions = cfg.max_target_positions
        self.share_input_output_embed = True
        self.embed_scale = 1.0
        self.register_buffer("version", torch.tensor([3.0]))
        self.embed_tokens = _Table(cfg.vocab_size, D)
        self.embed_positions = _Table(cfg.max_target_positions + cfg.padding_idx + 1, D)
        self.layers = nn.ModuleList([_DecoderLayer(D, F) for _ in range(cfg.decoder_layers)])
        self.layer_norm = _Affine((D,), (D,))
        self.inference = True
        self.return_inner_states = False
        # capacity (positions) of the KV cache the next prefill allocates; None = grow on demand
        self.kv_cache_capacity: Optional[int] = None
        self._state_key = str(uuid.uuid4()) + ".kv_cache"
        self._lib = None
        if state_dict is not None:
            self.load_state_dict(state_dict)
        self.to(device)
        if cfg.quantize_int8:
            self.quantize_int8_()

    # ------------------------------------------------------------------ weights
    def load_state_dict(self, state_dict, strict=True, **kw):
        sd = dict(state_dict)
        # accept a model-level dict ("decoder." prefix) and the tied duplicate key
        if any(k.startswith("decoder.") for k in sd):
            sd = {k[len("decoder."):]: v for k, v in sd.items() if k.startswith("decoder.")}
        sd.pop("output_projection.weight", None)
        return super().load_state_dict(sd, strict=strict, **kw)

    def quantize_int8_(self):
        """Symmetric per-output-channel int8 for qkv / out_proj / fc1 / fc2 (the matrices the
        reference quantises for serving, metaseq/scripts/convert_metaseq_ft.py:118-129):
        scale_j = fp16(max_i |W_ji| / 127), q = clamp(rint(W / scale_j), -127, 127).  The fp16
        matrices are released."""
        for layer in self.layers:
            for lin in (layer.self_attn.qkv_proj, layer.self_attn.out_proj, layer.fc1, layer.fc2):
                w = lin.weight.data.float()
                scales = (w.abs().amax(dim=1) / 127.0).to(torch.float16)
                s = scales.float().clamp_min(1e-30).unsqueeze(1)
                lin.qweight = torch.clamp(torch.round(w / s), -127, 127).to(torch.int8).contiguous()
                lin.scales = scales.contiguous()
                lin.weight.data = torch.empty(0, dtype=torch.float16, device=w.device)
                del w
        self.cfg.quantize_int8 = True
        return self

    def dequantized_state_dict(self):
        """Reference-named fp16 weights with quantised matrices replaced by round(q * scale):
        what a reference model must be loaded with to be compared against the int8 path."""
        sd = {"decoder." + k: v for k, v in self.state_dict().items()}
        for i, layer in enumerate(self.layers):
            for name, lin in (("self_attn.qkv_proj", layer.self_attn.qkv_proj),
                              ("self_attn.out_proj", layer.self_attn.out_proj),
                              ("fc1", layer.fc1), ("fc2", layer.fc2)):
                if lin.qweight is not None:
                    sd[f"decoder.layers.{i}.{name}.weight"] = (
                        lin.qweight.float() * lin.scales.float().unsqueeze(1)).to(torch.float16)
        return sd

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
    def _linear(self, lib, stream, x, lin, M, N, K, bias=True, residual=None, relu=False,
                out=None):
        y = out if out is not None else torch.empty(M, N, dtype=torch.float16, device=x.device)
        flags = MSA_EPI_RELU if relu else 0
        b = lin.bias if bias else None
        if lin.qweight is not None:
            check(lib.msa_linear_w8a16(ptr(x), ptr(lin.qweight), ptr(lin.scales), ptr(b),
                                       ptr(residual), ptr(y), M, N, K, flags, None, 0, stream))
        else:
            check(lib.msa_linear_f16(ptr(x), ptr(lin.weight), ptr(b), ptr(residual), ptr(y), M, N,
                                     K, flags, None, 0, stream))
        return y

    def _layernorm(self, lib, stream, x, ln, rows, D, out=None):
        y = out if out is not None else torch.empty_like(x)
        check(lib.msa_layernorm_f16(ptr(x), ptr(ln.weight), ptr(ln.bias), ptr(y), rows, D, 1e-5,
                                    stream))
        return y

    # ------------------------------------------------------------------ forward
    def extract_features(self, prev_output_tokens, incremental_state=None,
                         token_embeddings=None, self_attn_padding_mask=None):
        """Embedding, L pre-LN layers and the final LayerNorm
        (metaseq/models/transformer_decoder.py:348-396).  Returns features ``[B, T, D]``
        (the reference returns the same values as ``[T, B, D]``)."""
        cfg = self.cfg
        if token_embeddings is not None:
            raise NotImplementedError("precomputed token_embeddings are not supported")
        tokens = prev_output_tokens
        if tokens.dim() != 2:
            raise AssertionError("prev_output_tokens must be [batch, tgt_len]")
        if not tokens.is_cuda:
            raise RuntimeError("metaseq_amd: tokens must live on the GPU (no CPU path exists)")
        if tokens.dtype != torch.long:
            tokens = tokens.long()
        if tokens.stride(1) != 1:
            tokens = tokens.contiguous()
        lib = self._lib or _capi.load()
        self._lib = lib
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
        mask = None
        if self_attn_padding_mask is not None:
            mask = self_attn_padding_mask
        elif prefill:
            m = tokens.eq(self.padding_idx)
            if bool(m.any()):
                mask = m
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
        elif S0 + 1 > cache.capacity:
            cache.grow(min(max(self.max_positions(), S0 + 1), int(cache.capacity * 1.5) + 64))

        M = B * T
        x = torch.empty(M, D, dtype=torch.float16, device=dev)
        positions = torch.empty(B, T, dtype=torch.long, device=dev)
        check(lib.msa_embed_f16(ptr(tokens), tokens.stride(0), B, n, T,
                                ptr(self.embed_tokens.weight), cfg.vocab_size,
                                ptr(self.embed_positions.weight),
                                self.embed_positions.weight.shape[0], self.padding_idx, D,
                                ptr(x), ptr(positions), None, stream))
        inner_states = [{"tok": None, "pos": positions, "emb": None}]
        if self.return_inner_states:
            inner_states[0]["emb"] = x.view(B, T, D).transpose(0, 1).clone()

        h = torch.empty_like(x)
        q = torch.empty_like(x)
        o = torch.empty_like(x)
        u = torch.empty(M, F, dtype=torch.float16, device=dev)
        mask_stride = mask.stride(0) if mask is not None else 0
        for i, layer in enumerate(self.layers):
            self._layernorm(lib, stream, x, layer.self_attn_layer_norm, M, D, out=h)
            qkv = layer.self_attn.qkv_proj
            kc, vc = cache.k(i), cache.v(i)
            if qkv.qweight is not None:
                check(lib.msa_qkv_proj_w8a16(ptr(h), ptr(qkv.qweight), ptr(qkv.scales),
                                             ptr(qkv.bias), ptr(q), ptr(kc), ptr(vc), B, T, H, hd,
                                             S0, cache.capacity, D, None, 0, stream))
            else:
                check(lib.msa_qkv_proj_f16(ptr(h), ptr(qkv.weight), ptr(qkv.bias), ptr(q),
                                           ptr(kc), ptr(vc), B, T, H, hd, S0, cache.capacity, D,
                                           None, 0, stream))
            check(lib.msa_attention_f16(ptr(q), ptr(kc), ptr(vc), ptr(mask), mask_stride, ptr(o),
                                        B, H, hd, T, S0, cache.capacity, stream))
            # x = round(round(o Wo^T + bo) + x)   (transformer_decoder_layer.py:222-230)
            self._linear(lib, stream, o, layer.self_attn.out_proj, M, D, D, residual=x, out=x)
            self._layernorm(lib, stream, x, layer.final_layer_norm, M, D, out=h)
            self._linear(lib, stream, h, layer.fc1, M, F, D, relu=True, out=u)
            self._linear(lib, stream, u, layer.fc2, M, D, F, residual=x, out=x)
        cache.length = S0 + T
        if incremental_state is not None:
            incremental_state[self._state_key] = cache
        if self.return_inner_states:
            inner_states.append(x.view(B, T, D).transpose(0, 1).clone())
        else:
            inner_states.append(None)
        self._layernorm(lib, stream, x, self.layer_norm, M, D, out=h)
        return h.view(B, T, D), {"inner_states": inner_states}

    def output_layer(self, features, **kwargs):
        """Tied vocabulary projection without bias
        (metaseq/models/transformer_decoder.py:398-428). features ``[B, T, D]``."""
        lib = self._lib or _capi.load()
        B, T, D = features.shape
        V = self.cfg.vocab_size
        f = features.contiguous().view(B * T, D)
        y = torch.empty(B * T, V, dtype=torch.float16, device=f.device)
        check(lib.msa_linear_f16(ptr(f), ptr(self.embed_tokens.weight), None, None, ptr(y), B * T,
                                 V, D, 0, None, 0, _capi.stream_ptr()))
        return y.view(B, T, V)

    def forward(self, prev_output_tokens,
                incremental_state: Optional[Dict[str, Any]] = None,
                features_only: bool = False, src_lengths=None, token_embeddings=None,
                self_attn_padding_mask=None):
        """metaseq/models/transformer_decoder.py:494-537."""
        x, extra = self.extract_features(prev_output_tokens, incremental_state=incremental_state,
                                         token_embeddings=token_embeddings,
                                         self_attn_padding_mask=self_attn_padding_mask)
        if not features_only:
            x = self.output_layer(x)
        return x, extra


# the name the reference's model code uses for this class
ModelParallelTransformerDecoder = TransformerDecoder
