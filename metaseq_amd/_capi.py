"""ctypes binding of libmetaseq_amd.so (the C ABI declared in include/metaseq_amd.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
Shape / argument errors surface as ValueError, capacity overruns as ValueError, HIP
failures as RuntimeError (the reference's serving loop treats a RuntimeError from
``generate`` as a device fault and restarts the worker, metaseq/cli/interactive_hosted.py:161-171).
"""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmetaseq_amd.so")

MSA_EPI_RELU = 1
MSA_IN_PACKED = 2
MSA_OUT_PACKED = 4
MSA_EMBED_COL_FROM_LEN = 8
MSA_EMBED_ROWS_GIVEN = 32
MSA_ROW_BAN_EARLY = 1
MSA_ROW_ONLY_EOS = 2
MSA_ROW_SKIP = 4

_P = c_void_p
MSA_STEP_NO_ADVANCE = 16


class DecoderConfig(ctypes.Structure):
    """msa_decoder_config"""
    _fields_ = [(n, c_int) for n in ("layers", "d_model", "heads", "ffn", "vocab", "n_pos_rows",
                                     "pad_idx", "int8")]


class LayerWeights(ctypes.Structure):
    """msa_layer_weights: device pointers of one layer's parameters."""
    _fields_ = [(n, c_void_p) for n in (
        "ln1_gamma", "ln1_beta", "qkv_weight", "qkv_scales", "qkv_bias", "out_weight",
        "out_scales", "out_bias", "ln2_gamma", "ln2_beta", "fc1_weight", "fc1_scales",
        "fc1_bias", "fc2_weight", "fc2_scales", "fc2_bias")]


class StepArgs(ctypes.Structure):
    """msa_step_args"""
    _fields_ = [("tokens", c_void_p), ("tok_stride", c_int64), ("n", c_int), ("B", c_int),
                ("k_cache", ctypes.POINTER(c_void_p)), ("v_cache", ctypes.POINTER(c_void_p)),
                ("S0", c_int), ("S_cap", c_int), ("len_dev", c_void_p),
                ("key_pad_mask", c_void_p), ("mask_stride", c_int64), ("flags", c_uint),
                ("workspace", c_void_p), ("workspace_bytes", c_int64), ("logits", c_void_p),
                ("tok", c_void_p), ("tok_stride_out", c_int64), ("score", c_void_p),
                ("score_stride", c_int64), ("temperature", c_float),
                ("banned", ctypes.POINTER(c_int32)), ("n_banned", c_int),
                ("stop", ctypes.POINTER(c_int32)), ("n_stop", c_int), ("finished", c_void_p),
                ("row_mode", c_void_p), ("force_eos_all", c_int), ("eos_idx", c_int),
                ("col_dev", c_void_p)]


# name -> argtypes, in the order of include/metaseq_amd.h
SIGNATURES = {
    "msa_pack_weight_f16": [_P, _P, c_int, c_int, _P],
    "msa_unpack_weight_f16": [_P, _P, c_int, c_int, _P],
    "msa_pack_weight_i8": [_P, _P, c_int, c_int, _P],
    "msa_unpack_weight_i8": [_P, _P, c_int, c_int, _P],
    "msa_expand_weight_w8_f16": [_P, _P, _P, c_int, c_int, _P],
    "msa_layernorm_f16": [_P, _P, _P, _P, c_int64, c_int, c_float, c_uint, _P],
    "msa_residual_layernorm_f16": [_P, c_int, _P, _P, _P, _P, _P, c_int64, c_int, c_float, c_uint,
                                   _P],
    "msa_advance_len": [_P, _P, c_int, c_int, _P],
    "msa_embed_f16": [_P, c_int64, c_int, c_int, c_int, _P, c_int, _P, c_int, c_int, c_int, _P, _P,
                      _P, _P, _P, c_uint, _P],
    "msa_linear_f16": [_P, _P, _P, _P, _P, c_int64, c_int, c_int, c_uint, _P],
    "msa_linear_w8a16": [_P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_uint, _P],
    "msa_linear_partial_f16": [_P, _P, _P, c_int64, c_int, c_int, c_int, c_uint, _P],
    "msa_linear_partial_w8a16": [_P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_uint, _P],
    "msa_linear_default_splits": [c_int64, c_int, c_int],
    "msa_linear_default_splits_w8a16": [c_int64, c_int, c_int],
    "msa_linear_default_splits_rows": [c_int64, c_int, c_int],
    "msa_qkv_proj_f16": [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_uint, _P, _P],
    "msa_qkv_proj_w8a16": [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_uint, _P, _P],
    "msa_attention_f16": [_P, _P, _P, _P, c_int64, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                          c_uint, _P, _P],
    "msa_attention_split_f16": [_P, _P, _P, _P, c_int64, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                c_uint, _P, _P],
    "msa_attention_prefers_split": [c_int, c_int, c_int, c_int],
    "msa_greedy_select_f16": [_P, c_int64, c_int, c_int, c_float, _P, c_int, _P, c_int, _P, _P,
                              c_int, c_int, _P, c_int64, _P, c_int64, _P, _P],
    "msa_sample_topp_f16": [_P, c_int64, c_int, c_int, c_float, _P, _P, c_int, _P, c_int, _P, _P,
                            c_int, c_int, _P, c_float, _P, _P, _P, c_float, c_float, c_float,
                            c_float, _P, _P, c_int64, _P, c_int64, _P, c_int64, _P],
    "msa_log_softmax_f16": [_P, c_int64, c_int64, c_int, c_int, c_int, c_float, _P, c_int64,
                            c_int64, _P],
    "msa_target_logprob_f16": [_P, c_int64, c_int64, c_int, c_float, _P, _P, _P],
    "msa_lm_head_greedy_select_f16": [_P, _P, _P, _P, c_int, c_int, c_int, c_float, _P, c_int, _P,
                                      c_int, _P, _P, c_int, c_int, _P, c_int64, _P, c_int64, _P,
                                      _P],
    "msa_lm_head_greedy_select_noalloc_f16": [_P, _P, _P, c_int, c_int, c_int, c_float, _P, c_int,
                                              _P, c_int, _P, _P, c_int, c_int, _P, c_int64, _P,
                                              c_int64, _P, _P],
    "msa_decoder_create": [ctypes.POINTER(DecoderConfig), _P, _P, _P, _P, _P,
                           ctypes.POINTER(LayerWeights), ctypes.POINTER(c_void_p)],
    "msa_decoder_step": [_P, ctypes.POINTER(StepArgs), _P],
    "msa_probe_stream_read": [_P, c_int64, _P],
}
OTHER_SYMBOLS = ["msa_last_error", "msa_version", "msa_lm_head_select_workspace_bytes",
                 "msa_decoder_destroy", "msa_decoder_step_workspace_bytes",
                 "msa_attention_split_workspace_bytes"]

_lib = None


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "metaseq_amd: %s is missing - build it with `python -m metaseq_amd.csrc.build` "
            "(there is no non-HIP fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.msa_last_error.argtypes = []
    lib.msa_last_error.restype = c_char_p
    lib.msa_version.argtypes = []
    lib.msa_version.restype = c_int
    lib.msa_lm_head_select_workspace_bytes.argtypes = [c_int]
    lib.msa_lm_head_select_workspace_bytes.restype = c_int64
    lib.msa_decoder_destroy.argtypes = [_P]
    lib.msa_decoder_destroy.restype = None
    lib.msa_decoder_step_workspace_bytes.argtypes = [_P, c_int]
    lib.msa_decoder_step_workspace_bytes.restype = c_int64
    lib.msa_attention_split_workspace_bytes.argtypes = [c_int, c_int, c_int]
    lib.msa_attention_split_workspace_bytes.restype = c_int64
    _lib = lib
    return lib


def check(rc, lib=None):
    if rc == 0:
        return
    lib = lib or load()
    msg = lib.msa_last_error().decode("utf-8", "replace")
    if rc == -3:
        raise RuntimeError("metaseq_amd HIP failure: " + msg)
    raise ValueError("metaseq_amd: " + msg)


def ptr(t):
    """Device pointer of a torch tensor (or NULL for None)."""
    return None if t is None else t.data_ptr()


def stream_ptr():
    """hipStream_t of torch's current stream, so kernels order with torch's own work."""
    import torch

    return torch.cuda.current_stream().cuda_stream
