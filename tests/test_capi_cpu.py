"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, and the Python binding's signature table matches the header."""
import ctypes
import os
import re

import pytest

from metaseq_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "metaseq_amd.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(msa_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = [a.strip() for a in m.group(2).split(",") if a.strip() and a.strip() != "void"]
        decls[m.group(1)] = args
    return decls


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_capi.LIB_PATH):
        from metaseq_amd.csrc.build import build
        build(force=True, verbose=False)
    lib = ctypes.CDLL(_capi.LIB_PATH)
    decls = _declared()
    assert len(decls) >= 12
    for name in decls:
        assert hasattr(lib, name), name


def test_binding_table_matches_header_arity():
    decls = _declared()
    for name, argtypes in _capi.SIGNATURES.items():
        assert name in decls, name
        assert len(argtypes) == len(decls[name]), (name, len(argtypes), decls[name])
    for name in decls:
        assert name in _capi.SIGNATURES or name in _capi.OTHER_SYMBOLS, name


def test_loader_reports_version_and_fails_loudly_without_library(monkeypatch, tmp_path):
    lib = _capi.load()
    assert lib.msa_version() >= 1
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(RuntimeError, match="no non-HIP fallback"):
        _capi.load()


def test_argument_validation_needs_no_gpu():
    """Entry points reject bad arguments before touching the device."""
    lib = _capi.load()
    assert lib.msa_layernorm_f16(None, None, None, None, 1, 64, 1e-5, 0, None) == -1
    assert b"null pointer" in lib.msa_last_error()
    one = ctypes.c_void_p(16)
    assert lib.msa_linear_f16(one, one, None, None, one, 4, 16, 40, 0, None) == -1
    assert b"multiple of 32" in lib.msa_last_error()
    assert lib.msa_attention_f16(one, one, one, None, 0, one, 1, 1, 64, 2, 9, 10, 0, None, None) == -2
    with pytest.raises(ValueError):
        _capi.check(-2, lib)
    # split-K counts that would leave a slice of the partial sums unwritten are refused
    assert lib.msa_linear_partial_f16(one, one, one, 58, 50272, 160, 4, 2, None) == -1
    assert b"leaves a K range empty" in lib.msa_last_error()
    assert lib.msa_linear_partial_w8a16(one, one, one, one, 52, 8000, 768, 8, 2, None) == -1
    assert b"leaves a K range empty" in lib.msa_last_error()


def test_decoder_handle_is_host_only_bookkeeping():
    """msa_decoder_create validates and copies a pointer table without touching a GPU; the
    workspace size grows with the row count; a bad configuration or a missing pointer is
    refused."""
    lib = _capi.load()
    conf = _capi.DecoderConfig(2, 128, 2, 512, 64, 40, 1, 0)
    table = (_capi.LayerWeights * 2)()
    for t in table:
        for name, _ in _capi.LayerWeights._fields_:
            setattr(t, name, 4096)
    h = ctypes.c_void_p()
    one = ctypes.c_void_p(4096)
    assert lib.msa_decoder_create(ctypes.byref(conf), one, one, one, one, one, table,
                                  ctypes.byref(h)) == 0
    w8, w40 = (lib.msa_decoder_step_workspace_bytes(h, b) for b in (8, 40))
    w100 = lib.msa_decoder_step_workspace_bytes(h, 100)
    assert 0 < w8 < w40 and w100 > 0 and lib.msa_decoder_step_workspace_bytes(h, 129) == 0
    args = _capi.StepArgs()
    assert lib.msa_decoder_step(h, ctypes.byref(args), None) == -1     # nothing filled in
    lib.msa_decoder_destroy(h)
    table[1].fc2_bias = None
    assert lib.msa_decoder_create(ctypes.byref(conf), one, one, one, one, one, table,
                                  ctypes.byref(h)) == -1
    assert b"layer 1" in lib.msa_last_error()
    bad = _capi.DecoderConfig(2, 160, 2, 512, 64, 40, 1, 0)            # head_dim 80
    assert lib.msa_decoder_create(ctypes.byref(bad), one, one, one, one, one, table,
                                  ctypes.byref(h)) == -1
