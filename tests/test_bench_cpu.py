"""CPU-side checks of the benchmark's bookkeeping: the algorithmic byte and flop counts the
roofline fractions are computed from, and the one-GPU contract of the command line."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402
from metaseq_amd import opt_config  # noqa: E402


def test_decode_step_bytes_of_the_headline_config():
    """OPT-6.7B shape, fp16, batch 32: 32 layers x (12 D^2 + 13 D) x 2 B of layer weights =
    12.888 GB, 0.412 GB of vocabulary projection, 16.78 MB of keys and values per attended
    position; 30.5 GB at 1025 positions and 34.8 GB at 1280."""
    cfg = opt_config("6.7b")
    L, D, V, B = 32, 4096, 50272, 32
    layers = L * (12 * D * D + 13 * D) * 2
    assert abs(layers - 12.888e9) < 2e6
    assert abs(V * D * 2 - 0.412e9) < 1e6
    per_pos = bench.step_bytes(cfg, B, 1001) - bench.step_bytes(cfg, B, 1000)
    assert per_pos == 2 * L * B * D * 2 == 16777216
    fixed = layers + 2 * D * 2 + V * D * 2 + 2 * L * B * D * 2
    assert bench.step_bytes(cfg, B, 1025) == fixed + 1025 * per_pos
    assert abs(bench.step_bytes(cfg, B, 1025) - 30.5e9) < 0.05e9
    assert abs(bench.step_bytes(cfg, B, 1280) - 34.8e9) < 0.05e9


def test_int8_step_bytes_count_one_byte_per_weight_plus_scales():
    cfg = opt_config("66b")
    L, D = cfg.decoder_layers, cfg.decoder_embed_dim
    d = bench.step_bytes(cfg, 64, 600, int8=False) - bench.step_bytes(cfg, 64, 600, int8=True)
    assert d == L * 12 * D * D - L * 9 * D * 2


def test_attention_bytes_and_prefill_flops():
    cfg = opt_config("6.7b")
    # K and V rows of every head read once, q read, output written
    assert bench.attn_bytes(cfg, 32, 1281) == 2 * 32 * 1281 * 4096 * 2 + 2 * 32 * 4096 * 2 == 672137216
    # 453 TFLOP for batch 32 x 1025 positions (attention counted un-causal: 17.6 TFLOP of it)
    fl = bench.prefill_flops(cfg, 32, 1025)
    assert abs(fl - 453e12) < 1e12
    assert abs(4.0 * 32 * 32 * 1025 * 1025 * 4096 - 17.6e12) < 0.1e12


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_cpu_baseline_is_a_measured_run_of_the_cpu_runnable_case():
    """The baseline leg runs the oracle's greedy generation on OPT-125m (batch 1, prompt 32, 32
    generated tokens) and reports decode tokens/s over the timed generations."""
    r = bench.cpu_baseline(warm=0, timed=1)
    assert r["kind"] == "port" and r["timing"] == "measured" and r["unit"] == "tokens/s"
    assert r["cores"] >= 1 and "OPT-125m" in r["sample"]
    assert r["value"] == pytest.approx(32 / r["decode_s_mean"])
    assert 0 < r["prefill_s_mean"] < r["decode_s_mean"]
