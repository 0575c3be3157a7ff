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


def test_counter_traffic_scales_the_readings_by_the_calibration_copy(tmp_path):
    """Counter files as the profiler writes them (one row per dispatch and counter), made up so
    that the answer is known: a FETCH_SIZE unit of 2 KiB, a WRITE_SIZE unit of 1 KiB, and
    attention launches that move exactly their algorithmic bytes plus 1 %."""
    import csv
    import json
    cfg = opt_config("6.7b")
    B, K, W, L = 32, 2, 1, cfg.decoder_layers
    S_end = 1030
    contexts = [S_end - 2, S_end - 1, S_end] + [S_end] * 5  # warm-up, two timed steps, timing loop
    rows_f = [("__amd_rocclr_copyBuffer", 524288.0), ("prefill_attention_kernelILi128EE", 9e9),
              ("__amd_rocclr_copyBuffer", 16.0)]
    rows_w = [("__amd_rocclr_copyBuffer", 1048576.0)]
    for S in contexts:
        read = 2 * B * S * 4096 * 2 + B * 4096 * 2
        for _ in range(L):
            rows_f.append(("attention_kernelILi128EEEvPKDF16_", 1.01 * read / 1024 / 2))
            rows_w.append(("attention_kernelILi128EEEvPKDF16_", 1.01 * B * 4096 * 2 / 1024))
    for name, rows, counter in (("f", rows_f, "FETCH_SIZE"), ("w", rows_w, "WRITE_SIZE")):
        os.makedirs(tmp_path / name)
        with open(tmp_path / name / "b_counter_collection.csv", "w", newline="") as fh:
            wr = csv.writer(fh)
            wr.writerow(["Kernel_Name", "Counter_Name", "Counter_Value"])
            for kernel, v in rows:
                wr.writerow([kernel, counter, v])
    run = tmp_path / "run.json"
    run.write_text("noise\n" + json.dumps({"steps": K, "warmup": W, "repeats": 1,
                                           "roofline": {"context": S_end}}) + "\n")
    r = bench.counter_traffic(str(tmp_path / "f" / "*.csv"), str(tmp_path / "w" / "*.csv"),
                              str(run), cfg, B)
    assert r["launches"] == len(contexts) * L
    assert abs(r["fetch_scale"] - 2.0) < 1e-12 and abs(r["write_scale"] - 1.0) < 1e-12
    assert abs(r["ratio"] - 1.01) < 1e-9
    with pytest.raises(SystemExit):  # a launch count that does not fit the run is refused
        run.write_text(json.dumps({"steps": K + 1, "warmup": W, "repeats": 1,
                                   "roofline": {"context": S_end}}))
        bench.counter_traffic(str(tmp_path / "f" / "*.csv"), str(tmp_path / "w" / "*.csv"),
                              str(run), cfg, B)


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
