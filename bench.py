#!/usr/bin/env python3
"""Decode-throughput benchmark of the OPT incremental-decoding forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 6.7b]

Workload (BASELINE config 3): OPT-6.7B shape, fp16, seeded random weights, batch 32, prompt
EOS + 1024 uniform-random ids, greedy decoding.  A "step" is one per-token forward of the
whole batch (embedding, 32 layers, final LayerNorm, vocabulary projection, fused greedy
selection) at the context length the generation has reached.  Weights, KV cache and token
buffers are resident in HBM before the timed region; the prompt is prefetched through the
library's own prefill kernels.

Prints ONE JSON line: decode tokens/s, the HBM-roofline record of the dominant kernel (decode
attention, timed live with device events on the launch stream) and the CPU baseline: the
oracle restatement of the reference forward and greedy loop, fp32, measured on this host's
cores on the reference's CPU-runnable case (OPT-125m, batch 1, prompt 32, 32 generated tokens).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # MI355X HBM3E, bytes/s
MFMA_PEAK = 2.5e15  # dense fp16 MFMA, flop/s
# HBM bytes per decode-attention launch over its algorithmic bytes, from rocprofv3 FETCH_SIZE +
# WRITE_SIZE scaled by a 1 GiB copy (profiles/decode_attention_opt6.7b_bs32_pmc_traffic.txt):
# 540.4 MB measured for 540.0 MB algorithmic.
ATTN_TRAFFIC_RATIO = 540.4 / 540.0

CONFIGS = {
    # name: (size, batch, prompt, generate)
    "125m": ("125m", 1, 32, 32),
    "1.3b": ("1.3b", 8, 512, 128),
    "6.7b": ("6.7b", 32, 1024, 256),
    "30b": ("30b", 16, 2048, 128),
    "66b-int8": ("66b", 64, 512, 128),
}


def step_bytes(cfg, B, S, int8=False):
    """Algorithmic HBM bytes of one decode step attending S positions (new token included)."""
    L, D, V = cfg.decoder_layers, cfg.decoder_embed_dim, cfg.vocab_size
    w = 1 if int8 else 2
    weights = L * (12 * D * D * w + 13 * D * 2) + 2 * D * 2
    if int8:
        weights += L * 9 * D * 2
    return weights + V * D * 2 + 2 * L * B * S * D * 2 + 2 * L * B * D * 2


def prefill_flops(cfg, B, T):
    """2*(12*D^2*L + V*D)*B*T for the GEMMs + 4*L*B*T^2*D for attention counted un-causal."""
    L, D, V = cfg.decoder_layers, cfg.decoder_embed_dim, cfg.vocab_size
    return 2.0 * (12 * D * D * L + V * D) * B * T + 4.0 * L * B * T * T * D


def attn_bytes(cfg, B, S):
    """Algorithmic bytes of one decode-attention launch (one layer): K and V rows read, q read,
    output written."""
    D = cfg.decoder_embed_dim
    return 2 * B * S * D * 2 + 2 * B * D * 2


def counter_traffic(fetch_glob, write_glob, run_json, cfg, B):
    """HBM bytes per decode-attention launch over its algorithmic bytes, from the counter files
    of two earlier runs of this program under the profiler:

        rocprofv3 --pmc FETCH_SIZE --output-format csv -d DIR_F -o b -- python3 bench.py \
            --steps 4 --warmup 1 --repeats 1 --no-cpu-baseline --pmc-calibration > RUN.json
        rocprofv3 --pmc WRITE_SIZE ... (the same command)

    ``fetch_glob`` / ``write_glob`` match their ``*counter_collection.csv``; ``run_json`` holds
    the line either of them printed (its steps, warm-up steps, repeats and context say which
    contexts the traced launches attended).  Each counter is scaled by what it reads for the
    1 GiB device copy --pmc-calibration adds (1 048 576 KiB read and as much written)."""
    import csv
    import glob

    def readings(pattern, counter):
        attn, copy = [], 0.0
        paths = glob.glob(pattern, recursive=True)
        if not paths:
            raise SystemExit("bench.py: no counter file matches %r" % pattern)
        for path in paths:
            for r in csv.DictReader(open(path)):
                if r["Counter_Name"] != counter:
                    continue
                name, v = r["Kernel_Name"], float(r["Counter_Value"])
                if "attention_kernel" in name and "prefill" not in name:
                    attn.append(v)
                elif "copyBuffer" in name:
                    copy = max(copy, v)
        if not attn or copy <= 0:
            raise SystemExit("bench.py: %r holds no %s readings of the decode attention kernel "
                             "and the calibration copy" % (pattern, counter))
        return attn, copy

    run = None
    for line in open(run_json):
        if line.startswith("{"):
            run = json.loads(line)
    if run is None:
        raise SystemExit("bench.py: no result line in %r" % run_json)
    K, W, R = run["steps"], run["warmup"], run.get("repeats", 1)
    S_end, L = run["roofline"]["context"], cfg.decoder_layers
    # the contexts of every traced launch: warm-up steps once, the timed window R times, then
    # the timing loop of the attention kernel (one untimed + four timed passes over the layers)
    contexts = [S_end - K - W + 1 + j for j in range(W)]
    contexts += [S_end - K + 1 + j for j in range(K)] * R
    contexts += [S_end] * 5
    algorithmic = sum(attn_bytes(cfg, B, S) for S in contexts) / len(contexts)
    fetch, fcopy = readings(fetch_glob, "FETCH_SIZE")
    write, wcopy = readings(write_glob, "WRITE_SIZE")
    if len(fetch) != len(contexts) * L or len(write) != len(fetch):
        raise SystemExit("bench.py: %d / %d traced attention launches, %d expected from %r"
                         % (len(fetch), len(write), len(contexts) * L, run_json))
    kib = float(1 << 20)
    measured = (sum(fetch) / len(fetch) * kib / fcopy + sum(write) / len(write) * kib / wcopy) * 1024
    return {"ratio": measured / algorithmic, "launches": len(fetch),
            "fetch_scale": kib / fcopy, "write_scale": kib / wcopy,
            "measured_bytes_per_launch": measured, "algorithmic_bytes_per_launch": algorithmic}


def _host_cores():
    """Threads to use on this host: its CPU share, not what the machine reports in total."""
    n = os.cpu_count() or 1
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except (AttributeError, OSError):
        pass
    for var in ("OMP_NUM_THREADS", "MAX_JOBS"):
        v = os.environ.get(var, "")
        if v.isdigit() and int(v) > 0:
            n = min(n, int(v))
    return max(1, n)


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(warm=5, timed=5, seed=1234):
    """The reference's CPU-runnable case, measured: the oracle restatement of the reference
    forward and greedy loop (fp32, torch CPU ops, every host core) on OPT-125m, batch 1, prompt
    EOS + 32 ids, greedy decoding of 32 tokens; `warm` untimed generations, then `timed` timed
    ones.  As for the GPU figure, the value is decode tokens/s: generated tokens over the time of
    the per-token forwards and their selection, the prefill excluded (reported beside it)."""
    import torch

    from metaseq_amd import opt_config, random_prompts, random_state_dict
    from oracle.opt_oracle import OracleConfig, OracleDecoder, greedy_generate

    size, B, P, G = CONFIGS["125m"]
    cfg = opt_config(size)
    cores = _host_cores()
    torch.set_num_threads(cores)
    sd = random_state_dict(cfg, seed=seed, dtype=torch.float32)
    oc = OracleConfig(cfg.decoder_layers, cfg.decoder_embed_dim, cfg.decoder_attention_heads,
                      cfg.decoder_ffn_embed_dim, cfg.vocab_size, cfg.max_target_positions)
    dec = OracleDecoder(oc, sd, dtype=torch.float32)
    src = random_prompts(cfg, B, P, seed=4321)
    n0 = src.shape[1]
    max_len = n0 + G + 1
    marks = []

    def timed_decoder(tokens, incremental_state=None):
        out = dec(tokens, incremental_state=incremental_state)
        marks.append(time.perf_counter())  # end of every forward; the first is the prefill
        return out
    timed_decoder.max_positions = dec.max_positions

    decode_s, prefill_s = [], []
    with torch.no_grad():
        for i in range(warm + timed):
            del marks[:]
            t0 = time.perf_counter()
            greedy_generate(timed_decoder, src, max_len_b=max_len, min_len=max_len - 1)
            t1 = time.perf_counter()
            if i >= warm:
                prefill_s.append(marks[0] - t0)
                decode_s.append(t1 - marks[0])
    mean = sum(decode_s) / len(decode_s)
    std = (sum((d - mean) ** 2 for d in decode_s) / len(decode_s)) ** 0.5
    return {
        "value": B * G / mean, "unit": "tokens/s", "cores": cores, "kind": "port",
        "timing": "measured",
        # another model, batch and context than the GPU headline: not a speed-up denominator
        "comparable_to_headline": False,
        "cpu": _cpu_model(),
        "sample": ("oracle restatement of the reference forward + greedy loop, fp32, on the "
                   "reference's CPU-runnable case: OPT-125m, batch %d, prompt EOS+%d, %d generated "
                   "tokens; %d warm-up + %d timed generations, prefill excluded"
                   % (B, P, G, warm, timed)),
        "ms_per_step": mean / G * 1e3,
        "decode_s_mean": mean, "decode_s_std": std,
        "prefill_s_mean": sum(prefill_s) / len(prefill_s),
    }


def cpu_baseline_same_shape(size, B, S, seed=1234):
    """Context figure beside the measured baseline: oracle (fp32, torch CPU ops) decode steps at
    the GPU workload's own shape with 1 and 3 layers; per-layer and fixed (embedding + final LN +
    vocabulary projection) costs are separated and EXTRAPOLATED to the full depth, which the
    host could not hold or finish in the benchmark's time."""
    import torch

    from metaseq_amd import opt_config, random_state_dict
    from oracle.opt_oracle import OracleConfig, OracleDecoder

    full = opt_config(size)
    cores = _host_cores()
    torch.set_num_threads(cores)
    times = {}
    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(4, full.vocab_size, (B, S + 4), generator=g)
    toks[:, 0] = 2
    for nl in (1, 3):
        cfg = opt_config(size, decoder_layers=nl)
        sd = random_state_dict(cfg, seed=seed, dtype=torch.float32)
        oc = OracleConfig(nl, cfg.decoder_embed_dim, cfg.decoder_attention_heads,
                          cfg.decoder_ffn_embed_dim, cfg.vocab_size, cfg.max_target_positions)
        dec = OracleDecoder(oc, sd, dtype=torch.float32)
        del sd
        H, hd = cfg.decoder_attention_heads, cfg.head_dim
        inc = {}
        for lid in dec.layer_ids:
            inc[lid + ".attn_state"] = {
                "prev_key": torch.randn(B, H, S - 1, hd, generator=g),
                "prev_value": torch.randn(B, H, S - 1, hd, generator=g),
                "prev_key_padding_mask": None,
            }
        ts = []
        for i in range(3):  # 1 warm-up + 2 timed steps, the cache grows by one each
            t0 = time.perf_counter()
            dec(toks[:, :S + i], incremental_state=inc)
            ts.append(time.perf_counter() - t0)
        times[nl] = sum(ts[1:]) / 2
        del dec, inc
    per_layer = (times[3] - times[1]) / 2
    fixed = max(times[1] - per_layer, 0.0)
    t_full = fixed + full.decoder_layers * per_layer
    return {
        "value": B / t_full, "unit": "tokens/s", "cores": cores, "kind": "port",
        "timing": "extrapolated",
        "sample": ("oracle fp32 decode steps at the GPU workload's shape (B=%d, context %d) with "
                   "1 and 3 layers, 2 timed steps each; per-layer %.3f s and fixed %.3f s "
                   "extrapolated to %d layers" % (B, S, per_layer, fixed, full.decoder_layers)),
        "ms_per_step": t_full * 1e3,
    }


def torch_eager_steps(cfg, sd, B, S_first, K, warmup, dev):
    """The reference's per-token forward written with stock PyTorch operators in fp16 on the same
    GPU (linear / layer_norm / bmm / softmax, key and value history grown with torch.cat as
    metaseq/modules/multihead_attention.py:451-467 does), greedy selection included; K timed
    steps whose first one attends S_first positions.  Context figure only: what the same
    arithmetic costs when every operator is a library call."""
    import torch
    import torch.nn.functional as F

    L, D, H, hd = (cfg.decoder_layers, cfg.decoder_embed_dim, cfg.decoder_attention_heads,
                   cfg.head_dim)
    w = lambda k: sd["decoder." + k]
    g = torch.Generator(device=dev).manual_seed(99)
    n_hist = S_first - 1 - warmup
    hist = [[torch.randn(B * H, n_hist, hd, device=dev, dtype=torch.float16, generator=g)
             for _ in range(2)] for _ in range(L)]
    tok = torch.randint(4, cfg.vocab_size, (B,), device=dev, generator=g)

    def step(tok, n):
        pos = torch.full((B,), n + 2, device=dev, dtype=torch.long)  # pad index 1 + 1 + n
        x = F.embedding(tok, w("embed_tokens.weight")) + F.embedding(pos, w("embed_positions.weight"))
        for i in range(L):
            p = "layers.%d." % i
            h = F.layer_norm(x, (D,), w(p + "self_attn_layer_norm.weight"),
                             w(p + "self_attn_layer_norm.bias"))
            k, v, q = F.linear(h, w(p + "self_attn.qkv_proj.weight"),
                               w(p + "self_attn.qkv_proj.bias")).split(D, dim=-1)
            q = (q * hd ** -0.5).reshape(B * H, 1, hd)
            hist[i][0] = torch.cat([hist[i][0], k.reshape(B * H, 1, hd)], dim=1)
            hist[i][1] = torch.cat([hist[i][1], v.reshape(B * H, 1, hd)], dim=1)
            pr = F.softmax(torch.bmm(q, hist[i][0].transpose(1, 2)), dim=-1,
                           dtype=torch.float32).to(x.dtype)
            o = torch.bmm(pr, hist[i][1]).reshape(B, D)
            x = F.linear(o, w(p + "self_attn.out_proj.weight")) + w(p + "self_attn.out_proj.bias") + x
            h = F.layer_norm(x, (D,), w(p + "final_layer_norm.weight"), w(p + "final_layer_norm.bias"))
            u = F.relu(F.linear(h, w(p + "fc1.weight"), w(p + "fc1.bias")))
            x = x + F.linear(u, w(p + "fc2.weight"), w(p + "fc2.bias"))
        x = F.layer_norm(x, (D,), w("layer_norm.weight"), w("layer_norm.bias"))
        lprobs = F.log_softmax(F.linear(x, w("embed_tokens.weight")).float(), dim=-1)
        return lprobs.max(dim=-1)[1]

    with torch.no_grad():
        n = n_hist
        for _ in range(warmup):
            tok = step(tok, n)
            n += 1
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(K):
            tok = step(tok, n)
            n += 1
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / K
    return {"value": B / dt, "unit": "tokens/s", "ms_per_step": dt * 1e3,
            "what": "stock PyTorch fp16 operators, same shapes, same GPU, %d steps attending "
                    "%d..%d positions" % (K, S_first, S_first + K - 1)}


def service_throughput(config, slots, prefill_batch, prefill_wait, seed=1):
    """A request-level run beside the headline: ``ContinuousBatcher`` with ``slots`` rows over
    the configuration's model shape (random weights), three requests per slot with prompts of
    16-95 random ids and 32-127 new tokens, every other one sampled (temperature 0.8, top-p
    0.9).  Times everything from the first admission to the last answer, host work included."""
    import torch

    from metaseq_amd import (Dictionary, GeneratorInterface, TransformerLanguageModel, opt_config,
                             random_state_dict)
    from metaseq_amd.service import ContinuousBatcher
    size = CONFIGS[config][0]
    int8 = config.endswith("int8")
    cfg = opt_config(size, max_target_positions=2048)
    dev = torch.device("cuda:0")
    sd = random_state_dict(cfg, seed=1234, dtype=torch.float16, device=dev)
    model = TransformerLanguageModel.build_model(cfg, sd, device=dev)
    del sd
    if int8:
        model.decoder.quantize_int8_()
    torch.cuda.empty_cache()
    engine = ContinuousBatcher(GeneratorInterface(model, Dictionary(cfg.vocab_size)), slots=slots,
                               capacity=256, prefill_batch=prefill_batch,
                               prefill_wait=prefill_wait)
    g = torch.Generator().manual_seed(seed)

    def run(count, shortest, longest):
        replies = []
        for i in range(count):
            n = int(torch.randint(16, 96, (1,), generator=g))
            options = dict(max_tokens=int(torch.randint(shortest, longest, (1,), generator=g)),
                           min_tokens=shortest)
            if i % 2:
                options.update(temperature=0.8, top_p=0.9)
            prompt = torch.randint(4, cfg.vocab_size, (n,), generator=g).tolist()
            replies.append(engine.submit(prompt, **options))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while engine.step():
            pass
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        new = 0
        for r in replies:
            result = r.get_nowait()[1]
            if isinstance(result, Exception):
                raise result
            new += len(result[0]["tokens"])
        return seconds, new

    # untimed: one short request per slot, so that first uses (kernel attributes, the allocator's
    # and the engine's buffers at this width) are not in the timed run
    run(slots, 8, 16)
    steps0, rows0 = engine.steps, engine.rows_stepped
    seconds, new = run(3 * slots, 32, 128)
    steps, rows = engine.steps - steps0, engine.rows_stepped - rows0
    return {
        "metric": "continuous batching, new tokens/s end to end, OPT-%s shape, 1xMI355X" % size,
        "value": new / seconds, "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
        "dtype": "f16" if not int8 else "int8-weights/f16", "data": "synthetic",
        "config": {"workload": "%d requests (prompts of 16-95 ids, 32-127 new tokens, half of "
                               "them sampled) through %d slots" % (3 * slots, slots),
                   "slots": slots, "prefill_batch": prefill_batch, "prefill_wait": prefill_wait},
        "warmup": "%d requests of 8-15 new tokens" % slots,
        "seconds": seconds, "new_tokens": new, "decode_steps": steps,
        "rows_per_step": rows / max(1, steps),
        "ms_per_step_overall": seconds / max(1, steps) * 1e3,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed decode steps (default: the workload's generation length minus "
                         "the warm-up steps, so warm-up + timed = the configured decode length)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--repeats", type=int, default=5,
                    help="how many times the window of exactly --steps timed steps is run (over "
                         "the same contexts: the cache length is wound back); ms_per_step is "
                         "their mean, reported with its standard deviation and minimum")
    ap.add_argument("--config", default="6.7b", choices=sorted(CONFIGS))
    ap.add_argument("--batch", type=int, default=None,
                    help="override the configuration's batch size (service-style batches)")
    ap.add_argument("--prompt", type=int, default=None,
                    help="override the configuration's prompt length")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-same-shape", action="store_true",
                    help="also time the oracle on the host at the GPU workload's own shape "
                         "(1 and 3 layers, extrapolated to the full depth)")
    ap.add_argument("--graph", action="store_true",
                    help="replay the captured decode-step hipGraph instead of launching every "
                         "kernel from Python (measured slower on this ROCm: 5.81 vs 5.66 ms/step)")
    ap.add_argument("--unfused-select", action="store_true",
                    help="store the logits and run the stand-alone selection kernel instead of "
                         "selecting inside the vocabulary projection (for comparison)")
    ap.add_argument("--python-step", action="store_true",
                    help="drive every kernel of a decode step from Python instead of the one-call "
                         "msa_decoder_step (same kernels, same results; for comparison)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy, the known-size kernel that "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--traffic-from", nargs=3, metavar=("FETCH_CSV", "WRITE_CSV", "RUN_JSON"),
                    help="take roofline.traffic from the counter files of two earlier "
                         "--pmc-calibration runs under rocprofv3 (--pmc FETCH_SIZE, --pmc "
                         "WRITE_SIZE; glob patterns of their counter_collection.csv) and the "
                         "result line one of them printed, instead of the ratio on record")
    ap.add_argument("--service", type=int, default=0, metavar="SLOTS",
                    help="instead of the headline run: requests through the continuous "
                         "batching engine with this many slots, one JSON line of its own")
    ap.add_argument("--prefill-batch", type=int, default=1,
                    help="--service: requests that may share one prefill")
    ap.add_argument("--prefill-wait", type=int, default=0,
                    help="--service: steps admissible requests may be held back for company")
    ap.add_argument("--torch-eager", action="store_true",
                    help="also time the same decode steps written with stock PyTorch fp16 "
                         "operators on this GPU (reported as torch_eager_same_gpu)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (nothing in the "
              "path uses a second device)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    from metaseq_amd import (Dictionary, SequenceGenerator, TransformerLanguageModel, _capi,
                             opt_config, random_prompts, random_state_dict)

    if not os.path.exists(_capi.LIB_PATH):
        from metaseq_amd.csrc.build import build
        build(force=True)
    if args.service:
        print(json.dumps(service_throughput(args.config, args.service, args.prefill_batch,
                                            args.prefill_wait)))
        return

    size, B, P, G = CONFIGS[args.config]
    B, P = args.batch or B, args.prompt or P
    int8 = args.config.endswith("int8")
    W = args.warmup
    K = args.steps if args.steps is not None else max(1, G - W)
    total_gen = max(G, K + W + 1)
    n0 = P + 1
    max_len = n0 + total_gen + 1
    cfg = opt_config(size, max_target_positions=max(2048, max_len))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.pmc_calibration:
        a = torch.ones(1 << 29, dtype=torch.float16, device=dev)
        bcopy = torch.empty_like(a)
        for _ in range(3):
            bcopy.copy_(a)
        torch.cuda.synchronize()
        del a, bcopy
        torch.cuda.empty_cache()

    t0 = time.time()
    sd = random_state_dict(cfg, seed=1234, dtype=torch.float16, device=dev)
    model = TransformerLanguageModel.build_model(cfg, sd, device=dev)
    del sd
    if int8:
        model.decoder.quantize_int8_()
    torch.cuda.empty_cache()
    src = random_prompts(cfg, B, P, seed=4321, device=dev)
    gen = SequenceGenerator([model], Dictionary(cfg.vocab_size), max_len_b=max_len,
                            min_len=max_len - 1)
    lib = _capi.load()
    decoder = model.decoder
    decoder.kv_cache_capacity = max_len
    decoder.native_step = not args.python_step

    tokens = torch.full((B, max_len), 1, dtype=torch.long, device=dev)
    scores = torch.zeros(B, max_len, dtype=torch.float32, device=dev)
    finished = torch.zeros(B, dtype=torch.uint8, device=dev)
    tokens[:, :n0] = src
    # the first prefill also packs the weights and grows the allocator's pools (reported as
    # prefill_cold_s); the timed one is the second, as a serving process would see it
    prefill_times = []
    for _ in range(2):
        inc = {}
        torch.cuda.synchronize()
        t1 = time.time()
        logits = model(tokens[:, :n0], incremental_state=inc)[0]
        step_logits = logits[:, -1, :].contiguous()
        del logits
        torch.cuda.synchronize()
        prefill_times.append(time.time() - t1)
    prefill_cold_s, prefill_s = prefill_times

    st = None
    if args.graph and B <= 64:  # (a captured step selects inside the vocabulary projection)
        st = gen.static_state(decoder, decoder.get_cache(inc), tokens, scores, finished,
                              step_logits)

    min_len = max_len - 1
    fused = st is None and B <= 128 and not args.unfused_select
    if fused:
        # the generator's fast path: the token at n0 comes from the prefill logits, every later
        # one is chosen inside the decode step's vocabulary projection
        gen._select(lib, step_logits, n0, min_len, max_len, finished, tokens, scores)

    def one_step(step, step_logits):
        if st is not None:  # selection + forward + length advance as one graph replay
            gen._graph_step(lib, st, step, min_len, max_len)
            return st["logits"]
        if fused:  # forward over the history up to `step`, selection of the token at step + 1
            nxt = step + 1
            decoder.forward_select(
                tokens[:, :nxt], inc, temperature=gen.temperature,
                banned=gen._banned(nxt, min_len), stop=gen.stop, finished=finished,
                force_eos=nxt >= max_len - 1, eos=gen.eos, tok_out=tokens[:, nxt],
                tok_stride=tokens.stride(0), score_out=scores[:, nxt],
                score_stride=scores.stride(0))
            return None
        gen._select(lib, step_logits, step, min_len, max_len, finished, tokens, scores)
        out = decoder(tokens[:, :step + 1], incremental_state=inc)[0]
        return out.view(B, -1)

    step = n0
    for _ in range(W):
        step_logits = one_step(step, step_logits)
        step += 1
    torch.cuda.synchronize()
    S_first = step + 1  # positions attended by the first timed forward
    cache = decoder.get_cache(inc)
    start_step, start_len, start_logits = step, cache.length, step_logits
    R = max(1, args.repeats) if st is None else 1  # a replayed graph keeps its length on the device
    walls, gpus = [], []
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(R):
        # every window times exactly K steps over the same contexts: wind the history back (the
        # steps are deterministic, so they rewrite the same tokens, keys and values)
        step, cache.length, step_logits = start_step, start_len, start_logits
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        ev0.record()
        for _ in range(K):
            step_logits = one_step(step, step_logits)
            step += 1
        ev1.record()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - wall0) / K)
        gpus.append(ev0.elapsed_time(ev1) / 1e3 / K)
    t_step = sum(walls) / R
    t_std = (sum((w - t_step) ** 2 for w in walls) / R) ** 0.5
    gpu_s = sum(gpus) / R * K
    S_last = step
    S_mean = (S_first + S_last) / 2.0
    bytes_mean = sum(step_bytes(cfg, B, s, int8) for s in range(S_first, S_last + 1)) / K
    fracs = [bytes_mean / w / HBM_PEAK for w in walls]
    frac_mean = sum(fracs) / R
    frac_std = (sum((f - frac_mean) ** 2 for f in fracs) / R) ** 0.5

    # ---- live timing of the dominant kernel: decode attention over every layer's cache ----
    S_probe = cache.length
    D, H, hd = cfg.decoder_embed_dim, cfg.decoder_attention_heads, cfg.head_dim
    q = torch.randn(B, D, device=dev).half()
    o = torch.empty_like(q)
    stream = _capi.stream_ptr()
    reps = 4

    def attn_all_layers():
        for i in range(cfg.decoder_layers):
            _capi.check(lib.msa_attention_f16(q.data_ptr(), cache.k(i).data_ptr(),
                                              cache.v(i).data_ptr(), None, 0, o.data_ptr(), B, H,
                                              hd, 1, S_probe - 1, cache.capacity, 0, None, stream))
    attn_all_layers()
    torch.cuda.synchronize()
    a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a0.record()
    for _ in range(reps):
        attn_all_layers()
    a1.record()
    torch.cuda.synchronize()
    attn_s = a0.elapsed_time(a1) / 1e3 / (reps * cfg.decoder_layers)
    ab = attn_bytes(cfg, B, S_probe)
    achieved = ab / attn_s / 1e9

    # ---- what a plain streaming read reaches on this GPU (context for the fractions of the
    # published peak): the library's probe kernel over slices of a 4 GiB region, one launch per
    # slice so that every launch reads cold memory, as the step's kernels do
    probe = torch.empty(1 << 31, dtype=torch.float16, device=dev).zero_()
    probe_bytes = probe.numel() * 2

    def loop_time(fn, n):
        """Average seconds per call of fn(i), i = 0 .. n - 1, after one untimed round."""
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        a0.record()
        for i in range(n):
            fn(i)
        a1.record()
        torch.cuda.synchronize()
        return a0.elapsed_time(a1) / 1e3 / n

    def plain_read_GBps(nbytes):
        nbytes = max(16, min(probe_bytes, int(nbytes)) // 16 * 16)
        slices = max(1, probe_bytes // nbytes)
        n = max(5, min(slices, 64))
        t = loop_time(lambda i: _capi.check(lib.msa_probe_stream_read(
            probe.data_ptr() + (i % slices) * nbytes, nbytes, stream)), n)
        return nbytes / t / 1e9

    stream_read = plain_read_GBps(probe_bytes)
    attn_ceiling = plain_read_GBps(ab)

    # ---- the step's other kernels, each timed live over every layer's weights in turn (cold
    # reads, as in the step) next to a plain read of the same number of bytes
    kernels = {"attention": {"bytes": ab, "us": attn_s * 1e6, "GBps": achieved,
                             "frac_of_peak": achieved * 1e9 / HBM_PEAK,
                             "plain_read_GBps_at_size": attn_ceiling,
                             "frac_of_plain_read": achieved / attn_ceiling}}
    if B <= 128:
        from metaseq_amd._capi import MSA_IN_PACKED, MSA_OUT_PACKED
        F, L, V = cfg.decoder_ffn_embed_dim, cfg.decoder_layers, cfg.vocab_size
        wb = 1 if int8 else 2
        bufs = decoder._step_buffers(cache, B)
        layers = decoder.layers
        S0 = cache.length - 1
        IN, OUT = MSA_IN_PACKED, MSA_OUT_PACKED
        tok1 = torch.zeros(B, dtype=torch.long, device=dev)
        sc1 = torch.zeros(B, dtype=torch.float32, device=dev)
        fin1 = torch.zeros(B, dtype=torch.uint8, device=dev)

        def lm_head(i):
            decoder._select_from(lib, bufs["h"], B, 1.0, [1], [], fin1, None, False, 2, tok1, 1,
                                 sc1, 1, None)
        flush_bytes = 1 << 29  # evicts the one vocabulary matrix between its launches

        def flush(i):
            _capi.check(lib.msa_probe_stream_read(probe.data_ptr() + (i % 4) * flush_bytes,
                                                  flush_bytes, stream))
        t_flush = loop_time(flush, 8)
        t_lm = loop_time(lambda i: (flush(i), lm_head(i)), 8) - t_flush
        timed = {
            "qkv_proj": (3 * D * D * wb, loop_time(lambda i: decoder._qkv(
                lib, stream, bufs["h"], layers[i].self_attn.qkv_proj, bufs["q"], cache.k(i),
                cache.v(i), B, 1, H, hd, S0, cache.capacity, D, IN, None), L)),
            "out_proj (split-K partial sums)": (D * D * wb, loop_time(
                lambda i: decoder._linear_partial(lib, stream, bufs["o"],
                                                  layers[i].self_attn.out_proj, bufs["part"], B,
                                                  D, D, bufs["S_o"]), L)),
            "fc1": (F * D * wb, loop_time(lambda i: decoder._linear(
                lib, stream, bufs["h"], layers[i].fc1, B, F, D, relu=True, out=bufs["u"],
                flags=IN | OUT), L)),
            "fc2 (split-K partial sums)": (D * F * wb, loop_time(
                lambda i: decoder._linear_partial(lib, stream, bufs["u"], layers[i].fc2,
                                                  bufs["part"], B, D, F, bufs["S_f"]), L)),
            "vocabulary projection + selection": (V * D * 2, t_lm),
        }
        for name, (nbytes, t) in timed.items():
            ceiling = plain_read_GBps(nbytes)
            kernels[name] = {"bytes": nbytes, "us": t * 1e6, "GBps": nbytes / t / 1e9,
                             "frac_of_peak": nbytes / t / HBM_PEAK,
                             "plain_read_GBps_at_size": ceiling,
                             "frac_of_plain_read": nbytes / t / 1e9 / ceiling}
        t_ln = loop_time(lambda i: _capi.check(lib.msa_residual_layernorm_f16(
            bufs["part"].data_ptr(), bufs["S_o"], layers[i].self_attn.out_proj.bias.data_ptr(),
            bufs["x"].data_ptr(), layers[i].final_layer_norm.weight.data_ptr(),
            layers[i].final_layer_norm.bias.data_ptr(), bufs["h"].data_ptr(), B, D, 1e-5, OUT,
            stream)), L)
        kernels["bias + residual + LayerNorm tail"] = {"bytes": 0, "us": t_ln * 1e6,
                                                        "launches_per_layer": 2}
        per_layer = (attn_s + sum(timed[k][1] for k in timed if "vocabulary" not in k) + 2 * t_ln)
        kernels["sum_of_kernels_ms_per_step"] = (L * per_layer + t_lm + t_ln) * 1e3
    del probe

    if args.traffic_from:
        counters = counter_traffic(*args.traffic_from, cfg, B)
        traffic = ab * counters["ratio"]
        traffic_source = dict(counters, files=list(args.traffic_from))
    elif args.config == "6.7b" and (B, P) == CONFIGS["6.7b"][1:3]:
        traffic = ab * ATTN_TRAFFIC_RATIO
        traffic_source = ("ratio %.4f on record in profiles/decode_attention_opt6.7b_bs32_pmc_"
                          "traffic.txt; --traffic-from re-derives it from fresh counter files"
                          % ATTN_TRAFFIC_RATIO)
    else:
        traffic = traffic_source = None
    result = {
        "metric": ("decode tokens/sec + % HBM roofline, OPT-6.7B-shape fp16 bs32, 1xMI355X"
                   if args.config == "6.7b" and (B, P) == CONFIGS["6.7b"][1:3] else
                   "decode tokens/sec + %% HBM roofline, OPT-%s shape bs%d, 1xMI355X" % (size, B)),
        "value": B / t_step,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": t_step * 1e3,
        "ms_per_step_std": t_std * 1e3,
        "ms_per_step_min": min(walls) * 1e3,
        "ms_per_step_windows": [w * 1e3 for w in walls],
        "repeats": R,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if not int8 else "int8-weights/f16",
        "data": "synthetic",
        "config": {
            "workload": "OPT-%s shape, batch %d, prompt EOS+%d random ids, greedy decode; timed "
                        "steps attend %d..%d positions" % (size, B, P, S_first, S_last),
            "layers": cfg.decoder_layers, "d_model": D, "heads": H, "vocab": cfg.vocab_size,
        },
        "hbm_frac_step": frac_mean,
        "hbm_frac_step_std": frac_std,
        "hbm_frac_step_mean_minus_std": frac_mean - frac_std,
        "hbm_frac_step_best_window": max(fracs),
        "step_bytes_mean": bytes_mean,
        "gpu_ms_per_step": gpu_s / K * 1e3,
        "graph_replay": st is not None,
        "prefill_s": prefill_s,
        "prefill_cold_s": prefill_cold_s,
        "prefill_tflops": prefill_flops(cfg, B, n0) / prefill_s / 1e12,
        "prefill_mfma_frac": prefill_flops(cfg, B, n0) / prefill_s / MFMA_PEAK,
        "setup_s": t1 - t0,
        "roofline": {
            "kernel": "attention_kernel<%d> (decode, T=1)" % hd,
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": achieved * 1e9 / HBM_PEAK,
            "traffic": traffic, "traffic_source": traffic_source,
            "bytes_per_launch": ab, "avg_launch_us": attn_s * 1e6, "context": S_probe,
            "plain_stream_read_GBps": stream_read,
        },
        "kernels": kernels,
    }
    if args.torch_eager and not int8:
        del inc, cache
        sd = model.state_dict()
        del model, gen, decoder
        torch.cuda.empty_cache()
        result["torch_eager_same_gpu"] = torch_eager_steps(cfg, sd, B, S_first, K, W, dev)
        del sd
        model = gen = inc = cache = decoder = None
    if not args.no_cpu_baseline:
        del model, gen, inc, cache, decoder
        torch.cuda.empty_cache()
        result["cpu_baseline"] = cpu_baseline()
        if args.cpu_same_shape:
            result["cpu_same_shape_extrapolated"] = cpu_baseline_same_shape(size, B, int(S_mean))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
