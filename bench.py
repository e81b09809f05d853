#!/usr/bin/env python3
"""Benchmark: train tokens/s of the GPT-124M-shape bf16 AdamW step on one MI355X.

One "step" is one full optimizer step (forward, backward, clip_grad_norm, AdamW,
loss readback) of the GPT-2-shaped model of BASELINE.json configs[2]
(12 layers, d_model 768, 12 heads of 64, MLP 3072, ctx 1024, vocab 50304,
batch 16 = 16384 tokens), bf16 operands with f32 master weights, on synthetic
tokens that are resident in HBM before the clock starts.

Prints one JSON line. `roofline` covers the dominant kernel, the bf16 MFMA GEMM:
algorithmic 2*M*N*K FLOPs of its launches divided by their summed duration,
measured with HIP events on the library's own stream during the timed steps.
`roofline_per_kernel` gives the same for the other kernel classes of the step
(flash attention forward and backward against the MFMA peak; cross-entropy,
AdamW, RMSNorm forward and backward and the embedding backward against HBM
bandwidth), each from the dispatch timestamps of its own launches in the same
timed steps. `cpu_baseline` times the CPU oracle (a C++ restatement of the
reference's CPU Exact arithmetic; the Rust reference cannot be built without
cargo) on the host cores, on a bounded sample of the same workload, with all
cores and with one thread, five repeats each (minimum, median and spread reported).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, vendor figure
F32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, vendor figure
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, vendor figure
# HBM bytes per GEMM op (MFMA kernel + split-K reduce), averaged over a step's GEMM ops (a strided
# batch of the stacked layers' weight gradients is one op): rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per
# dispatch, scaled by what the same counters read for the AdamW pass, whose traffic is known
# (profiles/gemm_hbm_traffic_all_workloads.txt holds the runs and the tables for each workload).
# The algorithmic figure of the gpt124m step (every operand read once, every output written once)
# is 2.326e10 bytes per step: 2.258e8 per product, 2.237e8 per launch (its 103 products run as 104
# launches: the head's weight gradient is cut by rows into two).
GEMM_HBM_BYTES_PER_LAUNCH = {"gpt124m": 3.42e8, "gpt124m-muon": 2.75e8, "lora1b": 4.13e8, "nanolab124m": 2.68e8}


# Kernel classes of omx_profile_kernels beyond the GEMM products: (bit, key, kernels, roofline).
KERNEL_CLASSES = [
    (1, "flash_attention_forward", "flash_fwd_kernel", "mfma"),
    (2, "flash_attention_backward", "flash_key_mean_kernel + flash_bwd_dq_kernel + flash_bwd_dkv_kernel", "mfma"),
    (3, "cross_entropy", "ce_row_fused_kernel", "hbm"),
    (4, "adamw", "adamw_apply_kernel (after adamw_check_kernel when it runs)", "hbm"),
    (5, "rms_norm_forward", "rms_fwd_vec_kernel", "hbm"),
    (6, "rms_norm_backward", "rms_bwd_vec_kernel + column_sum kernels", "hbm"),
    (7, "embedding_backward", "count / scan / fill / sort kernels + embedding_bwd_kernel", "hbm"),
]
ALL_CLASSES_MASK = 0xFF


def kernel_rooflines(lib, ctx, timed_steps: int):
    """Reads the per-class records of omx_profile_kernels: achieved = the launches' algorithmic FLOPs
    (matrix-unit classes, causal-counted for attention) or bytes (every operand read once, every
    result written once) over their summed dispatch durations."""
    out = {}
    for bit, key, kernels, bound in KERNEL_CLASSES:
        launches, ms, work = C.c_uint64(), C.c_double(), C.c_double()
        lib.omx_profile_kernels_report(ctx, C.c_int32(bit), C.byref(launches), C.byref(ms), C.byref(work))
        if launches.value == 0:
            continue
        peak = BF16_MFMA_PEAK_TFLOPS if bound == "mfma" else HBM_PEAK_GBS
        achieved = work.value / (ms.value * 1e-3) / (1e12 if bound == "mfma" else 1e9)
        out[key] = {"bound": bound, "kernel": kernels, "achieved": achieved, "peak": peak,
                    "unit": "TFLOP/s" if bound == "mfma" else "GB/s", "frac": achieved / peak, "traffic": None,
                    "launches": int(launches.value), "avg_launch_us": ms.value * 1e3 / launches.value,
                    "ms_per_step": ms.value / max(1, timed_steps)}
    return out


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def repeat_timed(fn, repeats: int = 5):
    """fn() -> seconds of the part it times itself; one untimed run first (page faults, thread
    start-up), then the sorted list of `repeats` runs."""
    fn()
    return sorted(fn() for _ in range(repeats))


def median_of(runs):
    return runs[len(runs) // 2]


def timed(fn, inner: int = 1):
    """(median seconds of `inner` calls of fn, its last result). The host is shared: a single timing of
    a one-second piece is off by 10-20 % now and then, the median of three rarely."""
    ts, result = [], None
    for _ in range(inner):
        t0 = time.perf_counter()
        result = fn()
        ts.append(time.perf_counter() - t0)
    return median_of(sorted(ts)), result


def spread_of(runs):
    """(max - min) / median of sorted timings."""
    return (runs[-1] - runs[0]) / median_of(runs)


def cpu_baseline(cfg, threads: int):
    """Times the oracle on a bounded sample of the same model and scales it to the step.

    Sequences share nothing but the weights and blocks cost the same, so the step's time is
    tokens x (rest + layers x block) / sample tokens + the optimizer pass. `block` comes from the
    model at one and at three blocks over a 256-entry vocabulary (the head is then a negligible part
    of both timings, so their difference is two blocks and little else), `rest` (embedding, final
    norm, the head over the real vocabulary) from the one-block model at the real vocabulary minus a
    block, and the optimizer (clip + AdamW) from one block's parameters scaled by the parameter
    count. A configuration small enough (the tiny one) is timed whole instead. All cores (the
    thread count is set explicitly) and one thread, one untimed run then five timed ones each; in the
    all-cores runs every model's time is itself the median of three calls. `value` is the median of
    the all-cores runs, `spread` their (max - min) / median."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_api as orc
    from ojas_amd.trainer import GptConfig, synthetic_batch

    tokens = cfg.batch * cfg.ctx
    whole = tokens * cfg.layers * cfg.d_model * cfg.d_model < 3e9  # the tiny configuration: 0.5e9
    rng = np.random.default_rng(0)

    def model(layers, batch, ctx, vocab=None):
        vocab = vocab or cfg.vocab
        sample = GptConfig(layers, cfg.d_model, cfg.heads, cfg.head_dim, cfg.mlp, ctx, vocab, batch, cfg.gelu_tanh, 0)
        ocfg = orc.GptConfig(layers, cfg.d_model, cfg.heads, cfg.head_dim, cfg.mlp, ctx, vocab, batch, cfg.gelu_tanh)
        params = [np.ones(n, np.float32) if n == cfg.d_model else rng.normal(0, 0.02, n).astype(np.float32)
                  for n in orc.gpt_param_lens(ocfg)]
        ids, targets = synthetic_batch(sample, 1)
        return ocfg, params, ids.reshape(-1), targets.reshape(-1)

    def optimizer_seconds(params, grads):
        moments = [(np.zeros_like(p), np.zeros_like(p)) for p in params]
        t0 = time.perf_counter()
        _, clipped = orc.clip_grad_norm(grads, 1.0)
        for p, g, (m, v) in zip(params, clipped, moments):
            orc.adamw_step(p, g, m, v, 0, 3e-4, 0.9, 0.95, 1e-8, 0.1, exact=True)
        return time.perf_counter() - t0

    def measure(n_threads, sample_ctx, inner):
        orc.set_threads(n_threads)
        if whole:
            ocfg, params, ids, targets = model(cfg.layers, cfg.batch, cfg.ctx)

            def once():
                dt, (_, grads) = timed(lambda: orc.gpt_loss_and_grads(ocfg, params, ids, targets), inner)
                return dt + optimizer_seconds(params, grads)

            runs = repeat_timed(once)
            return runs, f"the whole step ({cfg.batch}x{cfg.ctx} tokens)"
        one, small_one, small_three = model(1, 1, sample_ctx), model(1, 1, sample_ctx, 256), model(3, 1, sample_ctx, 256)
        n_params = sum(orc.gpt_param_lens(orc.GptConfig(cfg.layers, cfg.d_model, cfg.heads, cfg.head_dim, cfg.mlp,
                                                        cfg.ctx, cfg.vocab, cfg.batch, cfg.gelu_tanh)))
        block_params = [p for p in one[1][2:-1]]  # the block's eight tensors

        def once():
            t = [timed(lambda m=m: orc.gpt_loss_and_grads(*m), inner)[0] for m in (small_one, small_three, one)]
            block = max((t[1] - t[0]) / 2, 1e-9)
            rest = max(t[2] - block, 0.0)
            opt = optimizer_seconds(block_params, [np.full_like(p, 1e-3) for p in block_params])
            opt *= n_params / sum(p.size for p in block_params)
            return tokens * (rest + cfg.layers * block) / sample_ctx + opt

        runs = repeat_timed(once)
        return runs, (f"one and three blocks over a 256-entry vocabulary (a block) and one block over the real one "
                      f"(the rest) on 1x{sample_ctx} tokens, clip + AdamW on one block's parameters, scaled to "
                      f"{cfg.layers} blocks, {tokens} tokens and {n_params} parameters")

    all_runs, how = measure(threads, 512, 3)
    one_runs, how_one = measure(1, 64, 1)
    note = ("" if whole else " Attention grows with the sequence: at these sample lengths it is a smaller share than at "
            f"{cfg.ctx}, so the estimate favours the CPU by up to its 8 % of the step's work.")
    median, spread = median_of, spread_of
    return {"value": tokens / median(all_runs), "unit": "tokens/s", "cores": threads, "kind": "port",
            "cpu_model": cpu_model(), "repeats": len(all_runs), "step_seconds_min": all_runs[0],
            "step_seconds_median": median(all_runs), "spread": spread(all_runs),
            "single_thread": {"value": tokens / median(one_runs), "cores": 1, "step_seconds_min": one_runs[0],
                              "step_seconds_median": median(one_runs), "spread": spread(one_runs), "sample": how_one},
            "sample": f"same model (L{cfg.layers} d{cfg.d_model} vocab{cfg.vocab}) in f32 Exact arithmetic: {how}."
                      f"{note} C++ restatement of ojas-cpu, not the Rust binary"}


def kv_decode(args) -> int:
    """Secondary workload, the step after the training path: one `cached_attention_forward` call of
    a decode step (one new token per sequence) over a full KV cache, GPT-124M shape: batch 64,
    12 heads of 64, 1024 cached positions, f32 caches as the reference's trait prescribes. The op is
    bound by reading both caches once; `value` is those bytes over the call time."""
    sys.path.insert(0, str(ROOT / "tests"))
    from ojas_amd.backend import MiBackend

    b, h, d, t = 64, 12, 64, 1024
    be = MiBackend(0)
    r = np.random.default_rng(0)
    q = be.upload(r.standard_normal((b, 1, h, d)).astype(np.float32))
    kc = be.upload(r.standard_normal((b, t, h, d)).astype(np.float32))
    vc = be.upload(r.standard_normal((b, t, h, d)).astype(np.float32))
    for _ in range(args.warmup):
        be.cached_attention_forward(q, kc, vc, t)
    be.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = be.cached_attention_forward(q, kc, vc, t)
    be.sync()
    dt = (time.perf_counter() - t0) / args.steps
    nbytes = 2 * b * t * h * d * 4
    gbs = nbytes / dt / 1e9
    line = {
        "metric": "KV-cache attention, decode step (GPT-124M shape, batch 64, 1024 cached positions): cache GB/s",
        "value": gbs, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cached_attention_forward: q [64,1,12,64], caches [64,1024,12,64] f32, kv_len 1024",
                   "tokens_per_step": b},
        "roofline": {"bound": "hbm", "kernel": "cached_attention_group_kernel + cached_attention_merge_kernel",
                     "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                     "traffic": None, "algorithmic_bytes_per_launch": nbytes},
    }
    if not args.no_cpu_baseline:
        import oracle_api as orc

        sb = 4  # a bounded sample: 4 of the 64 sequences
        hq, hk, hv = (be.download(x)[:sb] for x in (q, kc, vc))
        c0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - c0 < 5.0:
            want = orc.cached_attention_forward(hq, hk, hv, t)
            reps += 1
        cdt = (time.perf_counter() - c0) / reps
        got = be.download(out)[:sb]
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
        line["cpu_baseline"] = {"value": 2 * sb * t * h * d * 4 / cdt / 1e9, "unit": "GB/s",
                                "cores": min(16, os.cpu_count() or 1), "kind": "port",
                                "sample": f"{sb} of the 64 sequences, {reps} calls in 5 s; C++ restatement of "
                                          "ojas-cpu/src/kv.rs (per-row Exact kernel), not the Rust binary"}
    be.close()
    print(json.dumps(line))
    return 0


def attention(args) -> int:
    """Secondary workload: the training step's attention alone, forward + backward of one block's
    causal attention at the headline shape (batch 16, 12 heads, 1024 tokens, head_dim 64, bf16;
    `--attention-batch 8` is the isolated attention case of the baseline's configs) through
    `causal_sdpa_forward` / `causal_sdpa_backward`. `value` is causal-counted TFLOP/s over both
    passes (forward 2 B H T^2 D, backward 5 B H T^2 D), from the median of five timed runs of each."""
    from ojas_amd.backend import BF16, MiBackend

    b, h, t, d = args.attention_batch, 12, 1024, 64
    be = MiBackend(0)
    r = np.random.default_rng(0)
    q, k, v, gy = (be.upload(r.standard_normal((b, h, t, d)).astype(np.float32), BF16) for _ in range(4))
    out, lse = be.causal_sdpa_forward(q, k, v, None, BF16)
    times, fastest = {}, {}
    for name, fn in (("forward", lambda: be.causal_sdpa_forward(q, k, v, None, BF16)),
                     ("backward", lambda: be.causal_sdpa_backward(q, k, v, out, lse, gy, None, BF16))):
        # Five timed runs of `steps` calls each, `warmup` untimed calls before every one: a run of 50
        # calls is a few milliseconds, shorter than the clock takes to settle after an idle stretch,
        # so single runs differ by 10 %. `us` is the median run, `us_min` the fastest.
        runs = []
        for _ in range(5):
            for _ in range(args.warmup):
                fn()
            be.sync()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                fn()
            be.sync()
            runs.append((time.perf_counter() - t0) / args.steps)
        runs.sort()
        times[name], fastest[name] = runs[2], runs[0]
    unit = 2.0 * b * h * t * t * d
    flops = {"forward": unit, "backward": 2.5 * unit}
    total = sum(times.values())
    line = {
        "metric": f"causal attention forward + backward (B{b} H12 T1024 D64 bf16): causal-counted TFLOP/s",
        "value": sum(flops.values()) / total / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": total * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"causal_sdpa_forward + causal_sdpa_backward: q, k, v [{b},12,1024,64] bf16",
                   "tokens_per_step": b * t},
        "roofline": {"bound": "mfma", "kernel": "flash_fwd_kernel; flash_key_mean_kernel + flash_bwd_dq_kernel + "
                                                "flash_bwd_dkv_kernel",
                     "achieved": sum(flops.values()) / total / 1e12, "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": sum(flops.values()) / total / 1e12 / BF16_MFMA_PEAK_TFLOPS, "traffic": None},
        "us": {name: dt * 1e6 for name, dt in times.items()},
        "us_min": {name: dt * 1e6 for name, dt in fastest.items()},
        "tflops": {name: flops[name] / dt / 1e12 for name, dt in times.items()},
    }
    be.close()
    print(json.dumps(line))
    return 0


def lora_cpu_baseline(cfg, threads: int):
    """Times the oracle's LoRA step on a bounded sample of the same model at full width: one short
    sequence, once with one block and once with two; the difference is a block's time, the rest the
    table, final norm and head; the step is tokens x (rest + layers x block) / sample tokens plus
    clip + AdamW on the adapters (timed on one block's, scaled by their count). The block's time comes
    from a small-vocabulary pair of models, as in `cpu_baseline`. All cores and one thread, one
    untimed run then five timed ones each; `value` is the median of the all-cores runs."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_api as orc

    tokens = cfg.batch * cfg.seq
    rng = np.random.default_rng(0)

    def model(layers, seq, vocab):
        ocfg = orc.LoraConfig(layers, cfg.d_model, cfg.heads, cfg.head_dim, cfg.hidden, vocab, 1, seq, cfg.rank,
                              cfg.rms_eps, cfg.lora_scale, cfg.rope_base)
        frozen = []
        for shape in orc.lora_frozen_shapes(ocfg):
            if len(shape) == 1:
                frozen.append(np.ones(shape, np.float32))
            elif shape[0] == vocab:
                frozen.append(rng.normal(0, 0.02, shape).astype(np.float32))
            else:  # codes and scales drawn directly: the values a quantised N(0, 0.02) matrix dequantises to
                codes = rng.integers(-127, 128, shape).astype(np.int8)
                scales = np.full((shape[0], shape[1] // 32), 0.05 / 127, np.float32)
                frozen.append(orc.dequant_i8_group(codes, scales, 32))
        adapters = [rng.normal(0, 0.02, sh).astype(np.float32) for sh in orc.lora_adapter_shapes(ocfg)]
        ids = rng.integers(0, vocab, seq).astype(np.uint32)
        targets = rng.integers(0, vocab, seq).astype(np.uint32)
        return ocfg, frozen, adapters, ids, targets

    def measure(n_threads, seq, inner):
        orc.set_threads(n_threads)
        # A block's time from one and three blocks over a 256-entry vocabulary (the head is then a
        # negligible part of both timings); the rest from one block over the real vocabulary. Every
        # model's time is the median of `inner` calls.
        small_one, small_three, one = model(1, seq, 256), model(3, seq, 256), model(1, seq, cfg.vocab)

        def once():
            t = []
            for m in (small_one, small_three, one):
                dt, (_, grads) = timed(lambda m=m: orc.lora_loss_and_grads(*m), inner)
                t.append(dt)
            flat = [a.reshape(-1).copy() for a in one[2]]
            moments = [(np.zeros_like(p), np.zeros_like(p)) for p in flat]
            t0 = time.perf_counter()
            _, clipped = orc.clip_grad_norm(grads, 1.0)
            for p, g, (m, v) in zip(flat, clipped, moments):
                orc.adamw_step(p, g, m, v, 0, 1e-4, 0.9, 0.95, 1e-8, 0.0, exact=True)
            opt = (time.perf_counter() - t0) * cfg.layers
            block = max((t[1] - t[0]) / 2, 1e-9)
            rest = max(t[2] - block, 0.0)
            return tokens * (rest + cfg.layers * block) / seq + opt

        return repeat_timed(once, 5 if n_threads > 1 else 3)

    all_runs = measure(threads, 128, 3)
    one_runs = measure(1, 32, 1)
    return {"value": tokens / median_of(all_runs), "unit": "tokens/s", "cores": threads, "kind": "port",
            "cpu_model": cpu_model(), "repeats": len(all_runs), "step_seconds_min": all_runs[0],
            "step_seconds_median": median_of(all_runs), "spread": spread_of(all_runs),
            "single_thread": {"value": tokens / median_of(one_runs), "cores": 1, "step_seconds_min": one_runs[0],
                              "step_seconds_median": median_of(one_runs), "spread": spread_of(one_runs), "sample": "as below on 1x32 tokens"},
            "sample": f"same model at full width in f32 Exact arithmetic on dequantised weights: one and three blocks over a "
                      f"256-entry vocabulary (a block) and one block over the real one (the rest) on 1x128 tokens, one "
                      f"untimed run then five timed ones, clip + AdamW on one block's adapters, scaled to {cfg.layers} "
                      f"blocks and {tokens} tokens. Attention grows with the sequence: at this sample length it is a "
                      f"smaller share than at {cfg.seq}, so the estimate favours the CPU by up to its 9 % of the step's "
                      f"work. C++ restatement of ojas-cpu, not the Rust binary"}


def lora_step(args) -> int:
    """BASELINE configs[4]: one LoRA rank-16 fine-tune step on a frozen ~1B int8 decoder."""
    from ojas_amd.backend import AdamWConfig, MiBackend
    from ojas_amd.lora import LoraTrainer, adapter_params, base_params, config_lora1b, step_flops

    cfg = config_lora1b()
    be = MiBackend(0)
    tr = LoraTrainer(be, cfg)
    tr.init_base(1234, 0.02)
    tr.init_adapters(99, 0.02)
    rng = np.random.default_rng(42)
    window = rng.integers(0, cfg.vocab, (cfg.batch, cfg.seq + 1)).astype(np.uint32)
    tr.set_batch(window[:, :-1], window[:, 1:])
    adamw = AdamWConfig(1e-4, 0.9, 0.95, 1e-8, 0.0)
    losses = [tr.step(adamw, 1.0)[0] for _ in range(args.warmup)]
    be.sync()
    lib = be._lib
    timed_every = max(1, args.timed_every)
    step_ms = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        lib.omx_profile_kernels(be._ctx, C.c_uint32(ALL_CLASSES_MASK if i % timed_every == 0 else 0))
        s0 = time.perf_counter()
        losses.append(tr.step(adamw, 1.0)[0])  # ends with the loss readback: the step is complete
        step_ms.append((time.perf_counter() - s0) * 1e3)
    be.sync()
    dt = time.perf_counter() - t0
    launches, gemm_ms, gemm_flops = C.c_uint64(), C.c_double(), C.c_double()
    lib.omx_profile_gemm_report(be._ctx, C.byref(launches), C.byref(gemm_ms), C.byref(gemm_flops))
    per_kernel = kernel_rooflines(lib, be._ctx, len(range(0, args.steps, timed_every)))
    lib.omx_profile_kernels(be._ctx, C.c_uint32(0))
    tokens = cfg.batch * cfg.seq
    ms_per_step = dt / args.steps * 1e3
    flops = step_flops(cfg)
    achieved = gemm_flops.value / (gemm_ms.value * 1e-3) / 1e12 if gemm_ms.value > 0 else 0.0
    timed_steps = len(range(0, args.steps, timed_every))
    out = {
        "metric": "train tokens/s on 1 MI355X (LoRA r16 step on a frozen int8-g32 ~1B decoder, BASELINE configs[4])",
        "value": tokens * args.steps / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_min": float(np.min(step_ms)),
        "ms_per_step_median": float(np.median(step_ms)), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "LoRA rank-16 fine-tune step (BASELINE configs[4]): L16 d2048 H16x128 SwiGLU8192 ctx2048 "
                               "batch4 vocab32000, RoPE 1e4, base int8 symmetric in groups of 32 along K with f32 "
                               "scales through the dequant-fused product, adapters on q/k/v/o (A ~ N(0,0.02), B = 0), "
                               "AdamW lr1e-4 on the adapters only, clip 1.0",
                   "tokens_per_step": tokens, "base_params": base_params(cfg), "adapter_params": adapter_params(cfg)},
        "step_tflops": flops / (ms_per_step * 1e-3) / 1e12,
        "pct_bf16_mfma_peak": 100.0 * flops / (ms_per_step * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        "loss_first": losses[0], "loss_last": losses[-1],
        "roofline": {"bound": "mfma",
                     "kernel": "gemm_q8_kernel (int8-g32 dequant-fused bf16 MFMA product) with the adapters' and the "
                               "head's bf16 products",
                     "achieved": achieved, "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / BF16_MFMA_PEAK_TFLOPS, "traffic": GEMM_HBM_BYTES_PER_LAUNCH["lora1b"],
                     "launches": int(launches.value),
                     "avg_launch_us": gemm_ms.value * 1e3 / max(1, launches.value), "timed_steps": timed_steps,
                     "gemm_ms_per_step": gemm_ms.value / max(1, timed_steps)},
        "roofline_per_kernel": per_kernel,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = lora_cpu_baseline(cfg, min(16, os.cpu_count() or 1))
    tr.close()
    be.close()
    print(json.dumps(out))
    return 0


def nanolab_cpu_baseline(spec, batch, seq, threads: int):
    """The oracle's nanolab step on a bounded sample: one and three blocks over a small vocabulary
    give a block's time, one block over the real vocabulary the rest (table, final norm, head), all on
    one short sequence; clip + Muon-NS5 (f32 iteration) on one block's matrices and AdamW on its
    vectors and on the table give the optimizer's. Scaled to the model's blocks and the step's
    tokens. All cores and one thread, one untimed run then five timed ones each."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_api as orc
    from ojas_amd.nanolab import NanolabSpec

    tokens = batch * seq
    rng = np.random.default_rng(0)

    def model(layers, sample_seq, vocab):
        sp = NanolabSpec(**{**spec.__dict__, "n_layer": layers, "vocab": vocab})
        cfg = orc.NanolabConfig(layers=layers, n_embd=sp.n_embd, n_head=sp.n_head, n_kv_head=sp.n_kv_head,
                                head_dim=sp.head_dim, hidden=sp.hidden, vocab=sp.vocab, batch=1, seq=sample_seq, window=0,
                                rms_eps=sp.rms_eps, rope_base=sp.rope_base)
        shapes = sp.param_shapes()
        params = [np.ones(shapes[n], np.float32).reshape(-1) if len(shapes[n]) == 1
                  else rng.normal(0, 0.02, shapes[n]).astype(np.float32).reshape(-1) for n in sp.param_names()]
        ids = rng.integers(0, sp.vocab, (1, sample_seq)).astype(np.uint32)
        return sp, cfg, params, ids

    def measure(n_threads, sample_seq, inner):
        orc.set_threads(n_threads)
        # A block's time from one and three blocks over a 256-entry vocabulary (the head is then a
        # negligible part of both timings); the rest from one block over the real vocabulary. Every
        # model's time is the median of `inner` calls (the optimizer, a twentieth of the step, is timed once).
        small_one, small_three, one = model(1, sample_seq, 256), model(3, sample_seq, 256), model(1, sample_seq, spec.vocab)
        shapes = one[0].param_shapes()
        names = one[0].param_names()

        def once():
            t = [timed(lambda m=m: orc.nanolab_loss_and_grads(m[1], m[2], m[3], m[3]), inner)[0]
                 for m in (small_one, small_three, one)]
            block = max((t[1] - t[0]) / 2, 1e-9)
            rest = max(t[2] - block, 0.0)
            # optimizer on the one-block model: the table and final norm once, the block's tensors per block
            t_table, t_block = 0.0, 0.0
            for n, p in zip(names, one[2]):
                g = np.full_like(p, 1e-3)
                if len(shapes[n]) == 2 and n != "tok_emb.weight":
                    w, g2, mom = p.reshape(shapes[n]).copy(), g.reshape(shapes[n]), np.zeros(shapes[n], np.float32)
                    dt = timed(lambda: orc.muon_ns5_step(w, g2, mom, lr=0.025, momentum=0.99, weight_decay=0.1,
                                                         nesterov=True, bf16=False))[0]
                else:
                    w, m1, m2 = p.copy(), np.zeros_like(p), np.zeros_like(p)
                    dt = timed(lambda: orc.adamw_step(w, g, m1, m2, 0, 6e-4, 0.9, 0.95, 1e-8, 0.0, exact=True))[0]
                if n.startswith("blocks."):
                    t_block += dt
                else:
                    t_table += dt
            return tokens * (rest + spec.n_layer * block) / sample_seq + t_table + spec.n_layer * t_block

        return repeat_timed(once, 5 if n_threads > 1 else 3)

    all_runs = measure(threads, 128, 3)
    one_runs = measure(1, 32, 1)
    return {"value": tokens / median_of(all_runs), "unit": "tokens/s", "cores": threads, "kind": "port",
            "cpu_model": cpu_model(), "repeats": len(all_runs), "step_seconds_min": all_runs[0],
            "step_seconds_median": median_of(all_runs), "spread": spread_of(all_runs),
            "single_thread": {"value": tokens / median_of(one_runs), "cores": 1, "step_seconds_min": one_runs[0],
                              "step_seconds_median": median_of(one_runs), "spread": spread_of(one_runs), "sample": "as below on 1x32 tokens"},
            "sample": f"same model in f32 Exact arithmetic: one and three blocks over a 256-entry vocabulary (a block) and one "
                      f"block over the real one (the rest) on 1x128 tokens, one untimed run then five timed ones, Muon-NS5 "
                      f"and AdamW on one block's parameters and the table, scaled to {spec.n_layer} blocks and {tokens} "
                      f"tokens. Attention grows with the sequence: at this sample length it is a smaller share than at "
                      f"{seq}, so the estimate favours the CPU by up to its 8 % of the step's work. C++ restatement of "
                      f"ojas-cpu, not the Rust binary"}


def nanolab_step(args) -> int:
    """The reference's own model at its 124M size (ModelSpec::nanolab_124m, ojas-model/src/spec.rs:74-91):
    one Trainer::run step (Muon-NS5 on the matrices, AdamW on the table and the vectors) of one
    16 x 1024 micro-batch through the C++ step driver, bf16 storage."""
    from ojas_amd.backend import MiBackend
    from ojas_amd.nanolab import NativeNanolabTrainer, nanolab_step_flops, spec_nanolab_124m

    spec = spec_nanolab_124m()
    batch, seq = 16, 1024
    be = MiBackend(0)
    tr = NativeNanolabTrainer(be, spec, batch, seq, bf16=True, ns5_bf16=True)
    tr.init(1234)
    rng = np.random.default_rng(42)
    window = rng.integers(0, spec.vocab, (batch, seq + 1)).astype(np.uint32)
    tr._micro(window[:, :-1], window[:, 1:], 1.0, 1.0, True)  # uploads the batch; it stays resident
    losses = [tr.run_resident(1.0).loss for _ in range(args.warmup)]
    be.sync()
    lib = be._lib
    timed_every = max(1, args.timed_every)
    step_ms = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        lib.omx_profile_kernels(be._ctx, C.c_uint32(ALL_CLASSES_MASK if i % timed_every == 0 else 0))
        s0 = time.perf_counter()
        losses.append(tr.run_resident(1.0).loss)  # ends with the loss readback: the step is complete
        step_ms.append((time.perf_counter() - s0) * 1e3)
    be.sync()
    dt = time.perf_counter() - t0
    timed_steps = len(range(0, args.steps, timed_every))
    launches, gemm_ms, gemm_flops = C.c_uint64(), C.c_double(), C.c_double()
    lib.omx_profile_gemm_report(be._ctx, C.byref(launches), C.byref(gemm_ms), C.byref(gemm_flops))
    per_kernel = kernel_rooflines(lib, be._ctx, timed_steps)
    lib.omx_profile_kernels(be._ctx, C.c_uint32(0))
    tokens = batch * seq
    ms_per_step = dt / args.steps * 1e3
    flops = nanolab_step_flops(spec, batch, seq)
    achieved = gemm_flops.value / (gemm_ms.value * 1e-3) / 1e12 if gemm_ms.value > 0 else 0.0
    out = {
        "metric": "train tokens/s on 1 MI355X (nanolab-124M bf16 step: Muon-NS5 + AdamW, the reference's own model)",
        "value": tokens * args.steps / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_min": float(np.min(step_ms)),
        "ms_per_step_median": float(np.median(step_ms)), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "nanolab-124M training step (ModelSpec::nanolab_124m): L12 d768 H12x64 (12 KV heads) SwiGLU "
                               "2048 vocab 50304 ctx 1024 batch 16, QK-norm, RoPE 1e4, per-head sigmoid gate, value "
                               "residual, tied head; bf16 activations and operand copies, f32 master weights; Muon-NS5 "
                               "(bf16 iteration, lr 0.025, momentum 0.99, wd 0.1) on the matrices, AdamW lr 6e-4 on the "
                               "table and the vectors, clip 1.0; one micro-batch per step",
                   "tokens_per_step": tokens, "params": int(sum(tr.lens))},
        "step_tflops": flops / (ms_per_step * 1e-3) / 1e12,
        "pct_bf16_mfma_peak": 100.0 * flops / (ms_per_step * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        "loss_first": losses[0], "loss_last": losses[-1],
        "roofline": {"bound": "mfma", "kernel": "gemm_w4_kernel / gemm_dma_kernel / gemm_kernel (bf16 MFMA GEMM, all operand layouts)",
                     "achieved": achieved, "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / BF16_MFMA_PEAK_TFLOPS, "traffic": GEMM_HBM_BYTES_PER_LAUNCH["nanolab124m"],
                     "launches": int(launches.value),
                     "avg_launch_us": gemm_ms.value * 1e3 / max(1, launches.value), "timed_steps": timed_steps,
                     "gemm_ms_per_step": gemm_ms.value / max(1, timed_steps)},
        "roofline_per_kernel": per_kernel,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = nanolab_cpu_baseline(spec, batch, seq, min(16, os.cpu_count() or 1))
    tr.close()
    be.close()
    print(json.dumps(out))
    return 0


def gemm(args) -> int:
    """Secondary workload: one bf16 product through `omx_gemm`, `--gemm-shape M,K,N` in layout
    `--gemm-layout` (NN: A [M,K] and B^T [N,K] both k-contiguous, a forward product; NT: B [K,N], an
    input gradient; TT: A^T [K,M] too, a weight gradient), bf16 output (f32 for TT), the tiling
    chosen by the library unless `--gemm-tiling` forces one. `value` is 2 M N K over the median of
    five timed runs of `--steps` launches."""
    import ctypes as C

    from ojas_amd.backend import BF16, F32, MiBackend

    m, k, n = (int(v) for v in args.gemm_shape.split(","))
    layout = args.gemm_layout
    be = MiBackend(0)
    lib = be._lib
    a = be.empty((m * k,), BF16)
    b = be.empty((k * n,), BF16)
    for t, seed in ((a, 1), (b, 2)):
        be._check(lib.omx_init_normal(be._ctx, be._p(t), C.c_int32(BF16), C.c_uint64(t.numel), C.c_uint64(seed),
                                      C.c_float(0.05)))
    out_dtype = F32 if layout == "TT" else BF16
    c = be.empty((m, n), out_dtype)
    a_strides = (1, m) if layout == "TT" else (k, 1)
    b_strides = (1, k) if layout == "NN" else (n, 1)
    be.set_option("gemm_dma", args.gemm_tiling)

    def launch():
        be._check(lib.omx_gemm(be._ctx, be._p(a), C.c_uint64(a_strides[0]), C.c_uint64(a_strides[1]), be._p(b),
                               C.c_uint64(b_strides[0]), C.c_uint64(b_strides[1]), C.c_int32(BF16), be._p(c),
                               C.c_int32(out_dtype), C.c_uint64(m), C.c_uint64(k), C.c_uint64(n), C.c_int32(0)))

    runs = []
    for _ in range(5):
        for _ in range(args.warmup):
            launch()
        be.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            launch()
        be.sync()
        runs.append((time.perf_counter() - t0) / args.steps)
    runs.sort()
    flops = 2.0 * m * n * k
    nbytes = 2.0 * (m * k + k * n) + (4.0 if out_dtype == F32 else 2.0) * m * n
    line = {
        "metric": f"bf16 GEMM {layout} {m}x{k}x{n}: TFLOP/s", "value": flops / runs[2] / 1e12, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": runs[2] * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"omx_gemm {layout}: A [{m},{k}], B [{k},{n}] bf16, tiling option {args.gemm_tiling}"},
        "roofline": {"bound": "mfma", "kernel": "gemm_w4_kernel / gemm_dma_kernel / gemm_kernel",
                     "achieved": flops / runs[2] / 1e12, "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / runs[2] / 1e12 / BF16_MFMA_PEAK_TFLOPS, "traffic": None,
                     "algorithmic_bytes_per_launch": nbytes},
        "us": runs[2] * 1e6, "us_min": runs[0] * 1e6,
    }
    be.close()
    print(json.dumps(line))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--timed-every", type=int, default=10,
                    help="the kernels of every N-th timed step carry events for the roofline figures")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--config", default="gpt124m", choices=["gpt124m", "tiny", "lora1b", "nanolab124m"])
    ap.add_argument("--optimizer", default="adamw", choices=["adamw", "muon"],
                    help="adamw: BASELINE configs[2], the headline (default); muon: configs[3], Muon-NS5 (bf16 "
                         "iteration, lr 0.02, momentum 0.95) on the hidden matrices and AdamW on tables and norms")
    ap.add_argument("--attention-batch", type=int, default=16, help="batch of --workload attention")
    ap.add_argument("--gemm-shape", default="8192,8192,8192", help="M,K,N of --workload gemm")
    ap.add_argument("--gemm-layout", default="NN", choices=["NN", "NT", "TT"], help="operand layout of --workload gemm")
    ap.add_argument("--gemm-tiling", type=int, default=1, choices=[0, 1, 3, 4, 9, 10],
                    help="the library's gemm_dma option for --workload gemm (1: chosen by shape)")
    ap.add_argument("--workload", default="train_step", choices=["train_step", "kv_decode", "attention", "gemm"],
                    help="train_step: the headline metric (default); kv_decode: the decode attention op alone; "
                         "attention: the step's causal attention alone, forward + backward; gemm: one bf16 product")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        return 2
    if args.workload == "kv_decode":
        return kv_decode(args)
    if args.workload == "attention":
        return attention(args)
    if args.workload == "gemm":
        return gemm(args)
    if args.config == "lora1b":
        return lora_step(args)
    if args.config == "nanolab124m":
        return nanolab_step(args)

    from ojas_amd.backend import AdamWConfig, MiBackend, MuonNs5Config
    from ojas_amd.trainer import GptTrainer, config_gpt124m_bf16, config_tiny_f32, step_flops, synthetic_batch

    cfg = config_gpt124m_bf16() if args.config == "gpt124m" else config_tiny_f32()
    be = MiBackend(0)
    tr = GptTrainer(be, cfg)
    tr.init(1234)
    ids, targets = synthetic_batch(cfg, 42)
    tr.set_batch(ids, targets)
    adamw = AdamWConfig.nanolab(3e-4, 0.1)
    if args.optimizer == "muon":
        muon = MuonNs5Config(0.02, 0.95, 0.1, 1, 1 if cfg.bf16 else 0)
        adamw = AdamWConfig.nanolab(3e-4, 0.0)
        one_step = lambda: tr.step_hybrid(muon, adamw, 1.0)[0]
    else:
        one_step = lambda: tr.step(adamw, 1.0)[0]
    losses = []
    for _ in range(args.warmup):
        losses.append(one_step())
    be.sync()
    lib = be._lib
    # The kernels of every tenth timed step (--timed-every) carry HIP events on their dispatches
    # (begin and end timestamps of the kernels themselves): the GEMM products and the classes of
    # KERNEL_CLASSES. All steps would cost about a millisecond per step on the number being measured
    # (the timed launch path is slower: 104 GEMM launches and some 80 others per step); two steps of
    # the default run's twenty are 208 timed GEMM launches.
    timed_every = max(1, args.timed_every)
    step_ms = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        lib.omx_profile_kernels(be._ctx, C.c_uint32(ALL_CLASSES_MASK if i % timed_every == 0 else 0))
        s0 = time.perf_counter()
        losses.append(one_step())  # ends with the loss readback: the step is complete
        step_ms.append((time.perf_counter() - s0) * 1e3)
    be.sync()
    dt = time.perf_counter() - t0
    launches, gemm_ms, gemm_flops = C.c_uint64(), C.c_double(), C.c_double()
    lib.omx_profile_gemm_report(be._ctx, C.byref(launches), C.byref(gemm_ms), C.byref(gemm_flops))
    per_kernel = kernel_rooflines(lib, be._ctx, len(range(0, args.steps, timed_every)))
    lib.omx_profile_kernels(be._ctx, C.c_uint32(0))

    tokens = cfg.batch * cfg.ctx
    ms_per_step = dt / args.steps * 1e3
    value = tokens * args.steps / dt
    flops = step_flops(cfg)
    achieved = gemm_flops.value / (gemm_ms.value * 1e-3) / 1e12 if gemm_ms.value > 0 else 0.0
    gemm_peak = BF16_MFMA_PEAK_TFLOPS if cfg.bf16 else F32_MFMA_PEAK_TFLOPS
    out = {
        "metric": "train tokens/s on 1 MI355X (nanolab-GPT tiny f32 AdamW step, BASELINE configs[0])"
                  if args.config == "tiny"
                  else "train tokens/s on 1 MI355X (GPT-124M bf16 AdamW step); % bf16 MFMA peak" if args.optimizer == "adamw"
                  else "train tokens/s on 1 MI355X (GPT-124M bf16 Muon-NS5 + AdamW step, BASELINE configs[3])",
        "value": value,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_min": float(np.min(step_ms)),
        "ms_per_step_median": float(np.median(step_ms)),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg.bf16 else "f32",
        "data": "synthetic",
        "config": {"workload": ("GPT-124M-shape training step (BASELINE configs[2]): L12 d768 H12x64 mlp3072 ctx1024 "
                                "vocab50304 batch16, bf16 operands, f32 master weights, AdamW lr3e-4 wd0.1, clip 1.0"
                                if args.optimizer == "adamw" else
                                "GPT-124M-shape training step (BASELINE configs[3]): L12 d768 H12x64 mlp3072 ctx1024 "
                                "vocab50304 batch16, bf16 operands, f32 master weights, Muon-NS5 (bf16 iteration, lr 0.02, "
                                "momentum 0.95, wd 0.1, Nesterov) on the 72 hidden matrices, AdamW lr3e-4 on tables and "
                                "norms, clip 1.0")
                   if args.config == "gpt124m" else "nanolab-GPT tiny f32 step (BASELINE configs[0])",
                   "tokens_per_step": tokens, "params": sum(tr.param_lens())},
        "step_tflops": flops / (ms_per_step * 1e-3) / 1e12,
        "pct_bf16_mfma_peak": 100.0 * flops / (ms_per_step * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS if cfg.bf16 else None,
        "loss_first": losses[0], "loss_last": losses[-1],
        "roofline": {"bound": "mfma",
                     "kernel": "gemm_w4_kernel / gemm_dma_kernel / gemm_kernel (bf16 MFMA GEMM, all operand layouts)" if cfg.bf16
                               else "gemm_kernel<float> (f32 MFMA GEMM, all operand layouts)",
                     "achieved": achieved, "peak": gemm_peak, "unit": "TFLOP/s", "frac": achieved / gemm_peak,
                     "traffic": GEMM_HBM_BYTES_PER_LAUNCH.get(
                         "gpt124m" if args.optimizer == "adamw" else "gpt124m-muon") if args.config == "gpt124m" else None,
                     "launches": int(launches.value), "avg_launch_us": gemm_ms.value * 1e3 / max(1, launches.value),
                     "timed_steps": len(range(0, args.steps, timed_every)),
                     "gemm_ms_per_step": gemm_ms.value / max(1, len(range(0, args.steps, timed_every)))},
        "roofline_per_kernel": per_kernel,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, min(16, os.cpu_count() or 1))
    tr.close()
    be.close()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
