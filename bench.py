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
`cpu_baseline` times the CPU oracle (a C++ restatement of the reference's CPU
Exact arithmetic; the Rust reference cannot be built without cargo) on the
host cores, on a bounded sample of the same workload.
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
# HBM bytes per GEMM op (MFMA kernel + split-K reduce) on the gpt124m workload, averaged over the
# step's 103 GEMM ops (a strided batch of the stacked layers' weight gradients is one op): rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by what the same
# counters read for the AdamW pass, whose traffic is known (profiles/gemm_hbm_traffic_gpt124m_bf16.txt).
# The algorithmic figure (every operand read once, every output written once) is 2.258e8.
GEMM_HBM_BYTES_PER_LAUNCH_GPT124M = 3.82e8


def cpu_baseline(cfg, threads: int):
    """Times the oracle on a bounded sample: the same model on one 1 x 1024 token
    sequence (forward + backward + clip + AdamW), reported per token."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_api as orc
    from ojas_amd.trainer import GptConfig, synthetic_batch

    sample = GptConfig(cfg.layers, cfg.d_model, cfg.heads, cfg.head_dim, cfg.mlp, min(cfg.ctx, 1024), cfg.vocab, 1, cfg.gelu_tanh, 0)
    ocfg = orc.GptConfig(sample.layers, sample.d_model, sample.heads, sample.head_dim, sample.mlp, sample.ctx,
                         sample.vocab, sample.batch, sample.gelu_tanh)
    orc.set_threads(threads)
    rng = np.random.default_rng(0)
    params = [np.ones(n, np.float32) if n == sample.d_model else rng.normal(0, 0.02, n).astype(np.float32)
              for n in orc.gpt_param_lens(ocfg)]
    ids, targets = synthetic_batch(sample, 1)
    t0 = time.perf_counter()
    _, grads = orc.gpt_loss_and_grads(ocfg, params, ids.reshape(-1), targets.reshape(-1))
    _, grads = orc.clip_grad_norm(grads, 1.0)
    for p, g in zip(params, grads):
        orc.adamw_step(p, g, np.zeros_like(p), np.zeros_like(p), 0, 3e-4, 0.9, 0.95, 1e-8, 0.1, exact=True)
    dt = time.perf_counter() - t0
    tokens = sample.batch * sample.ctx
    return {"value": tokens / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"same model (L{sample.layers} d{sample.d_model} vocab{sample.vocab}), one step on "
                      f"1x{sample.ctx} tokens in f32 Exact arithmetic "
                      f"({dt:.1f} s), scaled per token; C++ restatement of ojas-cpu, not the Rust binary"}


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


def lora_cpu_baseline(cfg, threads: int):
    """Times the oracle's LoRA step on a bounded sample of the same model: full width, 256 tokens of
    one sequence, once with one block and once with two; the difference is a block's time, the rest
    the table, final norm and head, and the model's 16 blocks are extrapolated from the two."""
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_api as orc

    orc.set_threads(threads)
    seq = 256
    rng = np.random.default_rng(0)
    times = []
    for layers in (1, 2):
        ocfg = orc.LoraConfig(layers, cfg.d_model, cfg.heads, cfg.head_dim, cfg.hidden, cfg.vocab, 1, seq, cfg.rank,
                              cfg.rms_eps, cfg.lora_scale, cfg.rope_base)
        frozen = []
        for shape in orc.lora_frozen_shapes(ocfg):
            if len(shape) == 1:
                frozen.append(np.ones(shape, np.float32))
            elif shape[0] == cfg.vocab:
                frozen.append(rng.normal(0, 0.02, shape).astype(np.float32))
            else:
                codes, scales = orc.quantize_i8_group(rng.normal(0, 0.02, shape).astype(np.float32), 32)
                frozen.append(orc.dequant_i8_group(codes, scales, 32))
        adapters = [rng.normal(0, 0.02, sh).astype(np.float32) for sh in orc.lora_adapter_shapes(ocfg)]
        ids = rng.integers(0, cfg.vocab, seq).astype(np.uint32)
        targets = rng.integers(0, cfg.vocab, seq).astype(np.uint32)
        t0 = time.perf_counter()
        _, grads = orc.lora_loss_and_grads(ocfg, frozen, adapters, ids, targets)
        _, grads = orc.clip_grad_norm(grads, 1.0)
        for p, g in zip(adapters, grads):
            p = p.reshape(-1)
            orc.adamw_step(p, g, np.zeros_like(p), np.zeros_like(p), 0, 1e-4, 0.9, 0.95, 1e-8, 0.0, exact=True)
        times.append(time.perf_counter() - t0)
    per_block = max(times[1] - times[0], 1e-9)
    rest = max(times[0] - per_block, 0.0)
    full = rest + cfg.layers * per_block
    return {"value": seq / full, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"same model at full width, 1x{seq} tokens, f32 Exact arithmetic on dequantised weights: "
                      f"1 block {times[0]:.1f} s, 2 blocks {times[1]:.1f} s, extrapolated to {cfg.layers} blocks "
                      f"({full:.1f} s); C++ restatement of ojas-cpu, not the Rust binary"}


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
    timed_every = 4
    step_ms = []
    t0 = time.perf_counter()
    for i in range(args.steps):
        lib.omx_profile_gemm(be._ctx, C.c_int32(1 if i % timed_every == 0 else 0))
        s0 = time.perf_counter()
        losses.append(tr.step(adamw, 1.0)[0])  # ends with the loss readback: the step is complete
        step_ms.append((time.perf_counter() - s0) * 1e3)
    be.sync()
    dt = time.perf_counter() - t0
    launches, gemm_ms, gemm_flops = C.c_uint64(), C.c_double(), C.c_double()
    lib.omx_profile_gemm_report(be._ctx, C.byref(launches), C.byref(gemm_ms), C.byref(gemm_flops))
    lib.omx_profile_gemm(be._ctx, C.c_int32(0))
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
                     "frac": achieved / BF16_MFMA_PEAK_TFLOPS, "traffic": None, "launches": int(launches.value),
                     "avg_launch_us": gemm_ms.value * 1e3 / max(1, launches.value), "timed_steps": timed_steps,
                     "gemm_ms_per_step": gemm_ms.value / max(1, timed_steps)},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = lora_cpu_baseline(cfg, min(16, os.cpu_count() or 1))
    tr.close()
    be.close()
    print(json.dumps(out))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--config", default="gpt124m", choices=["gpt124m", "tiny", "lora1b"])
    ap.add_argument("--optimizer", default="adamw", choices=["adamw", "muon"],
                    help="adamw: BASELINE configs[2], the headline (default); muon: configs[3], Muon-NS5 (bf16 "
                         "iteration, lr 0.02, momentum 0.95) on the hidden matrices and AdamW on tables and norms")
    ap.add_argument("--workload", default="train_step", choices=["train_step", "kv_decode"],
                    help="train_step: the headline metric (default); kv_decode: the decode attention op alone")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        return 2
    if args.workload == "kv_decode":
        return kv_decode(args)
    if args.config == "lora1b":
        return lora_step(args)

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
    # The GEMM kernels of every fourth timed step carry HIP events on their dispatches (begin and
    # end timestamps of the kernels themselves). All steps would cost 0.7 ms per step on the
    # number being measured (the timed launch path is slower: 103 products per step); a quarter
    # of them is 515 timed products in the default run.
    timed_every = 4
    t0 = time.perf_counter()
    for i in range(args.steps):
        lib.omx_profile_gemm(be._ctx, C.c_int32(1 if i % timed_every == 0 else 0))
        losses.append(one_step())
    be.sync()
    dt = time.perf_counter() - t0
    launches, gemm_ms, gemm_flops = C.c_uint64(), C.c_double(), C.c_double()
    lib.omx_profile_gemm_report(be._ctx, C.byref(launches), C.byref(gemm_ms), C.byref(gemm_flops))
    lib.omx_profile_gemm(be._ctx, C.c_int32(0))

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
                     "kernel": "gemm_dma_kernel / gemm_kernel (bf16 MFMA GEMM, all operand layouts)" if cfg.bf16
                               else "gemm_kernel<float> (f32 MFMA GEMM, all operand layouts)",
                     "achieved": achieved, "peak": gemm_peak, "unit": "TFLOP/s", "frac": achieved / gemm_peak,
                     "traffic": GEMM_HBM_BYTES_PER_LAUNCH_GPT124M if args.config == "gpt124m" else None,
                     "launches": int(launches.value), "avg_launch_us": gemm_ms.value * 1e3 / max(1, launches.value),
                     "timed_steps": len(range(0, args.steps, timed_every)),
                     "gemm_ms_per_step": gemm_ms.value / max(1, len(range(0, args.steps, timed_every)))},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, min(16, os.cpu_count() or 1))
    tr.close()
    be.close()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
