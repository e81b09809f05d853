#!/usr/bin/env python3
"""Collects the reference's own golden data for this path into tests/golden/.

Run in the build container (needs /root/reference). Only DATA is taken:
  * FNV-1a digests of CPU Exact outputs      ojas-cpu/tests/exact_golden.rs:206-276
  * exp_exact input/output bit pairs         ojas-core/src/exp_exact_pins.txt (copied as is)
  * RMSNorm f64 vector                       ojas-oracle/fixtures/rms_norm_f64.json (copied as is)
  * one-step torch 2.13 float32 vectors      ojas-cpu/tests/torch_ref/data.rs (bit literals -> JSON)
  * torch f64 goldens for embed / CE rows    ojas-cuda/tests/fixtures/goldens/*.npy (copied as is)
  * 100-step torch AdamW parameters/moments  ojas-model/tests/fixtures/adamw_100/adamw_100.safetensors
  * erf / GELU known-answer tables           ojas-core/src/erf_exact.rs:86-140 (numbers -> JSON)
  * AdamW lerp-branch rows                   ojas-cpu/tests/adamw_lerp_oracle.rs (numbers -> JSON)
  * torch 2.13 vectors of the tiny nanolab   ojas-oracle/fixtures/tiny/{init,forward,grads_init}.safetensors and
    model and of stock nanolab's Muon step   muon_step_bf16.safetensors (copied as is)
  * the tiny model's 40-step f32-NS5 trace  ojas-oracle/fixtures/tiny/{trace_ns5_f32,grads_step5}.safetensors,
    (losses, grad norms, step-5 parameters)  its token bin, window starts and LR multipliers: tokens.bin,
                                             batch_starts.json, lr_schedules.json (copied as is)
  * torch's f32 and autocast-bf16 loss curves  ojas-oracle/fixtures/tiny/autocast_gap.json (copied as is)
    over those 40 steps
  * pinned window starts of the batch sampler  ojas-data/tests/sampler.rs:231-254 (numbers -> JSON)
No reference source text is kept: numeric literals are parsed into JSON.
"""
import json
import re
import shutil
from pathlib import Path

REF = Path("/root/reference")
OUT = Path(__file__).resolve().parent


def digests():
    src = (REF / "ojas-cpu/tests/exact_golden.rs").read_text()
    body = src[src.index("const GOLDEN"):]
    pairs = re.findall(r'\("([^"]+)", 0x([0-9a-f]{16})\)', body)
    (OUT / "exact_golden_digests.json").write_text(json.dumps(
        {"source": "ojas-cpu/tests/exact_golden.rs:206-276 (GOLDEN table: FNV-1a digests of CPU Exact outputs)",
         "digests": dict(pairs)}, indent=1))


def torch_ref():
    src = (REF / "ojas-cpu/tests/torch_ref/data.rs").read_text()
    out = {"source": "ojas-cpu/tests/torch_ref/data.rs (torch 2.13.0 float32, B=1 T=4 d=16 vocab=32, 1 head)"}
    for m in re.finditer(r"pub static (\w+): LazyLock<\[f32; (\d+)\]> = LazyLock::new\(\|\| \{(.*?)\}\);", src, re.S):
        name, n, body = m.group(1), int(m.group(2)), m.group(3)
        bits = [int(b, 16) for b in re.findall(r"from_bits\(0x([0-9a-f]+)\)", body)]
        assert len(bits) == n, (name, len(bits), n)
        out[name] = bits
    out["TARGETS"] = [int(x) for x in re.search(r"TARGETS: \[u32; 4\] = \[([^\]]+)\]", src).group(1).split(",")]
    out["LOSS"] = int(re.search(r"LOSS: LazyLock<f32> = LazyLock::new\(\|\| f32::from_bits\(0x([0-9a-f]+)\)", src).group(1), 16)
    out["COSINE_MULT_STEP8"] = int(re.search(r"COSINE_MULT_STEP8.*?f64::from_bits\(0x([0-9a-f]+)\)", src).group(1), 16)
    (OUT / "torch_ref_step.json").write_text(json.dumps(out))


def erf_tables():
    src = (REF / "ojas-core/src/erf_exact.rs").read_text()
    def table(name):
        body = re.search(rf"const {name}: \[\(f64, f64\); \d+\] = \[(.*?)\];", src, re.S).group(1)
        return [[float(a), float(b)] for a, b in re.findall(r"\(([-0-9.e]+), ([-0-9.e]+)\)", body)]
    (OUT / "erf_gelu_tables.json").write_text(json.dumps(
        {"source": "ojas-core/src/erf_exact.rs:86-140 (libm erf and exact GELU values)", "erf": table("ERF"),
         "gelu": table("GELU")}, indent=1))


def sampler_pins():
    src = (REF / "ojas-data/tests/sampler.rs").read_text()
    body = src[src.index("fn permutation_is_pinned"):]
    body = body[:body.index("];")]
    cases = []
    for seed, epoch, starts in re.findall(r"\((0x[0-9A-Fa-f_]+|\d+), (\d+), \[([0-9, ]+)\]\)", body):
        cases.append({"seed": int(seed.replace("_", ""), 0), "epoch": int(epoch),
                      "starts": [int(v) for v in starts.split(",")]})
    assert len(cases) == 6, len(cases)
    (OUT / "sampler_pins.json").write_text(json.dumps(
        {"source": "ojas-data/tests/sampler.rs:231-254 (permutation_is_pinned: bin of 1001 tokens, seq_len 10, "
                   "batch 1, window starts of ordinals 0..8)", "bin_tokens": 1001, "seq_len": 10, "windows": 100,
         "cases": cases}, indent=1))


def copies():
    shutil.copyfile(REF / "ojas-core/src/exp_exact_pins.txt", OUT / "exp_exact_pins.txt")
    shutil.copyfile(REF / "ojas-oracle/fixtures/rms_norm_f64.json", OUT / "rms_norm_f64.json")
    gold = REF / "ojas-cuda/tests/fixtures/goldens"
    (OUT / "cuda_goldens").mkdir(exist_ok=True)
    for f in sorted(gold.glob("embed_*.npy")) + sorted(gold.glob("ce_rows_c*.npy")):
        shutil.copyfile(f, OUT / "cuda_goldens" / f.name)
    (OUT / "adamw_100").mkdir(exist_ok=True)
    for f in ("adamw_100.safetensors", "manifest.json"):
        shutil.copyfile(REF / "ojas-model/tests/fixtures/adamw_100" / f, OUT / "adamw_100" / f)
    (OUT / "tiny").mkdir(exist_ok=True)
    for f in ("init.safetensors", "forward.safetensors", "grads_init.safetensors", "muon_step_bf16.safetensors",
              "trace_ns5_f32.safetensors", "grads_step5.safetensors", "tokens.bin", "batch_starts.json",
              "lr_schedules.json", "autocast_gap.json"):
        shutil.copyfile(REF / "ojas-oracle/fixtures/tiny" / f, OUT / "tiny" / f)


if __name__ == "__main__":
    digests()
    torch_ref()
    erf_tables()
    sampler_pins()
    copies()
    print("fixtures written to", OUT)
