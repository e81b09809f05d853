"""The `ojas-mi355x` crate (Rust source for the reference's workspace; no Rust toolchain here, so it
is checked as text): `src/ffi.rs` is what `gen_ffi.py` makes of `include/ojas_mi355x.h` today, it
declares every entry point with the header's argument count, every `ffi::omx_*` call in
`src/backend.rs` passes that many arguments, and the backend implements every trait method the
reference leaves without a default (ojas-core/src/backend.rs, `BackendCore` .. `BackendModule`) plus
the ones of the GPT op set that have one."""
import re
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CRATE = ROOT / "ojas-mi355x"


def header_functions():
    text = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / "ojas_mi355x.h").read_text(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(omx_\w+)\s*\(([^;{]*?)\)\s*;", text, re.S):
        params = m.group(2).strip()
        out[m.group(1)] = 0 if params in ("", "void") else params.count(",") + 1
    return out


def split_args(text: str):
    """Top-level comma split of a call's argument text."""
    args, depth, current = [], 0, ""
    for ch in text:
        if ch in "([{<" and not current.endswith("-"):
            depth += 1
        elif ch in ")]}>" and not current.endswith("-"):
            depth -= 1
        if ch == "," and depth == 0:
            args.append(current)
            current = ""
        else:
            current += ch
    if current.strip():
        args.append(current)
    return args


def test_ffi_is_the_generators_output_for_the_current_header():
    rc = subprocess.run([sys.executable, str(CRATE / "gen_ffi.py"), "--check"], capture_output=True, text=True)
    assert rc.returncode == 0, rc.stderr


def test_ffi_declares_every_entry_point_with_the_headers_argument_count():
    header = header_functions()
    assert len(header) >= 80
    ffi = (CRATE / "src" / "ffi.rs").read_text()
    declared = {m.group(1): len(split_args(m.group(2))) for m in re.finditer(r"pub fn (omx_\w+)\((.*?)\)(?: -> [^;]+)?;", ffi)}
    assert set(declared) == set(header), set(declared) ^ set(header)
    for name, count in header.items():
        assert declared[name] == count, (name, declared[name], count)
    for status in ("OMX_OK", "OMX_SHAPE", "OMX_PLACEMENT", "OMX_F32", "OMX_BF16", "OMX_U32"):
        assert re.search(rf"pub const {status}: i32 = \d+;", ffi), status


def test_every_ffi_call_in_the_crate_passes_the_declared_number_of_arguments():
    header = header_functions()
    calls = 0
    for source in ("backend.rs", "buffer.rs"):
        text = (CRATE / "src" / source).read_text()
        for m in re.finditer(r"ffi::(omx_\w+)\(", text):
            name = m.group(1)
            assert name in header, (source, name)
            depth, i = 1, m.end()
            while depth:
                depth += {"(": 1, ")": -1}.get(text[i], 0)
                i += 1
            args = split_args(text[m.end():i - 1])
            assert len(args) == header[name], (source, name, len(args), header[name])
            calls += 1
    assert calls >= 50


REQUIRED = """id budget silu_forward silu_backward mul_forward mul_backward residual_add_forward residual_add_backward
clip_grad_norm embedding_forward embedding_backward linear_forward linear_backward rms_norm_forward rms_norm_backward
rope_half_split_forward rope_half_split_backward rms_qk_norm_forward rms_qk_norm_backward causal_sdpa_forward
causal_sdpa_backward per_head_sigmoid_gate_forward per_head_sigmoid_gate_backward value_residual_blend_forward
value_residual_blend_backward cross_entropy_mean_forward cross_entropy_mean_backward adamw_step muon_ns5_step""".split()
GPT_SET_WITH_DEFAULTS = """numerics bf16_operands upload download sync optimizer_scratch_bytes cast_bf16 to_bf16 to_f32 permute
gelu_erf_forward gelu_erf_backward gelu_tanh_forward gelu_tanh_backward accumulate_grad scale_grad argmax_rows topk_rows
linear_backward_input causal_sdpa_backward_recompute per_head_sigmoid_gate_forward_saving
per_head_sigmoid_gate_backward_saved linear_cross_entropy_mean cached_attention_forward kv_cache_write""".split()


def test_backend_implements_the_required_methods_and_the_gpt_op_set():
    text = (CRATE / "src" / "backend.rs").read_text()
    for trait in ("BackendCore", "BackendFloat", "BackendInt", "BackendModule", "Backend"):
        assert re.search(rf"impl {trait} for Mi355xBackend", text), trait
    methods = set(re.findall(r"\n    fn (\w+)\(", text))
    missing = [m for m in REQUIRED + GPT_SET_WITH_DEFAULTS if m not in methods]
    assert not missing, missing
    # Every op runs its shared validator before anything else (docs/shape-contract.md).
    for validator in ("linear_forward_dims", "causal_sdpa_backward_dims", "rms_norm_backward_dims", "embedding_backward_dims",
                      "linear_ce_dims", "adamw_step_dims", "muon_ns5_step_dims", "clip_grad_norm_dims", "kv_cache_write_dims"):
        assert f"{validator}(" in text, validator
