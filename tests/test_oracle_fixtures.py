"""The oracle against the reference's own fixtures and known-answer tables
(everything but the 68 digests, which have their own file), and against what
the mathematics fixes where no fixture reaches."""
import json
import math
from pathlib import Path

import numpy as np
import pytest

import oracle_api as orc

GOLD = Path(__file__).parent / "golden"


def f32_from_bits(bits):
    return np.array(bits, dtype=np.uint32).view(np.float32)


# ---- exp_exact: ojas-core/src/exp_exact_pins.txt + the edge cases of exp_exact.rs:194-211 ----
def test_exp_exact_matches_every_pinned_correctly_rounded_value():
    pairs = [line.split() for line in (GOLD / "exp_exact_pins.txt").read_text().splitlines()
             if line and not line.startswith("#")]
    assert len(pairs) > 2000
    x = f32_from_bits([int(a, 16) for a, _ in pairs])
    want = np.array([int(b, 16) for _, b in pairs], dtype=np.uint32)
    got = orc.exp_exact_vec(x).view(np.uint32)
    assert np.array_equal(got, want)


def test_exp_exact_special_values_and_range_edges():
    assert math.isnan(orc.exp_exact(float("nan")))
    assert orc.exp_exact(float("inf")) == float("inf")
    assert orc.exp_exact(float("-inf")) == 0.0
    assert orc.exp_exact(0.0) == 1.0 and orc.exp_exact(-0.0) == 1.0
    edge = lambda bits: orc.exp_exact_vec(f32_from_bits([bits])).view(np.uint32)[0]
    assert edge(0x42B17217) == 0x7F7FFF84  # last finite result
    assert edge(0x42B17218) == 0x7F800000
    assert edge(0xC2CFF1B4) == 1           # smallest subnormal
    assert edge(0xC2CFF1B5) == 0


def test_log_sum_exp_and_log1p_against_libm():
    r = orc.SplitMix64(1)
    for _ in range(2000):
        m = float(r.vec(1, 50.0)[0])
        s = float(abs(r.vec(1, 1000.0)[0])) + 1e-3
        want = np.float32(np.float64(np.float32(m)) + math.log(np.float64(np.float32(s))))
        got = np.float32(orc.log_sum_exp_exact(m, s))
        assert abs(float(got) - float(want)) <= 1.2e-7 * max(1.0, abs(float(want)))
    for x in [0.0, 1e-30, 2.0**-24, 1e-3, 0.5, 1.0]:
        assert abs(orc.log1p_exact(x) - math.log1p(np.float64(np.float32(x)))) <= 1.2e-7 * max(math.log1p(x), 1e-38)
    assert math.isnan(orc.log1p_exact(1.5)) and math.isnan(orc.log1p_exact(-0.1))


# ---- erf / GELU: known-answer tables of ojas-core/src/erf_exact.rs:86-140 ----
def test_erf_and_gelu_known_answers():
    tables = json.loads((GOLD / "erf_gelu_tables.json").read_text())
    for x, want in tables["erf"]:
        assert abs(orc.erf_f64(x) - want) <= 1e-14 * max(abs(want), 1e-300)
    for x, want in tables["gelu"]:
        got = orc.gelu_erf(x)
        assert abs(got - want) <= 1.2e-7 * abs(want) + 1e-14


def test_gelu_forms_against_scipy_and_finite_differences():
    from scipy.special import erf

    xs = np.arange(-6.0, 6.0, 0.0731)
    for x in xs:
        xf = float(np.float32(x))
        want = 0.5 * xf * (1.0 + erf(xf / math.sqrt(2.0)))
        assert abs(orc.gelu_erf(xf) - want) <= 1.2e-7 * abs(want) + 1e-14
        t = math.tanh(0.7978845608028654 * (xf + 0.044715 * xf ** 3))
        want_t = 0.5 * xf * (1.0 + t)
        assert abs(orc.gelu_tanh(xf) - want_t) <= 1.2e-7 * abs(want_t) + 1e-12
        # Derivatives against central differences of the f64 closed forms.
        h = 1e-5
        f = lambda z: 0.5 * z * (1.0 + erf(z / math.sqrt(2.0)))
        g = lambda z: 0.5 * z * (1.0 + math.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        assert abs(orc.gelu_erf_backward(xf, 1.0) - (f(xf + h) - f(xf - h)) / (2 * h)) <= 1e-6
        assert abs(orc.gelu_tanh_backward(xf, 1.0) - (g(xf + h) - g(xf - h)) / (2 * h)) <= 1e-6
    # gelu_tanh.rs:95-107: limits.
    assert np.float32(orc.gelu_tanh(-20.0)).view(np.uint32) == np.float32(-0.0).view(np.uint32)
    assert orc.gelu_tanh(30.0) == 30.0


# ---- bf16 rule: ojas-core/src/autocast.rs:70-96 ----
def test_bf16_rounding_rule():
    cases = {0x3F800000: 0x3F80, 0x3F808000: 0x3F80, 0x3F808001: 0x3F81, 0x3F818000: 0x3F82, 0x7F7FFFFF: 0x7F80,
             0xFF7FFFFF: 0xFF80, 0x80000000: 0x8000, 0x7F800001: 0x7FC0, 0xFFC12345: 0xFFC1, 0x7FBFFFFF: 0x7FFF,
             0x00000001: 0x0000, 0x00008001: 0x0001}
    x = f32_from_bits(list(cases))
    assert np.array_equal(orc.to_bf16(x), np.array(list(cases.values()), np.uint16))
    widened = orc.bf16_to_f32(orc.to_bf16(x))
    assert np.array_equal(widened.view(np.uint32), np.array(list(cases.values()), np.uint32) << 16)


def test_bf16_round_to_nearest_even_against_brute_force():
    r = orc.SplitMix64(3)
    x = np.concatenate([r.vec(20000, 1000.0), r.vec(20000, 1e-3)])
    got = orc.to_bf16(x).astype(np.uint32) << 16
    lo = x.view(np.uint32) & 0xFFFF0000
    hi = lo + 0x10000
    xf = x.astype(np.float64)
    lo_f, hi_f = lo.view(np.float32).astype(np.float64), hi.view(np.float32).astype(np.float64)
    nearest = np.where(np.abs(xf - lo_f) < np.abs(hi_f - xf), lo, hi)
    tie = np.abs(xf - lo_f) == np.abs(hi_f - xf)
    nearest = np.where(tie, np.where((lo >> 16) & 1 == 0, lo, hi), nearest)
    assert np.array_equal(got, nearest.astype(np.uint32))


# ---- host scalars: unit tests inside ojas-core/src/backend.rs:3548-3680 ----
def test_pow_u64_clip_scale_and_adamw_scalars():
    assert orc.pow_u64(0.9, 0) == 1.0 and orc.pow_u64(0.9, 1) == 0.9
    assert abs(orc.pow_u64(0.95, 1000) - 0.95 ** 1000) <= 1e-12 * 0.95 ** 1000
    assert orc.clip_scale(1.0, 0.5) == 1.0
    assert orc.clip_scale(1.0, 4.0) == float(np.float32(1.0) / (np.float32(4.0) + np.float32(1e-6)))
    assert orc.clip_scale(float("inf"), 3.0) == 1.0
    with pytest.raises(orc.OracleError) as e:
        orc.clip_scale(-1.0, 1.0)
    assert e.value.code == orc.OUT_OF_RANGE
    with pytest.raises(orc.OracleError) as e:
        orc.clip_scale(1.0, float("nan"))
    assert e.value.code == orc.NON_FINITE
    words, flags = orc.adamw_scalars(3e-3, 0.9, 0.95, 1e-8, 0.1, 9)
    bc1, bc2 = 1.0 - 0.9 ** 10, 1.0 - 0.95 ** 10
    assert words[0] == 1.0 - 3e-3 * 0.1 and abs(words[4] - 3e-3 / bc1) < 1e-15 and abs(words[5] - math.sqrt(bc2)) < 1e-15
    assert flags == [1, 1, 1]
    for bad in [(1e-3, 1.0, 0.9, 1e-8, 0.0), (1e-3, 0.9, 0.9, 0.0, 0.0), (-1e-3, 0.9, 0.9, 1e-8, 0.0)]:
        with pytest.raises(orc.OracleError) as e:
            orc.adamw_scalars(*bad, 0)
        assert e.value.code == orc.OUT_OF_RANGE
    with pytest.raises(orc.OracleError):
        orc.adamw_scalars(1e-3, 0.9, 0.9, 1e-8, 0.0, 2 ** 64 - 1)


# ---- RMSNorm: ojas-oracle/fixtures/rms_norm_f64.json ----
def test_rms_norm_f64_fixture():
    fx = json.loads((GOLD / "rms_norm_f64.json").read_text())
    x = np.array(fx["input"], np.float32).reshape(1, -1)
    w = np.array(fx["weight"], np.float32)
    got = orc.rms_norm_forward(x, w, fx["eps"]).reshape(-1)
    assert np.max(np.abs(got.astype(np.float64) - np.array(fx["expected"]))) <= 2e-7 * np.max(np.abs(fx["expected"]))


# ---- one torch 2.13 float32 step: ojas-cpu/tests/torch_ref.rs:100-262, gate 1e-4 absolute ----
def test_one_step_matches_torch_2_13_float32():
    fx = json.loads((GOLD / "torch_ref_step.json").read_text())
    t = {k: f32_from_bits(v) for k, v in fx.items() if isinstance(v, list) and k != "TARGETS"}
    b, T, d, vocab = 1, 4, 16, 32
    x, norm_w = t["X"].reshape(T, d), t["NORM_W0"]
    wq, wk, wv, wo = t["WQ0"].reshape(d, d), t["WK0"].reshape(d, d), t["WV0"].reshape(d, d), t["WO0"].reshape(vocab, d)
    cos, sin = t["COS"].reshape(T, d), t["SIN"].reshape(T, d)
    targets = np.array(fx["TARGETS"], np.uint32)
    h = orc.rms_norm_forward(x, norm_w, 1e-6)
    q, k, v = orc.linear_forward(h, wq), orc.linear_forward(h, wk), orc.linear_forward(h, wv)
    q_r = orc.rope_forward(q.reshape(b, T, 1, d), cos, sin).reshape(b, 1, T, d)
    k_r = orc.rope_forward(k.reshape(b, T, 1, d), cos, sin).reshape(b, 1, T, d)
    v_a = v.reshape(b, 1, T, d)
    attn, lse = orc.causal_sdpa_forward(q_r, k_r, v_a)
    y = attn.reshape(T, d)
    logits = orc.linear_forward(y, wo)
    loss = orc.cross_entropy_mean_forward(logits, targets)
    g_logits = orc.cross_entropy_mean_backward(logits, targets)
    g_y, _ = orc.linear_backward(y, wo, g_logits)
    g_q, g_k, g_v = orc.causal_sdpa_backward(q_r, k_r, v_a, attn, lse, g_y.reshape(b, 1, T, d))
    g_q_lin = orc.rope_backward(g_q.reshape(b, T, 1, d), cos, sin).reshape(T, d)
    g_k_lin = orc.rope_backward(g_k.reshape(b, T, 1, d), cos, sin).reshape(T, d)
    gq_h, g_wq = orc.linear_backward(h, wq, g_q_lin)
    gk_h, _ = orc.linear_backward(h, wk, g_k_lin)
    gv_h, _ = orc.linear_backward(h, wv, g_v.reshape(T, d))
    g_h = gq_h + gk_h + gv_h
    _, g_norm = orc.rms_norm_backward(x, norm_w, g_h, 1e-6)
    # Cosine schedule, warmup 4 of 20, step 8, floor 0.1 (ojas-cpu/src/schedule.rs:66-92).
    tt = (8 - 4) / (20 - 4)
    mult = 0.1 + 0.9 * 0.5 * (1.0 + math.cos(math.pi * tt))
    want_mult = np.array([fx["COSINE_MULT_STEP8"]], np.uint64).view(np.float64)[0]
    assert abs(mult - want_mult) <= 1e-15
    lr = 6e-4 * mult
    wq_after, _, _ = orc.adamw_step(wq, g_wq, np.zeros_like(wq), np.zeros_like(wq), 0, lr, weight_decay=0.1)
    norm_after, _, _ = orc.adamw_step(norm_w, g_norm, np.zeros_like(norm_w), np.zeros_like(norm_w), 0, lr,
                                      weight_decay=0.0)
    err = lambda got, name: float(np.max(np.abs(np.asarray(got, np.float64).reshape(-1) - t[name].astype(np.float64))))
    assert err(h, "H") <= 1e-4 and err(attn, "ATTN") <= 1e-4 and err(logits, "LOGITS") <= 1e-4
    assert abs(float(loss) - float(f32_from_bits([fx["LOSS"]])[0])) <= 1e-4
    assert err(g_wq, "GWQ") <= 1e-4 and err(g_norm, "GWN") <= 1e-4
    assert err(wq_after, "WQ_AFTER") <= 1e-4 and err(norm_after, "NORM_AFTER") <= 1e-4


# ---- torch f64 goldens: ojas-cuda/tests/fixtures/goldens (embed, CE over rows of a tied head) ----
def test_embedding_goldens():
    g = lambda n: np.load(GOLD / "cuda_goldens" / f"embed_{n}.npy")
    ids = g("ids").astype(np.uint32)
    table = g("table").astype(np.float32)
    y = orc.embedding_forward(table, ids)
    assert np.array_equal(y, g("y").astype(np.float32))
    dt = orc.embedding_backward(ids, g("dy").astype(np.float32), table.shape[0])
    assert np.max(np.abs(dt.astype(np.float64) - g("dtable"))) <= 1e-6


@pytest.mark.parametrize("case", [0, 2])
def test_linear_cross_entropy_goldens_including_the_planted_margin(case):
    g = lambda n: np.load(GOLD / "cuda_goldens" / f"ce_rows_c{case}_{n}.npy")
    rows = g("rows").astype(np.int64)
    h = g("h")[rows].astype(np.float32)
    w = g("w").astype(np.float32)
    targets = g("targets").astype(np.uint32)
    assert float(g("scale")[0]) == 1.0
    loss, gx, gw = orc.linear_cross_entropy_mean(h, w, targets)
    # f32 arithmetic against an f64 golden of f64 inputs: 1e-5 relative on the loss.
    assert abs(float(loss) - float(g("loss")[0])) <= 1e-5 * abs(float(g("loss")[0]))
    assert np.max(np.abs(gx.astype(np.float64) - g("dh"))) <= 1e-5 * max(np.max(np.abs(g("dh"))), 1e-30)
    assert np.max(np.abs(gw.astype(np.float64) - g("dw"))) <= 1e-5 * max(np.max(np.abs(g("dw"))), 1e-30)


# ---- 100 torch AdamW steps: ojas-model/tests/adamw_torch_100.rs + fixtures/adamw_100 ----
def _hash32(salt, step, tensor, index):
    m = 0xFFFFFFFF
    x = (salt * 0x27D4EB2F + step * 0x9E3779B1 + tensor * 0x165667B1 + index * 0xC2B2AE35 + 0x85EBCA6B) & m
    x ^= x >> 16
    x = (x * 0x85EBCA6B) & m
    x ^= x >> 13
    x = (x * 0xC2B2AE35) & m
    return x ^ (x >> 16)


def test_adamw_100_steps_against_torch():
    from safetensors.numpy import load_file

    fx = load_file(str(GOLD / "adamw_100" / "adamw_100.safetensors"))
    bound = float(fx["bound"][0])
    tensors = [("lora_A", (16, 64), 2e-4, 0.01), ("lora_B", (64, 16), 2e-4, 0.01), ("d17", (17, 64), 1e-4, 0.01),
               ("span_head", (2, 64), 1e-4, 0.01), ("norm_nodecay", (64,), 1e-4, 0.0)]
    zero_grad = [(1, 30, 39), (4, 1, 3)]
    signed24 = lambda h: (h >> 8) - (1 << 23)
    for exact in (True, False):
        for tid, (name, shape, lr, wd) in enumerate(tensors):
            n = int(np.prod(shape))
            offset = np.array([signed24(_hash32(3, 0, tid, i)) >> 1 for i in range(n)], np.int64)
            p = (np.array([signed24(_hash32(1, 0, tid, i)) for i in range(n)], np.float32) * np.float32(2.0 ** -27))
            m = np.zeros(n, np.float32)
            v = np.zeros(n, np.float32)
            for step in range(1, 101):
                if any(t == tid and a <= step <= b for t, a, b in zero_grad):
                    g = np.zeros(n, np.float32)
                else:
                    noise = np.array([signed24(_hash32(2, step, tid, i)) for i in range(n)], np.int64)
                    g = (noise + offset).astype(np.float32) * np.float32(2.0 ** -33)
                p, m, v = orc.adamw_step(p, g, m, v, step - 1, lr, 0.9, 0.999, 1e-8, wd, exact=exact)
                if step in (1, 10, 50, 100):
                    ref = fx[f"p{step}.{name}"].reshape(-1).astype(np.float64)
                    assert np.max(np.abs(p - ref)) / np.max(np.abs(ref)) <= bound, (name, step, exact)
            for tag, got in (("m100", m), ("v100", v)):
                ref = fx[f"{tag}.{name}"].reshape(-1).astype(np.float64)
                assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= bound, (name, tag, exact)


# ---- what no fixture reaches: brute force and closed forms ----
def _attention_brute_force(q, k, v, window):
    b, h, t, d = q.shape
    hkv = k.shape[1]
    rep = h // hkv
    out = np.zeros_like(q, dtype=np.float64)
    lse = np.zeros((b, h, t))
    for bi in range(b):
        for hi in range(h):
            kk, vv = k[bi, hi // rep].astype(np.float64), v[bi, hi // rep].astype(np.float64)
            s = q[bi, hi].astype(np.float64) @ kk.T / math.sqrt(d)
            for ti in range(t):
                lo = max(0, ti + 1 - window) if window else 0
                row = s[ti, lo:ti + 1]
                mx = row.max()
                e = np.exp(row - mx)
                out[bi, hi, ti] = (e / e.sum()) @ vv[lo:ti + 1]
                lse[bi, hi, ti] = mx + math.log(e.sum())
    return out, lse


@pytest.mark.parametrize("shape,hkv,window", [((2, 4, 37, 8), 2, 0), ((1, 6, 50, 16), 2, 9), ((1, 2, 20, 4), 2, 1),
                                              ((1, 3, 33, 24), 3, 100)])
def test_sdpa_window_and_gqa_against_brute_force_and_finite_differences(shape, hkv, window):
    b, h, t, d = shape
    r = orc.SplitMix64(17)
    q = r.vec(b * h * t * d, 0.7).reshape(shape)
    k = r.vec(b * hkv * t * d, 0.7).reshape(b, hkv, t, d)
    v = r.vec(b * hkv * t * d, 0.7).reshape(b, hkv, t, d)
    gy = r.vec(b * h * t * d, 0.7).reshape(shape)
    out, lse = orc.causal_sdpa_forward(q, k, v, window)
    bo, bl = _attention_brute_force(q, k, v, window)
    assert np.max(np.abs(out - bo)) <= 2e-6 and np.max(np.abs(lse - bl)) <= 2e-6
    gq, gk, gv = orc.causal_sdpa_backward(q, k, v, out, lse, gy, window)
    loss = lambda q_, k_, v_: float(np.sum(_attention_brute_force(q_, k_, v_, window)[0] * gy))
    eps = 1e-3
    for arr, grad in ((q, gq), (k, gk), (v, gv)):
        for _ in range(6):
            idx = tuple(r.below(s) for s in arr.shape)
            plus, minus = arr.astype(np.float64).copy(), arr.astype(np.float64).copy()
            plus[idx] += eps
            minus[idx] -= eps
            args_p = [plus if a is arr else a for a in (q, k, v)]
            args_m = [minus if a is arr else a for a in (q, k, v)]
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - float(grad[idx])) <= 2e-5 * max(1.0, abs(fd)), (idx, fd, grad[idx])


def test_cross_entropy_against_torch_and_row_sum_invariant():
    import torch
    import torch.nn.functional as F

    r = orc.SplitMix64(23)
    rows, vocab = 40, 97
    logits = r.vec(rows * vocab, 5.0).reshape(rows, vocab)
    targets = np.array([r.below(vocab) for _ in range(rows)], np.uint32)
    targets[::7] = 3
    t = torch.tensor(logits.astype(np.float64), requires_grad=True)
    loss = F.cross_entropy(t, torch.tensor(targets.astype(np.int64)), ignore_index=3)
    loss.backward()
    assert abs(float(orc.cross_entropy_mean_forward(logits, targets, 3)) - float(loss)) <= 1e-6 * float(loss)
    grad = orc.cross_entropy_mean_backward(logits, targets, 3)
    assert np.max(np.abs(grad - t.grad.numpy())) <= 1e-7
    assert np.max(np.abs(grad.astype(np.float64).sum(axis=1))) <= 1e-7  # numerical_invariants.rs T1
    assert np.all(grad[targets == 3] == 0.0)
    with pytest.raises(orc.OracleError) as e:
        orc.cross_entropy_mean_forward(logits, np.full(rows, 3, np.uint32), 3)
    assert e.value.code == orc.NON_FINITE
    bad = targets.copy()
    bad[1] = vocab
    with pytest.raises(orc.OracleError) as e:
        orc.cross_entropy_mean_forward(logits, bad, 3)
    assert e.value.code == orc.OUT_OF_RANGE


def test_gemm_chain_is_the_naive_triple_loop_and_fused_ce_is_the_composed_path():
    r = orc.SplitMix64(29)
    a, b = r.vec(7 * 13, 1.0).reshape(7, 13), r.vec(13 * 5, 1.0).reshape(13, 5)
    want = np.zeros((7, 5), np.float32)
    for i in range(7):
        for j in range(5):
            acc = np.float32(0.0)
            for p in range(13):
                acc = np.float32(acc + np.float32(a[i, p] * b[p, j]))
            want[i, j] = acc
    assert np.array_equal(orc.gemm(a, b), want)
    assert np.array_equal(orc.gemm(a, b.T.copy().T), want)  # strides do not change the chain
    x, w = r.vec(9 * 6, 1.0).reshape(9, 6), r.vec(20 * 6, 0.5).reshape(20, 6)
    targets = np.array([r.below(20) for _ in range(9)], np.uint32)
    loss, gx, gw = orc.linear_cross_entropy_mean(x, w, targets)
    logits = orc.linear_forward(x, w)
    g = orc.cross_entropy_mean_backward(logits, targets)
    cgx, cgw = orc.linear_backward(x, w, g)
    assert loss == orc.cross_entropy_mean_forward(logits, targets)
    assert np.array_equal(gx, cgx) and np.array_equal(gw, cgw)  # framework_ce.rs:1-10


def test_muon_contracts_singular_values_toward_one():
    # numerical_invariants.rs T5: five Newton-Schulz steps push the singular values of the
    # normalised update into a band about one.
    r = orc.SplitMix64(31)
    for rows, cols, bf16 in ((48, 64, False), (130, 70, False), (64, 48, True)):
        p = np.zeros((rows, cols), np.float32)
        g = r.vec(rows * cols, 1.0).reshape(rows, cols)
        m = np.zeros_like(p)
        p2, m2 = orc.muon_ns5_step(p, g, m, lr=1.0, momentum=0.0, weight_decay=0.0, nesterov=False, bf16=bf16)
        assert np.array_equal(m2, g)
        ortho = -p2 / math.sqrt(max(1.0, rows / cols))
        sv = np.linalg.svd(ortho.astype(np.float64), compute_uv=False)
        assert sv.max() < 1.3 and sv.min() > 0.3, (sv.min(), sv.max())


def test_argmax_and_topk_against_brute_force():
    r = orc.SplitMix64(37)
    x = np.round(r.vec(12 * 40, 5.0)).reshape(12, 40).astype(np.float32)
    x[0, 5], x[0, 9] = -0.0, 0.0
    assert np.array_equal(orc.argmax_rows(x), np.argmax(x, axis=1).astype(np.uint32))
    vals, ids = orc.topk_rows(x, 7)
    for row in range(12):
        order = sorted(range(40), key=lambda i: (-(x[row, i] + 0.0), i))[:7]
        assert list(ids[row]) == order
        assert np.array_equal(vals[row], x[row, order])
    bad = x.copy()
    bad[3, 3] = np.inf
    with pytest.raises(orc.OracleError):
        orc.topk_rows(bad, 3)
    with pytest.raises(orc.OracleError):
        orc.argmax_rows(np.where(x == x[0, 0], -np.inf, x).astype(np.float32))


# ---- graph-B pointwise ops: the known answers of ojas-cpu/tests/ops.rs:599-623,667-696, and f64
# autograd for what those leave open (a wrong sign, a swapped operand or a dropped term fails) ----
def test_silu_and_mul_known_answers_and_derivatives():
    import torch

    y = orc.silu_forward(np.array([0.0, 1.0, -1.0], np.float32))
    s1 = 1.0 / (1.0 + math.exp(-1.0))
    assert abs(y[0]) < 1e-6 and abs(y[1] - s1) < 1e-6 and abs(y[2] + (1.0 - s1)) < 1e-6
    a, b = np.array([2.0, -3.0], np.float32), np.array([4.0, 0.5], np.float32)
    assert list(orc.mul_forward(a, b)) == [8.0, -1.5]
    ga, gb = orc.mul_backward(a, b, np.ones(2, np.float32))
    assert list(ga) == list(b) and list(gb) == list(a)
    r = orc.SplitMix64(41)
    x, gy = r.vec(4000, 6.0), r.vec(4000, 1.0)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = torch.nn.functional.silu(xt)
    yt.backward(torch.tensor(gy, dtype=torch.float64))
    np.testing.assert_allclose(orc.silu_forward(x), yt.detach().numpy(), rtol=3e-7, atol=1e-7)
    np.testing.assert_allclose(orc.silu_backward(x, gy), xt.grad.numpy(), rtol=1e-6, atol=2e-7)
    ga, gb = orc.mul_backward(x, gy, x)
    assert np.array_equal(ga, x * gy) and np.array_equal(gb, x * x)


def test_per_head_gate_known_answers_and_autograd():
    import torch

    y = orc.gate_forward(np.array([[1.0, 2.0]], np.float32), np.eye(2, dtype=np.float32), np.zeros(2, np.float32),
                         np.ones((1, 2, 1), np.float32))
    assert abs(y[0, 0, 0] - 1.0 / (1.0 + math.exp(-1.0))) < 1e-6
    assert abs(y[0, 1, 0] - 1.0 / (1.0 + math.exp(-2.0))) < 1e-6
    r = orc.SplitMix64(43)
    rows, din, heads, dh = 37, 24, 3, 8
    x = r.vec(rows * din, 1.0).reshape(rows, din)
    w = r.vec(heads * din, 0.5).reshape(heads, din)
    bias = r.vec(heads, 0.5)
    attn = r.vec(rows * heads * dh, 1.0).reshape(rows, heads, dh)
    gy = r.vec(rows * heads * dh, 1.0).reshape(rows, heads, dh)
    t = lambda a: torch.tensor(a, dtype=torch.float64, requires_grad=True)
    xt, wt, bt, at = t(x), t(w), t(bias), t(attn)
    yt = at * torch.sigmoid(xt @ wt.T + bt)[:, :, None]
    yt.backward(torch.tensor(gy, dtype=torch.float64))
    np.testing.assert_allclose(orc.gate_forward(x, w, bias, attn), yt.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(orc.gate_values(x, w, bias), torch.sigmoid(xt @ wt.T + bt).detach().numpy(), rtol=1e-5)
    gx, gw, gb, ga = orc.gate_backward(x, w, bias, attn, gy)
    for got, want in ((gx, xt.grad), (gw, wt.grad), (gb, bt.grad), (ga, at.grad)):
        want = want.numpy()
        assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
    # The bias is the first term of each logit's chain: with a zero input the gate is sigmoid(b).
    zero = orc.gate_values(np.zeros((2, din), np.float32), w, bias)
    assert np.array_equal(zero[0], np.array([orc.sigmoid_exact(float(v)) for v in bias], np.float32))
    with pytest.raises(orc.OracleError):
        orc.gate_forward(np.full((1, din), np.nan, np.float32), w, bias, attn[:1])


def test_value_residual_blend_known_answers_and_autograd():
    import torch

    out = orc.value_residual_forward(np.array([2.0, 2.0], np.float32), np.array([4.0, 6.0], np.float32), 0.0)
    assert list(out) == [3.0, 4.0]
    r = orc.SplitMix64(47)
    n, lam = 5000, 0.7
    v, v0, gy = r.vec(n, 1.0), r.vec(n, 1.0), r.vec(n, 1.0)
    t = lambda a: torch.tensor(a, dtype=torch.float64, requires_grad=True)
    vt, v0t, lt = t(v), t(v0), t(np.float64(np.float32(lam)))
    s = torch.sigmoid(lt)
    outt = (1 - s) * vt + s * v0t
    outt.backward(torch.tensor(gy, dtype=torch.float64))
    np.testing.assert_allclose(orc.value_residual_forward(v, v0, lam), outt.detach().numpy(), rtol=1e-6, atol=1e-7)
    gv, gv0, gl = orc.value_residual_backward(v, v0, lam, gy)
    np.testing.assert_allclose(gv, vt.grad.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(gv0, v0t.grad.numpy(), rtol=1e-6, atol=1e-7)
    assert abs(gl - lt.grad.item()) < 1e-4 * max(1.0, abs(lt.grad.item()))
    with pytest.raises(orc.OracleError):
        orc.value_residual_forward(v, v0, float("nan"))
