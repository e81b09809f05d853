"""Pins the oracle's group-wise int8 format and LoRA step (oracle/lora_exact.cpp).

The reference holds no fixture for int8 in groups of 32 (parity unpinned by the reference), so the
restatement is held to what the mathematics fixes: a known-answer table of codes and scales worked
by hand from the rule of ojas-cpu/src/quant_sparse.rs:306-326, the special case group == k_in (the
reference's per-channel form, restated here in numpy line by line), brute-force dequantise-then-
multiply in f64, and an independent torch f64 autograd of the whole LoRA graph.
"""
import numpy as np
import pytest
import torch

import oracle_api as orc


def test_quantizer_known_answers():
    # One row, two groups of 4. Group 0: abs_max 2.54 -> scale 0.02; codes round(v * 50).
    # Group 1: all zeros -> scale 1, codes 0 (quant_sparse.rs:312-314).
    w = np.array([[2.54, -1.27, 0.01, -0.03, 0.0, 0.0, 0.0, 0.0]], np.float32)
    codes, scales = orc.quantize_i8_group(w, 4)
    assert codes.tolist() == [[127, -64, 1, -2, 0, 0, 0, 0]]  # -63.5 rounds half away from zero; 0.5 -> 1; -1.5 -> -2
    assert scales[0, 0] == np.float32(2.54) / np.float32(127.0) and scales[0, 1] == 1.0
    # Sign symmetry and the clamp: the extreme value of a group is +-127 exactly, never -128.
    w2 = np.array([[-8.0, 8.0, 4.0, -4.0]], np.float32)
    c2, s2 = orc.quantize_i8_group(w2, 4)
    assert c2.tolist() == [[-127, 127, 64, -64]] and s2[0, 0] == np.float32(8.0) / np.float32(127.0)
    back = orc.dequant_i8_group(c2, s2, 4)
    assert back[0, 0] == -8.0 and back[0, 1] == 8.0  # 127 * (8 / 127) rounds back to 8
    with pytest.raises(orc.OracleError):
        orc.quantize_i8_group(np.array([[np.inf, 0, 0, 0]], np.float32), 4)


def _per_channel_reference(w):
    """QuantizedWeightI8::quantize (quant_sparse.rs:306-326) in numpy."""
    codes = np.empty(w.shape, np.int8)
    scales = np.empty(w.shape[0], np.float32)
    for r, row in enumerate(w):
        abs_max = np.float32(np.max(np.abs(row)))
        scales[r] = abs_max / np.float32(127.0) if abs_max > 0 else np.float32(1.0)
        inv = np.float32(127.0) / abs_max if abs_max > 0 else np.float32(0.0)
        q = row * inv
        q = np.sign(q) * np.floor(np.abs(q) + np.float32(0.5))  # round half away from zero
        codes[r] = np.clip(q, -127, 127).astype(np.int8)
    return codes, scales


def test_group_equal_to_row_is_the_per_channel_form():
    rng = np.random.default_rng(3)
    w = rng.normal(0, 0.02, (24, 96)).astype(np.float32)
    w[5] = 0.0
    codes, scales = orc.quantize_i8_group(w, 96)
    rc, rs = _per_channel_reference(w)
    assert np.array_equal(codes, rc) and np.array_equal(scales[:, 0], rs)
    # dequantize_f32 (quant_sparse.rs:335-344): code as f32 times scale, one rounding.
    assert np.array_equal(orc.dequant_i8_group(codes, scales, 96), rc.astype(np.float32) * rs[:, None])


def test_groups_are_independent_rows_of_the_per_channel_form():
    # Quantising [rows, cols] in groups of g equals the per-channel form of the same data viewed
    # as [rows * cols / g, g]: a transposed or misplaced scale index fails this.
    rng = np.random.default_rng(4)
    w = rng.normal(0, 1.0, (10, 128)).astype(np.float32)
    codes, scales = orc.quantize_i8_group(w, 32)
    rc, rs = _per_channel_reference(w.reshape(-1, 32))
    assert np.array_equal(codes.reshape(-1, 32), rc) and np.array_equal(scales.reshape(-1), rs)
    err = np.abs(orc.dequant_i8_group(codes, scales, 32) - w)
    assert np.all(err <= 0.5 * np.repeat(scales, 32, axis=1) * (1 + 1e-6))  # round to nearest code


def test_quantised_linear_is_dequantise_then_multiply():
    rng = np.random.default_rng(5)
    rows, kin, nout = 7, 64, 9
    x = rng.normal(0, 1, (rows, kin)).astype(np.float32)
    gy = rng.normal(0, 1, (rows, nout)).astype(np.float32)
    codes, scales = orc.quantize_i8_group(rng.normal(0, 0.05, (nout, kin)).astype(np.float32), 32)
    # Brute force in f64 from the codes and scales, element by element.
    y = np.zeros((rows, nout))
    gx = np.zeros((rows, kin))
    for o in range(nout):
        for k in range(kin):
            wv = float(np.float32(codes[o, k]) * scales[o, k // 32])
            y[:, o] += x[:, k].astype(np.float64) * wv
            gx[:, k] += gy[:, o].astype(np.float64) * wv
    got_y = orc.linear_i8_group_forward(x, codes, scales, 32)
    got_gx = orc.linear_i8_group_backward_input(codes, scales, gy, 32)
    assert np.max(np.abs(got_y - y)) <= 1e-5 * np.max(np.abs(y))
    assert np.max(np.abs(got_gx - gx)) <= 1e-5 * np.max(np.abs(gx))
    # ... and bit for bit the Exact linear of the dequantised weight.
    w = orc.dequant_i8_group(codes, scales, 32)
    assert np.array_equal(got_y, orc.linear_forward(x, w))


def _torch_lora(cfg, frozen, adapters, ids, targets):
    """The same graph in torch f64 autograd, written independently of the oracle."""
    t64 = lambda a: torch.tensor(np.asarray(a, np.float64))
    F = [t64(p) for p in frozen]
    A = [t64(p).requires_grad_(True) for p in adapters]
    B, T, H, D, d = cfg.batch, cfg.seq, cfg.heads, cfg.head_dim, cfg.d_model
    half = D // 2
    inv = torch.tensor([cfg.rope_base ** (-2.0 * i / D) for i in range(half)], dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().double(), torch.sin(ang).float().double()  # the tables are rounded to f32

    def norm(x, w):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + cfg.rms_eps) * w

    def rope(x):  # [B,T,H,D], half-split: (x1 cos - x2 sin, x2 cos + x1 sin)
        x1, x2 = x[..., :half], x[..., half:]
        c, s = cos[None, :, None, :], sin[None, :, None, :]
        return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1)

    def lora(x, w, a, b):
        return x @ w.T + (x @ a.T) @ (b * cfg.lora_scale).T

    x = F[0][torch.tensor(np.asarray(ids, np.int64).reshape(-1))]
    for l in range(cfg.layers):
        n1, wq, wk, wv, wo, n2, wg, wu, wd = F[1 + 9 * l: 10 + 9 * l]
        aq, bq, ak, bk, av, bv, ao, bo = A[8 * l: 8 * l + 8]
        h = norm(x, n1)
        q = rope(lora(h, wq, aq, bq).view(B, T, H, D)).transpose(1, 2)
        k = rope(lora(h, wk, ak, bk).view(B, T, H, D)).transpose(1, 2)
        v = lora(h, wv, av, bv).view(B, T, H, D).transpose(1, 2)
        att = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        ap = att.transpose(1, 2).reshape(B * T, d)
        x1 = x + lora(ap, wo, ao, bo)
        h2 = norm(x1, n2)
        x = x1 + (torch.nn.functional.silu(h2 @ wg.T) * (h2 @ wu.T)) @ wd.T
    logits = norm(x, F[-1]) @ F[0].T
    loss = torch.nn.functional.cross_entropy(logits, torch.tensor(np.asarray(targets, np.int64).reshape(-1)))
    loss.backward()
    return float(loss), [a.grad.numpy() for a in A]


def make_lora_case(cfg, seed, group=32):
    """Seeded frozen tensors (matrices as codes + scales and their dequantised values), adapters, batch."""
    rng = np.random.default_rng(seed)
    frozen, quant = [], []
    for shape in orc.lora_frozen_shapes(cfg):
        if len(shape) == 1:
            frozen.append((1.0 + 0.1 * rng.normal(size=shape)).astype(np.float32))
            quant.append(None)
        elif shape[0] == cfg.vocab:
            frozen.append(orc.round_bf16(rng.normal(0, 0.5, shape).astype(np.float32)))
            quant.append(None)
        else:
            codes, scales = orc.quantize_i8_group(rng.normal(0, 0.08, shape).astype(np.float32), group)
            frozen.append(orc.dequant_i8_group(codes, scales, group))
            quant.append((codes, scales))
    adapters = [rng.normal(0, 0.05, s).astype(np.float32) for s in orc.lora_adapter_shapes(cfg)]
    n = cfg.batch * cfg.seq
    ids = rng.integers(0, cfg.vocab, n).astype(np.uint32)
    targets = rng.integers(0, cfg.vocab, n).astype(np.uint32)
    return frozen, quant, adapters, ids, targets


def test_lora_step_matches_torch_f64_autograd():
    cfg = orc.LoraConfig(2, 64, 2, 32, 96, 50, 2, 12, 4, 1e-6, 2.0, 10000.0)
    frozen, _, adapters, ids, targets = make_lora_case(cfg, 11)
    loss, grads = orc.lora_loss_and_grads(cfg, frozen, adapters, ids, targets)
    tloss, tgrads = _torch_lora(cfg, frozen, adapters, ids, targets)
    assert abs(float(loss) - tloss) <= 1e-5 * abs(tloss)
    for i, (g, tg) in enumerate(zip(grads, tgrads)):
        tg = tg.reshape(-1)
        assert np.linalg.norm(tg) > 0, i
        assert np.linalg.norm(g - tg) <= 1e-4 * np.linalg.norm(tg), (i, np.linalg.norm(g - tg) / np.linalg.norm(tg))
    # B = 0 (the adapter's init, lora.rs:9-12): the loss equals the base model's and dA is exactly zero.
    zero_b = [a if i % 2 == 0 else np.zeros_like(a) for i, a in enumerate(adapters)]
    loss0, grads0 = orc.lora_loss_and_grads(cfg, frozen, zero_b, ids, targets)
    other_a = [2 * a if i % 2 == 0 else a for i, a in enumerate(zero_b)]
    assert loss0 == orc.lora_loss_and_grads(cfg, frozen, other_a, ids, targets, want_grads=False)[0]
    assert all(not np.any(g) for g in grads0[0::2]) and all(np.any(g) for g in grads0[1::2])
