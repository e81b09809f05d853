"""GPU parity of the LoRA fine-tune path (int8 group weights, head_dim 128 attention, the step)
against the oracle (oracle/lora_exact.cpp), through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import oracle_api as orc

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2  # per element, relative to the tensor's largest value (the bf16 tier's gate)


@pytest.fixture(scope="module")
def be():
    from ojas_amd.backend import MiBackend

    b = MiBackend(0)
    yield b
    b.close()


def _close(got, want, tol=BF16_TOL):
    scale = max(float(np.max(np.abs(want))), 1e-12)
    err = float(np.max(np.abs(got - want)))
    assert err <= tol * scale, (err / scale, got.shape)


# (rows, k_in, n_out): tile-exact, ragged in every direction, one step, many steps.
Q8_SHAPES = [(256, 64, 128), (300, 96, 100), (77, 32, 36), (512, 2048, 256), (1024, 256, 416), (33, 704, 160)]


@pytest.mark.parametrize("rows,kin,nout", Q8_SHAPES)
@pytest.mark.parametrize("with_add", [False, True])
def test_linear_i8_group_forward(be, rows, kin, nout, with_add):
    from ojas_amd.backend import BF16

    print(f"q8 forward rows={rows} kin={kin} nout={nout} add={with_add}", flush=True)
    rng = np.random.default_rng(rows * 7 + kin)
    x = orc.round_bf16(rng.normal(0, 1, (rows, kin)).astype(np.float32))
    codes, scales = orc.quantize_i8_group(rng.normal(0, 0.05, (nout, kin)).astype(np.float32) *
                                          rng.uniform(0.2, 3.0, (nout, 1)).astype(np.float32), 32)
    add = orc.round_bf16(rng.normal(0, 0.3, (rows, nout)).astype(np.float32)) if with_add else None
    want = orc.linear_i8_group_forward(x, codes, scales, 32) + (add if with_add else 0)
    y = be.linear_i8_group_forward(be.upload(x, BF16), be.upload(codes), be.upload(scales),
                                   be.upload(add, BF16) if with_add else None)
    _close(be.download_f32(y), want)
    # The same product left in f32: what the bf16 output is the rounding of.
    from ojas_amd.backend import F32
    y32 = be.linear_i8_group_forward(be.upload(x, BF16), be.upload(codes), be.upload(scales),
                                     be.upload(add, BF16) if with_add else None, out_dtype=F32)
    assert y32.dtype == F32
    assert np.array_equal(orc.round_bf16(be.download(y32)), be.download_f32(y))


@pytest.mark.parametrize("rows,kin,nout", [(256, 128, 64), (300, 96, 160), (77, 32, 32), (512, 256, 2048),
                                           (1024, 416, 256), (33, 160, 704)])
@pytest.mark.parametrize("with_add", [False, True])
def test_linear_i8_group_backward_input(be, rows, kin, nout, with_add):
    from ojas_amd.backend import BF16

    print(f"q8 input gradient rows={rows} kin={kin} nout={nout} add={with_add}", flush=True)
    rng = np.random.default_rng(rows * 5 + nout)
    gy = orc.round_bf16(rng.normal(0, 1, (rows, nout)).astype(np.float32))
    codes, scales = orc.quantize_i8_group(rng.normal(0, 0.05, (nout, kin)).astype(np.float32) *
                                          rng.uniform(0.2, 3.0, (nout, 1)).astype(np.float32), 32)
    add = orc.round_bf16(rng.normal(0, 0.3, (rows, kin)).astype(np.float32)) if with_add else None
    want = orc.linear_i8_group_backward_input(codes, scales, gy, 32) + (add if with_add else 0)
    gx = be.linear_i8_group_backward_input(be.upload(codes), be.upload(scales), be.upload(gy, BF16),
                                           be.upload(add, BF16) if with_add else None)
    _close(be.download_f32(gx), want)


def test_linear_i8_group_scale_per_group_is_exact(be):
    # One code per group set, powers of two as scales, a one-hot input: the product is exact in
    # bf16, so a scale taken from the wrong group or row, or a mis-signed code, shows bit for bit.
    from ojas_amd.backend import BF16

    nout, kin = 160, 128
    rng = np.random.default_rng(9)
    codes = rng.integers(-127, 128, (nout, kin)).astype(np.int8)
    codes[3, 5], codes[7, 64] = -127, 127
    scales = (2.0 ** rng.integers(-6, 3, (nout, kin // 32))).astype(np.float32)
    x = np.eye(kin, dtype=np.float32)  # row k picks column k of W
    y = be.download_f32(be.linear_i8_group_forward(be.upload(x, BF16), be.upload(codes), be.upload(scales)))
    want = orc.round_bf16(orc.dequant_i8_group(codes, scales, 32)).T
    assert np.array_equal(y, want)
    gy = np.eye(nout, dtype=np.float32)
    gx = be.download_f32(be.linear_i8_group_backward_input(be.upload(codes), be.upload(scales), be.upload(gy, BF16)))
    assert np.array_equal(gx, want.T)


@pytest.mark.parametrize("rows,kin,nout", [(300, 128, 104), (512, 2048, 256), (260, 384, 160)])
def test_blocked_layout_gives_the_same_products(be, rows, kin, nout):
    from ojas_amd.backend import BF16

    print(f"q8 blocked rows={rows} kin={kin} nout={nout}", flush=True)
    rng = np.random.default_rng(rows + kin + nout)
    x = be.upload(rng.normal(0, 1, (rows, kin)).astype(np.float32), BF16)
    gy = be.upload(rng.normal(0, 1, (rows, nout)).astype(np.float32), BF16)
    codes_h = rng.integers(-127, 128, (nout, kin)).astype(np.int8)
    scales_h = rng.uniform(1e-3, 2e-2, (nout, kin // 32)).astype(np.float32)
    codes, scales = be.upload(codes_h), be.upload(scales_h)
    bc, bs = be.pack_i8_group(codes, scales)
    # The blocked form is a permutation of the same bytes, spelled out here from its definition.
    r, c = np.meshgrid(np.arange(nout), np.arange(kin), indexing="ij")
    g = c // 32
    off = ((r // 8) * (kin // 128) + g // 4) * 1024 + (g % 4) * 256 + (r % 8) * 32 + c % 32
    want = np.empty(nout * kin, np.int8)
    want[off.reshape(-1)] = codes_h.reshape(-1)
    assert np.array_equal(be.download(bc).reshape(-1), want)
    rs, gs = np.meshgrid(np.arange(nout), np.arange(kin // 32), indexing="ij")
    soff = ((rs // 8) * (kin // 128) + gs // 4) * 32 + (gs % 4) * 8 + rs % 8
    swant = np.empty(scales_h.size, np.float32)
    swant[soff.reshape(-1)] = scales_h.reshape(-1)
    assert np.array_equal(be.download(bs).reshape(-1), swant)
    uc, us = be.unpack_i8_group(bc, bs)
    assert np.array_equal(be.download(uc), codes_h) and np.array_equal(be.download(us), scales_h)
    # Same arithmetic in the same order: bit-identical products.
    y0 = be.download(be.linear_i8_group_forward(x, codes, scales))
    y1 = be.download(be.linear_i8_group_forward(x, bc, bs, blocked=True))
    assert np.array_equal(y0, y1)
    if nout % 32 == 0:
        g0 = be.download(be.linear_i8_group_backward_input(codes, scales, gy))
        g1 = be.download(be.linear_i8_group_backward_input(bc, bs, gy, blocked=True))
        assert np.array_equal(g0, g1)


@pytest.mark.parametrize("rows,kin,nout,rank,blocks", [(300, 128, 256, 16, 1), (520, 256, 384, 16, 3),
                                                         (256, 64, 128, 48, 1)])
def test_low_rank_term_rides_in_the_accumulators(be, rows, kin, nout, rank, blocks):
    from ojas_amd.backend import BF16

    print(f"q8 low-rank rows={rows} kin={kin} nout={nout} rank={rank} blocks={blocks}", flush=True)
    rng = np.random.default_rng(rows + rank)
    bf = lambda a: orc.round_bf16(a.astype(np.float32))
    x = bf(rng.normal(0, 1, (rows, kin)))
    codes, scales = orc.quantize_i8_group(rng.normal(0, 0.05, (nout, kin)).astype(np.float32), 32)
    h = bf(rng.normal(0, 1, (rows, blocks * rank)))
    w = bf(rng.normal(0, 0.3, (nout, rank)))
    block_cols = nout // blocks
    want = orc.linear_i8_group_forward(x, codes, scales, 32)
    for j in range(blocks):
        cols = slice(j * block_cols, (j + 1) * block_cols)
        want[:, cols] += h[:, j * rank:(j + 1) * rank].astype(np.float64) @ w[cols].astype(np.float64).T
    y = be.linear_i8_group_forward(be.upload(x, BF16), be.upload(codes), be.upload(scales),
                                   low_rank=(be.upload(h, BF16), be.upload(w, BF16), block_cols if blocks > 1 else 0))
    _close(be.download_f32(y), want)
    # Input gradient: gx = gy W + gh A with A^T [kin, rank] as the term's second operand.
    gy = bf(rng.normal(0, 1, (rows, nout)))
    gh = bf(rng.normal(0, 1, (rows, rank)))
    at = bf(rng.normal(0, 0.3, (kin, rank)))
    if nout % 32 == 0:
        want = orc.linear_i8_group_backward_input(codes, scales, gy, 32) + gh.astype(np.float64) @ at.astype(np.float64).T
        gx = be.linear_i8_group_backward_input(be.upload(codes), be.upload(scales), be.upload(gy, BF16),
                                               low_rank=(be.upload(gh, BF16), be.upload(at, BF16), 0))
        _close(be.download_f32(gx), want)


def test_rope_in_place_and_swiglu(be):
    from ojas_amd.backend import BF16

    tokens, time, heads, dim, pitch = 48, 12, 6, 32, 6 * 32 + 64  # 4 query + 2 key heads, then 64 value columns
    rng = np.random.default_rng(21)
    x = orc.round_bf16(rng.normal(0, 1, (tokens, pitch)).astype(np.float32))
    cos, sin = orc.rope_tables(time, dim)
    rot = orc.rope_forward(np.ascontiguousarray(x[:, :heads * dim]).reshape(tokens // time, time, heads, dim), cos, sin)
    dx = be.upload(x, BF16)
    be.rope_half_split_inplace(dx, be.upload(cos), be.upload(sin), tokens, time, heads, dim)
    got = be.download_f32(dx)
    _close(got[:, :heads * dim], rot.reshape(tokens, heads * dim), 1e-2)
    assert np.array_equal(got[:, heads * dim:], x[:, heads * dim:])  # the value block is untouched
    # The backward is the inverse rotation: forward then backward returns the input (to bf16 rounding).
    be.rope_half_split_inplace(dx, be.upload(cos), be.upload(sin), tokens, time, heads, dim, backward=True)
    back = orc.rope_backward(rot, cos, sin).reshape(tokens, heads * dim)
    _close(be.download_f32(dx)[:, :heads * dim], back, 2e-2)
    # The rotation out of place from an f32 projection output: rotated heads and the value block in
    # one pass, one rounding each.
    from ojas_amd.backend import F32
    x32 = rng.normal(0, 1, (tokens, pitch)).astype(np.float32)
    rot32 = orc.rope_forward(np.ascontiguousarray(x32[:, :heads * dim]).reshape(tokens // time, time, heads, dim), cos, sin)
    for dtype, src in ((F32, x32), (BF16, x)):
        out = be.rope_half_split_pitched(be.upload(src, dtype), be.upload(cos), be.upload(sin), tokens, time, heads, 2, dim)
        got = be.download_f32(out)
        want = rot32 if dtype == F32 else rot
        _close(got[:, :heads * dim], want.reshape(tokens, heads * dim), 1e-2)
        assert np.array_equal(got[:, heads * dim:], orc.round_bf16(src[:, heads * dim:]))  # the value block: converted as it is
    # SwiGLU on a fused gate | up tensor.
    rows, hidden = 37, 72
    gu = orc.round_bf16(rng.normal(0, 1.5, (rows, 2 * hidden)).astype(np.float32))
    gm = orc.round_bf16(rng.normal(0, 1, (rows, hidden)).astype(np.float32))
    gate, up = np.ascontiguousarray(gu[:, :hidden]), np.ascontiguousarray(gu[:, hidden:])
    act = orc.silu_forward(gate)
    want = orc.mul_forward(act, up)
    dgu = be.upload(gu, BF16)
    _close(be.download_f32(be.swiglu_forward(dgu)), want)
    g_act, g_up = orc.mul_backward(act, up, gm)
    g_gate = orc.silu_backward(gate, g_act)
    got = be.download_f32(be.swiglu_backward(dgu, be.upload(gm, BF16)))
    _close(got[:, :hidden], g_gate)
    _close(got[:, hidden:], g_up)
    # The same on an unrounded f32 gate | up tensor (the projection's output kept in f32).
    from ojas_amd.backend import F32
    gu32 = rng.normal(0, 1.5, (rows, 2 * hidden)).astype(np.float32)
    gate, up = np.ascontiguousarray(gu32[:, :hidden]), np.ascontiguousarray(gu32[:, hidden:])
    act = orc.silu_forward(gate)
    dgu = be.upload(gu32, F32)
    out = be.swiglu_forward(dgu)
    assert out.dtype == BF16
    _close(be.download_f32(out), orc.mul_forward(act, up))
    g_act, g_up = orc.mul_backward(act, up, gm)
    got = be.download_f32(be.swiglu_backward(dgu, be.upload(gm, BF16)))
    _close(got[:, :hidden], orc.silu_backward(gate, g_act))
    _close(got[:, hidden:], g_up)


def test_linear_i8_group_refusals(be):
    from ojas_amd.backend import BF16, DTYPE, OUT_OF_RANGE, SHAPE, UNSUPPORTED, OjasError

    x = be.upload(np.zeros((8, 48), np.float32), BF16)
    codes = be.upload(np.zeros((32, 48), np.int8))
    scales = be.upload(np.zeros((32, 1), np.float32))
    with pytest.raises(OjasError) as e:  # k_in is not a multiple of the group
        be._check(be._lib.omx_linear_i8_group_forward(be._ctx, be._p(x), C.c_int32(1), be._p(codes), be._p(scales),
                                                      C.c_uint64(32), C.c_int32(0), None, None, be._p(x), C.c_int32(1), C.c_uint64(8), C.c_uint64(48),
                                                      C.c_uint64(32)))
    assert e.value.code == SHAPE
    with pytest.raises(OjasError) as e:
        be._check(be._lib.omx_linear_i8_group_forward(be._ctx, be._p(x), C.c_int32(1), be._p(codes), be._p(scales),
                                                      C.c_uint64(64), C.c_int32(0), None, None, be._p(x), C.c_int32(1), C.c_uint64(8), C.c_uint64(64),
                                                      C.c_uint64(32)))
    assert e.value.code == UNSUPPORTED
    with pytest.raises(OjasError) as e:
        be._check(be._lib.omx_linear_i8_group_forward(be._ctx, be._p(x), C.c_int32(0), be._p(codes), be._p(scales),
                                                      C.c_uint64(32), C.c_int32(0), None, None, be._p(x), C.c_int32(1), C.c_uint64(8), C.c_uint64(64),
                                                      C.c_uint64(32)))
    assert e.value.code == DTYPE
    # The kernel addresses a lane's bytes with 32 bits beside a 64-bit base: weights of 2 GiB or more and
    # k_in of 4 Mi or more are refused before anything is launched.
    for kin, nout in ((1 << 22, 32), (1 << 16, 1 << 15)):
        with pytest.raises(OjasError) as e:
            be._check(be._lib.omx_linear_i8_group_forward(be._ctx, be._p(x), C.c_int32(1), be._p(codes), be._p(scales),
                                                          C.c_uint64(32), C.c_int32(0), None, None, be._p(x), C.c_int32(1), C.c_uint64(8),
                                                          C.c_uint64(kin), C.c_uint64(nout)))
        assert e.value.code == OUT_OF_RANGE, (kin, nout)


# ---- the step: reduced shapes against the oracle ----
def _load_case(tr, cfg, frozen, quant):
    """Hands a seeded case (test_oracle_lora.make_lora_case) to the device trainer."""
    tr.set_embedding(frozen[0])
    for l in range(cfg.layers):
        base = 1 + 9 * l
        tr.set_norm(l, 0, frozen[base + 0])
        tr.set_norm(l, 1, frozen[base + 5])
        for which, idx in enumerate((1, 2, 3, 4, 6, 7, 8)):
            codes, scales = quant[base + idx]
            tr.set_matrix(l, which, codes, scales)
    tr.set_norm(cfg.layers, 0, frozen[-1])


# (layers, d, heads, head_dim, hidden, vocab, batch, seq, rank, scale)
LORA_STEP_SHAPES = [(2, 128, 2, 64, 256, 96, 2, 48, 16, 2.0), (1, 256, 2, 128, 384, 200, 1, 130, 16, 1.0),
                    (2, 128, 1, 128, 128, 64, 2, 64, 32, 0.5)]


@pytest.mark.parametrize("shape", LORA_STEP_SHAPES)
def test_lora_step_matches_the_oracle(be, shape):
    from test_oracle_lora import make_lora_case

    from ojas_amd.backend import AdamWConfig
    from ojas_amd.lora import LoraConfig, LoraTrainer

    print(f"lora step {shape}", flush=True)
    cfg = LoraConfig(*shape[:9], 1e-6, shape[9], 10000.0)
    ocfg = orc.LoraConfig(*shape[:9], 1e-6, shape[9], 10000.0)
    frozen, quant, adapters, ids, targets = make_lora_case(ocfg, 31 + shape[1])
    adapters = [orc.round_bf16(a) for a in adapters]  # bf16-exact operands on both sides
    tr = LoraTrainer(be, cfg)
    try:
        _load_case(tr, cfg, frozen, quant)
        tr.set_adapters(adapters)
        tr.set_batch(ids, targets)
        loss = tr.loss_and_grads()
        grads = tr.grads()
        oloss, ograds = orc.lora_loss_and_grads(ocfg, frozen, adapters, ids, targets)
        assert abs(loss - float(oloss)) <= 1e-3 * abs(float(oloss)), (loss, oloss)  # the bf16 tier's loss gate
        for i, (g, og) in enumerate(zip(grads, ograds)):
            scale = float(np.max(np.abs(og)))
            assert scale > 0, i
            err = float(np.max(np.abs(g - og)))
            assert err <= BF16_TOL * scale, (i, err / scale)
            assert np.linalg.norm(g - og) <= BF16_TOL * np.linalg.norm(og), i
        # One AdamW step moves every adapter element against its gradient's sign by about lr, and
        # nothing else: the update of an element with a solid gradient is lr to within 1 %.
        lr = 1e-3
        step_loss, norm = tr.step(AdamWConfig(lr, 0.9, 0.95, 1e-8, 0.0), 0.0)
        assert abs(step_loss - loss) <= 1e-6 * abs(loss)
        want_norm = float(np.sqrt(sum(float(np.sum(g.astype(np.float64) ** 2)) for g in grads)))
        assert abs(norm - want_norm) <= 1e-4 * want_norm
        after = tr.adapters()
        for a0, a1, g in zip(adapters, after, grads):
            solid = np.abs(g) > 1e-3 * np.max(np.abs(g))
            move = (a1 - a0.reshape(-1))[solid]
            assert np.all(np.abs(move + lr * np.sign(g[solid])) <= 1e-2 * lr + 4e-8 * np.abs(a0.reshape(-1)[solid]))
        assert tr.steps() == 1
    finally:
        tr.close()


def test_lora_adapter_starts_as_the_identity(be):
    # B = 0 (lora.rs:9-12): the loss is the base model's whatever A holds, dA is exactly zero and dB is not.
    from test_oracle_lora import make_lora_case

    from ojas_amd.lora import LoraConfig, LoraTrainer

    shape = (2, 128, 2, 64, 256, 96, 2, 48, 16)
    cfg = LoraConfig(*shape, 1e-6, 2.0, 10000.0)
    ocfg = orc.LoraConfig(*shape, 1e-6, 2.0, 10000.0)
    frozen, quant, adapters, ids, targets = make_lora_case(ocfg, 5)
    zero_b = [orc.round_bf16(a) if i % 2 == 0 else np.zeros_like(a) for i, a in enumerate(adapters)]
    tr = LoraTrainer(be, cfg)
    try:
        _load_case(tr, cfg, frozen, quant)
        tr.set_batch(ids, targets)
        tr.set_adapters(zero_b)
        loss0 = tr.loss_and_grads()
        grads = tr.grads()
        assert all(not np.any(g) for g in grads[0::2]) and all(np.any(g) for g in grads[1::2])
        tr.set_adapters([2 * a if i % 2 == 0 else a for i, a in enumerate(zero_b)])
        assert tr.loss_and_grads() == loss0
    finally:
        tr.close()
