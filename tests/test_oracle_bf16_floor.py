"""The nanolab oracle with bf16 roundings placed as a bf16 tier places them
(`orc_nanolab_loss_and_grads_rounded`, oracle/nanolab_exact.cpp): the modes themselves, and the
distance they put between a bf16 tier and the Exact result.

Every operation stays Exact f32 arithmetic; only where values are rounded to bf16 changes:
ROUND_OPERANDS rounds what a matrix product reads and nothing else (`prep`,
ojas-core/src/autocast.rs:518-525), ROUND_AUTOCAST every point the reference's own bf16 tier rounds
(`emit` :533-538 and `promote` :540-546 as well). The first is the least rounding any tier whose
products take bf16 operands can do, so its distance from the Exact gradients is a floor under such
a tier's; the GPU tests hold the device's bf16 tier to that floor where it lies above 2e-2."""
import numpy as np
import pytest

import oracle_api as orc


def model(layers, d, heads, head_dim, hidden, vocab, seq, seed):
    cfg = orc.NanolabConfig(layers=layers, n_embd=d, n_head=heads, n_kv_head=heads, head_dim=head_dim, hidden=hidden,
                            vocab=vocab, batch=1, seq=seq, window=0, rms_eps=1e-6, rope_base=10000.0)
    rng = np.random.default_rng(seed)
    params, matrix = [], []
    lens = orc.nanolab_param_lens(cfg)
    for i, n in enumerate(lens):
        which = None if i in (0, len(lens) - 1) else (i - 1) % 14
        if i == 0 or which in (1, 2, 3, 4, 7, 11, 12, 13):  # the table and the matrices: bf16-exact N(0, 0.02)
            params.append(orc.round_bf16(rng.normal(0, 0.02, n).astype(np.float32)))
        elif which == 8:
            params.append(rng.normal(0, 0.5, n).astype(np.float32))
        elif which == 9:
            params.append(rng.uniform(0.2, 0.8, n).astype(np.float32))
        else:
            params.append(np.ones(n, np.float32))
        matrix.append(i == 0 or which in (1, 2, 3, 4, 7, 11, 12, 13))
    window = rng.integers(0, vocab, seq + 1).astype(np.uint32)
    return cfg, params, window[:-1].copy(), window[1:].copy(), matrix


def worst_matrix_distance(grads, exact, matrix):
    pairs = [(g.astype(np.float64), e.astype(np.float64)) for g, e, m in zip(grads, exact, matrix) if m]
    return max(float(np.linalg.norm(g - e) / np.linalg.norm(e)) for g, e in pairs)


def test_no_rounding_is_the_exact_graph_bit_for_bit_and_unknown_modes_are_refused():
    cfg, params, ids, targets, _ = model(2, 64, 2, 32, 96, 80, 24, 1)
    loss, _, grads = orc.nanolab_loss_and_grads(cfg, params, ids, targets)
    loss0, grads0 = orc.nanolab_loss_and_grads_rounded(cfg, params, ids, targets, 0)
    assert loss0.tobytes() == loss.tobytes()
    assert all(a.tobytes() == b.tobytes() for a, b in zip(grads0, grads))
    with pytest.raises(orc.OracleError):
        orc.nanolab_loss_and_grads_rounded(cfg, params, ids, targets, 3)


def test_without_blocks_the_one_rounded_operand_is_the_head_input():
    """A model of no blocks is embedding, norm, tied head: the only product operand that is not a
    parameter is the norm's output. Rounding it by hand and calling the Exact head gives the bits
    of both rounded modes (the emitted gradient of the head's input has no reader that rounds it
    again before the norm's backward, which Autocast leaves in f32)."""
    cfg, params, ids, targets, _ = model(0, 64, 2, 32, 96, 80, 24, 2)
    table, norm_w = params
    x = orc.embedding_forward(table.reshape(80, 64), ids)
    hf = orc.round_bf16(orc.rms_norm_forward(x, norm_w))
    want_loss, ghf, g_head = orc.linear_cross_entropy_mean(hf, table.reshape(80, 64), targets)
    for mode in (orc.ROUND_OPERANDS,):
        loss, grads = orc.nanolab_loss_and_grads_rounded(cfg, params, ids, targets, mode)
        assert loss.tobytes() == np.float32(want_loss).tobytes()
        gx, g_norm = orc.rms_norm_backward(x, norm_w, ghf)
        assert grads[1].tobytes() == g_norm.astype(np.float32).tobytes()
    exact_loss, _, exact = orc.nanolab_loss_and_grads(cfg, params, ids, targets)
    assert exact_loss != loss and not np.array_equal(exact[1], grads[1])  # the rounding is really applied


def test_the_floor_under_a_bf16_tier_grows_with_depth_and_passes_2e_2_at_twelve_blocks():
    """At the nanolab-124M width (768, 12 heads of 64, SwiGLU 2048) the distance of the
    operands-only run from the Exact gradients is about 1e-2 per sqrt(block): past 2e-2 well before
    twelve blocks, and the reference's own rounding points lie above it at every depth."""
    orc.set_threads(8)
    floors = {}
    for layers in (2, 12):
        cfg, params, ids, targets, matrix = model(layers, 768, 12, 64, 2048, 512, 64, 7)
        _, _, exact = orc.nanolab_loss_and_grads(cfg, params, ids, targets)
        _, operands = orc.nanolab_loss_and_grads_rounded(cfg, params, ids, targets, orc.ROUND_OPERANDS)
        _, autocast = orc.nanolab_loss_and_grads_rounded(cfg, params, ids, targets, orc.ROUND_AUTOCAST)
        floors[layers] = (worst_matrix_distance(operands, exact, matrix), worst_matrix_distance(autocast, exact, matrix))
    print("operands-only / autocast distance:", floors)
    assert floors[2][0] < 2e-2 < 2.5e-2 < floors[12][0] < 5e-2
    assert floors[2][0] < floors[2][1] and floors[12][0] < floors[12][1]
