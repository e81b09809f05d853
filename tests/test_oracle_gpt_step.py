"""The oracle's composed GPT step against an independent float64 torch autograd
statement of the same graph. No reference fixture holds this graph (the
reference ships the nanolab block, not the GPT-2-shaped one), so this is the
pin: a dropped term, wrong sign, transposed operand or mis-ordered permute in
the oracle's forward or hand-written backward fails it."""
import numpy as np
import pytest

import oracle_api as orc
from gpt_reference_torch import loss_and_grads, param_shapes

CFG = dict(layers=2, d_model=32, heads=2, head_dim=16, mlp=64, ctx=16, vocab=50, batch=2)


def make_inputs(cfg, seed):
    r = orc.SplitMix64(seed)
    params = []
    for s in param_shapes(cfg):
        n = int(np.prod(s))
        params.append((np.float32(1.0) + r.vec(n, 0.1)) if len(s) == 1 else r.vec(n, 0.2))
    n_tok = cfg["batch"] * cfg["ctx"]
    ids = np.array([r.below(cfg["vocab"]) for _ in range(n_tok)], np.uint32)
    targets = np.array([r.below(cfg["vocab"]) for _ in range(n_tok)], np.uint32)
    return params, ids, targets


@pytest.mark.parametrize("gelu_tanh", [0, 1])
def test_oracle_gpt_step_matches_torch_f64_autograd(gelu_tanh):
    cfg = dict(CFG, gelu_tanh=gelu_tanh)
    params, ids, targets = make_inputs(cfg, 1234)
    c = orc.GptConfig(cfg["layers"], cfg["d_model"], cfg["heads"], cfg["head_dim"], cfg["mlp"], cfg["ctx"],
                      cfg["vocab"], cfg["batch"], gelu_tanh)
    assert orc.gpt_param_lens(c) == [int(np.prod(s)) for s in param_shapes(cfg)]
    loss, grads = orc.gpt_loss_and_grads(c, params, ids, targets)
    tloss, tgrads = loss_and_grads(cfg, params, ids, targets)
    assert abs(float(loss) - tloss) <= 1e-5 * abs(tloss)
    for i, (g, tg) in enumerate(zip(grads, tgrads)):
        err = np.max(np.abs(g.astype(np.float64) - tg))
        assert err <= 1e-4 * max(np.max(np.abs(tg)), 1e-6), (i, err, np.max(np.abs(tg)))
