"""An independent float64 torch statement of the GPT-2-shaped graph, used only
to pin the oracle's composed step (which no reference fixture covers)."""
import numpy as np
import torch
import torch.nn.functional as F


def param_shapes(cfg):
    d, mlp = cfg["d_model"], cfg["mlp"]
    shapes = [(cfg["vocab"], d), (cfg["ctx"], d)]
    for _ in range(cfg["layers"]):
        shapes += [(d,), (d, d), (d, d), (d, d), (d, d), (d,), (mlp, d), (d, mlp)]
    shapes.append((d,))
    return shapes


def rms(x, w, eps=1e-6):
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w


def loss_and_grads(cfg, params, ids, targets):
    ps = [torch.tensor(np.asarray(p, np.float64).reshape(s), requires_grad=True)
          for p, s in zip(params, param_shapes(cfg))]
    B, T, H, D = cfg["batch"], cfg["ctx"], cfg["heads"], cfg["head_dim"]
    ids_t = torch.tensor(ids.astype(np.int64)).reshape(B, T)
    x = ps[0][ids_t] + ps[1][torch.arange(T)][None]
    for l in range(cfg["layers"]):
        n1, wq, wk, wv, wo, n2, w1, w2 = ps[2 + 8 * l: 10 + 8 * l]
        h = rms(x, n1)
        q = (h @ wq.T).reshape(B, T, H, D).transpose(1, 2)
        k = (h @ wk.T).reshape(B, T, H, D).transpose(1, 2)
        v = (h @ wv.T).reshape(B, T, H, D).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + a.transpose(1, 2).reshape(B, T, H * D) @ wo.T
        h = rms(x, n2)
        u = h @ w1.T
        g = F.gelu(u, approximate="tanh" if cfg.get("gelu_tanh") else "none")
        x = x + g @ w2.T
    logits = rms(x, ps[-1]) @ ps[0].T
    loss = F.cross_entropy(logits.reshape(B * T, -1), torch.tensor(targets.astype(np.int64)).reshape(-1))
    loss.backward()
    return float(loss), [p.grad.numpy().reshape(-1) for p in ps]
