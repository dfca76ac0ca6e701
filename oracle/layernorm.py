"""Oracle for the sharded LayerNorm: all shards of the channel group are
simulated in one process, all-reduces become means / sums over the list. Test
infrastructure only."""

from __future__ import annotations

import torch


def forward(x_shards, w_shards, b_shards, eps):
    """``(y, x_norm, std)`` per shard.

    Follows _LayerNorm.forward, jigsaw/modules/normalization/_functional.py:46-59:
    local mean and biased variance (:46-47); mean = AVG over shards (:49-50);
    var = AVG(local_var + (local_mean - mean)^2) (:52-53); x_norm, affine (:55-58).
    ``std = sqrt(var + eps)`` is what setup_context saves (:75).
    """
    local_mean = [x.mean(dim=-1, keepdim=True) for x in x_shards]
    local_var = [x.var(dim=-1, keepdim=True, unbiased=False) for x in x_shards]
    mean = torch.stack(local_mean).mean(0)
    var = torch.stack([lv + (lm - mean) ** 2 for lv, lm in zip(local_var, local_mean)]).mean(0)
    ys, xns = [], []
    for x, w, b in zip(x_shards, w_shards, b_shards):
        x_norm = (x - mean) / torch.sqrt(var + eps)
        ys.append(w * x_norm + (b if b is not None else 0))
        xns.append(x_norm)
    return ys, xns, torch.sqrt(var + eps)


def partial_stats(x):
    """Local mean and biased variance of one shard (_functional.py:46-47)."""
    return x.mean(dim=-1, keepdim=True), x.var(dim=-1, keepdim=True, unbiased=False)


def backward(g_shards, xn_shards, w_shards, std, has_bias=True):
    """``(gx, gw, gb)`` per shard.

    Follows _LayerNorm.backward, jigsaw/modules/normalization/_functional.py:141-175:
    n = local width * group size (:141-143); gw = sum(g * x_norm), gb = sum(g) over
    the leading dims (:150-155); grad_x_norm = g * w (:158); its row mean is
    AVG-reduced (:160-163), sum(grad_x_norm * x_norm) is SUM-reduced (:165-168);
    gx = (1/std) * (gxn - mean - x_norm * sum / n) (:173-175).
    """
    G = len(g_shards)
    n = xn_shards[0].shape[-1] * G
    gxn = [g * w for g, w in zip(g_shards, w_shards)]
    mean_term = torch.stack([t.mean(dim=-1, keepdim=True) for t in gxn]).mean(0)
    sum_term = torch.stack([(t * xn).sum(dim=-1, keepdim=True) for t, xn in zip(gxn, xn_shards)]).sum(0)
    gxs, gws, gbs = [], [], []
    for g, xn, t, w in zip(g_shards, xn_shards, gxn, w_shards):
        gws.append((g * xn).sum_to_size(w.shape))
        gbs.append(g.sum_to_size(w.shape) if has_bias else None)
        gxs.append((1.0 / std) * (t - mean_term - xn * sum_term / n))
    return gxs, gws, gbs
