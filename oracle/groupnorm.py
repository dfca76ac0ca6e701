"""CPU restatement of the spatially sharded GroupNorm. Test infrastructure only.

Follows ``_GroupNorm`` (jigsaw/modules/normalization/_functional.py:317-468): the
shards of one spatial split are passed as a list and the all-reduces are the sums
over that list.
"""

from __future__ import annotations

import torch


def forward(shards, num_groups, weight, bias, eps):
    """Per shard ``(y, x_norm)`` plus the shared ``(rstd, n)`` — _functional.py:352-385."""
    xg = [x.reshape(x.shape[0], num_groups, -1) for x in shards]
    # global count and sum per (sample, group): the (count, sum) all-reduce (:356-360)
    n = sum(torch.full_like(t[..., 0], t.shape[-1]) for t in xg)
    total = sum(t.sum(dim=-1) for t in xg)
    mean = (total / n).unsqueeze(-1)
    # centred on the global mean before squaring, then the second all-reduce (:363-366)
    var = sum(((t - mean) ** 2).sum(dim=-1, keepdim=True) for t in xg)
    n = n.unsqueeze(-1)
    rstd = torch.rsqrt(var / n + eps)
    outs = []
    for x, t in zip(shards, xg):
        x_norm = ((t - mean) * rstd).reshape(x.shape)
        shape = (1, -1) + (1,) * (x.dim() - 2)
        y = x_norm
        if weight is not None:
            y = y * weight.reshape(shape)
        if bias is not None:
            y = y + bias.reshape(shape)
        outs.append((y, x_norm))
    return outs, rstd, n


def backward(grads, x_norms, rstd, n, num_groups, weight):
    """Per shard ``(gx, gw, gb)``; gw / gb are the shard's local sums — _functional.py:431-468."""
    shape = (x_norms[0].shape[0], num_groups, -1)
    ggs = []
    for g in grads:
        gxn = g if weight is None else g * weight.reshape((1, -1) + (1,) * (g.dim() - 2))
        ggs.append(gxn.reshape(shape))
    xgs = [t.reshape(shape) for t in x_norms]
    # both per-group reductions, summed over the shards (:458-460)
    g_sum = sum(t.sum(dim=-1) for t in ggs).unsqueeze(-1)
    gx_sum = sum((a * b).sum(dim=-1) for a, b in zip(ggs, xgs)).unsqueeze(-1)
    outs = []
    for g, gg, xg, xn in zip(grads, ggs, xgs, x_norms):
        gx = (rstd * (gg - g_sum / n - xg * gx_sum / n)).reshape(xn.shape)
        dims = (0, *range(2, g.dim()))
        outs.append((gx, (g * xn).sum(dim=dims), g.sum(dim=dims)))
    return outs
