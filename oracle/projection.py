"""CPU restatement of the projections around the attention core. Test infrastructure only.

Follows ``DistributedAttention.forward`` (jigsaw/modules/attention/_attention.py:881-918):
``qkv = self.qkv(x)``, ``rearrange(qkv, "... n s (three h d) -> three ... n h s d")``, and
after the core ``rearrange(out, "... n h s d -> ... n s (h d)")`` + ``self.head_concat(out)``.
The rearranges are written as explicit index loops on purpose (not einops), so that the
tests pin them against torch's own reshape / permute.
"""

from __future__ import annotations

import torch


def qkv_forward(x, weight, bias, heads):
    """``(*lead, s, C) -> (3, *lead, h, s, d)`` — _attention.py:881-890."""
    lead, s = tuple(x.shape[:-2]), x.shape[-2]
    qkv = x.reshape(-1, s, x.shape[-1]) @ weight.t()
    if bias is not None:
        qkv = qkv + bias
    d = weight.shape[0] // (3 * heads)
    out = torch.empty(3, qkv.shape[0], heads, s, d, dtype=qkv.dtype)
    for t in range(3):
        for h in range(heads):
            f0 = (t * heads + h) * d  # feature index "(three h d)": three slowest, d fastest
            out[t, :, h] = qkv[:, :, f0:f0 + d]
    return out.reshape(3, *lead, heads, s, d)


def heads_forward(out, weight, bias):
    """``(*lead, h, s, d) -> (*lead, s, n_out)`` — _attention.py:909-916."""
    lead = tuple(out.shape[:-3])
    h, s, d = out.shape[-3:]
    o = out.reshape(-1, h, s, d)
    flat = torch.empty(o.shape[0], s, h * d, dtype=out.dtype)
    for i in range(h):
        flat[:, :, i * d:(i + 1) * d] = o[:, i]  # "(h d)": head slowest
    y = flat @ weight.t()
    if bias is not None:
        y = y + bias
    return y.reshape(*lead, s, weight.shape[0])


def qkv_backward(grad, x, weight, heads):
    """``(gx, gw, gb)`` of :func:`qkv_forward` from ``grad (3, *lead, h, s, d)``."""
    s, c = x.shape[-2], x.shape[-1]
    d = weight.shape[0] // (3 * heads)
    g = grad.reshape(3, -1, heads, s, d)
    flat = torch.empty(g.shape[1], s, 3 * heads * d, dtype=grad.dtype)
    for t in range(3):
        for h in range(heads):
            f0 = (t * heads + h) * d
            flat[:, :, f0:f0 + d] = g[t, :, h]
    g2, x2 = flat.reshape(-1, 3 * heads * d), x.reshape(-1, c)
    return (g2 @ weight).reshape(x.shape), g2.t() @ x2, g2.sum(dim=0)


def heads_backward(grad, out, weight):
    """``(g_out, gw, gb)`` of :func:`heads_forward` from ``grad (*lead, s, n_out)``."""
    h, s, d = out.shape[-3:]
    o = out.reshape(-1, h, s, d)
    flat = torch.empty(o.shape[0], s, h * d, dtype=out.dtype)
    for i in range(h):
        flat[:, :, i * d:(i + 1) * d] = o[:, i]
    g2 = grad.reshape(-1, weight.shape[0])
    gflat = (g2 @ weight).reshape(o.shape[0], s, h * d)
    go = torch.empty_like(o)
    for i in range(h):
        go[:, i] = gflat[:, :, i * d:(i + 1) * d]
    return go.reshape(out.shape), g2.t() @ flat.reshape(-1, h * d), g2.sum(dim=0)
