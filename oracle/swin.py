"""Oracle for the Swin block of the reference's example: the block on an UNDIVIDED
token grid in plain torch (mesh 1x1: the roll is ``torch.roll``, the shift mask is
built from global positions). Test infrastructure only."""

from __future__ import annotations

import torch
import torch.nn.functional as F


def windows(x, window):
    """examples/swin.py:85-89."""
    b, h, w, c = x.shape
    x = x.view(b, h // window, window, w // window, window, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, -1, window * window, c)


def unwindows(x, h, w, window):
    """examples/swin.py:92-96."""
    b, c = x.shape[0], x.shape[-1]
    x = x.view(b, h // window, w // window, window, window, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, h, w, c)


def relative_position_index(window):
    """examples/swin.py:99-104."""
    ij = torch.stack(torch.meshgrid(*[torch.arange(window)] * 2, indexing="ij")).flatten(1)
    rel = ij[:, :, None] - ij[:, None, :] + (window - 1)
    return rel[0] * (2 * window - 1) + rel[1]


def shift_mask_global(h, w, window, shift):
    """examples/swin.py:107-126 for a tile that is the whole grid (group size 1)."""

    def region(size):
        idx = torch.arange(size)
        return (idx >= size - window).long() + (idx >= size - shift).long()

    ids = (region(h)[:, None] * 3 + region(w)[None, :])[None, :, :, None]
    ids = windows(ids, window).squeeze(-1).squeeze(0)
    same = ids[:, :, None] == ids[:, None, :]
    return torch.zeros(same.shape, dtype=torch.float64).masked_fill(~same, float("-inf"))


def block(x, p, heads, window, shift, eps=1e-5):
    """One Swin block on the undivided ``(B, H, W, C)`` grid (examples/swin.py:129-210).
    ``p`` maps parameter names of jigsaw_amd.swin.SwinBlock's state dict to tensors."""
    b, h, w, c = x.shape
    n = window * window
    y = F.layer_norm(x, (c,), p["norm1.weight"], p["norm1.bias"], eps)
    if shift:
        y = torch.roll(y, (-shift, -shift), (1, 2))
    t = windows(y, window)
    qkv = F.linear(t, p["attn.qkv.weight"], p["attn.qkv.bias"]).view(b, -1, n, 3, heads, c // heads)
    q, k, v = qkv.permute(3, 0, 1, 4, 2, 5).unbind(0)
    index = relative_position_index(window)
    bias = p["attn.bias_table"][index.view(-1)].view(n, n, -1).permute(2, 0, 1)
    if shift:
        bias = bias[None] + shift_mask_global(h, w, window, shift).to(bias.dtype)[:, None]
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=bias)
    out = out.transpose(2, 3).reshape(b, -1, n, c)
    y = unwindows(F.linear(out, p["attn.proj.weight"], p["attn.proj.bias"]), h, w, window)
    if shift:
        y = torch.roll(y, (shift, shift), (1, 2))
    x = x + y
    z = F.layer_norm(x, (c,), p["norm2.weight"], p["norm2.bias"], eps)
    z = F.linear(F.gelu(F.linear(z, p["mlp.0.weight"], p["mlp.0.bias"])), p["mlp.2.weight"], p["mlp.2.bias"])
    return x + z
