"""One rank's share of a Swin block on the GPU kernels of this package.

Mirrors the example model of the reference (examples/swin.py:64-210): tokens are
channels-last ``(B, h, w, C)`` tiles of a 2-D token grid; a block is
``x + unshift(attn(shift(norm1(x))))`` followed by ``x + mlp(norm2(x))``. The
LayerNorms (not sharded in the example) run on the fused unsharded-LayerNorm kernels,
the shift / unshift on the DistributedRoll kernels, the windowed attention with its
relative-position bias and shift mask on the attention core with an additive
bias. The linear layers are ``nn.Linear`` parameters (as in the reference example);
in bf16 they run on this package's projection GEMMs (head split / merge and bias
gradient fused in), otherwise through the library GEMMs with the weight gradient split
over the tokens, because its output is a few tiles and its contraction 65536 long.
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch
import torch.nn as nn

from .attention import window_attention
from .conv import TileGroup
from .layernorm import plain_layer_norm
from .projection import heads_projection, linear, qkv_projection
from .roll import _Roll


class _TokenLinear(torch.autograd.Function):
    """``F.linear`` over ``(tokens, features)`` whose weight gradient is a batched GEMM
    over chunks of the tokens, summed in fp32. ``dW = dy^T x`` has an output of only
    ``out x in`` (a handful of GEMM tiles) and a contraction as long as the token count,
    so a single library GEMM runs on a few compute units; the chunks spread it over the
    chip. Same arithmetic as ``nn.Linear`` otherwise (examples/swin.py:136-170, 183-190)."""

    CHUNK = 1024  # tokens per partial product

    @staticmethod
    def forward(ctx, x, weight, bias):  # noqa: D102
        ctx.dtypes = (x.dtype, weight.dtype, bias.dtype if bias is not None else None)
        if torch.is_autocast_enabled():
            dt = torch.get_autocast_dtype("cuda")
            x, weight = x.to(dt), weight.to(dt)
            bias = bias.to(dt) if bias is not None else None
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, gy):  # noqa: D102
        x, weight = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad
        gy2 = gy.reshape(-1, gy.shape[-1])
        x2 = x.reshape(-1, x.shape[-1])
        dt_x, dt_w, dt_b = ctx.dtypes
        gy2 = gy2.to(weight.dtype)
        gx = (gy2 @ weight).view(x.shape).to(dt_x) if need_x else None
        gw = None
        if need_w:
            t = x2.shape[0]
            chunk = _TokenLinear.CHUNK
            if t % chunk == 0 and t // chunk > 1:
                parts = torch.bmm(gy2.view(t // chunk, chunk, -1).transpose(1, 2), x2.view(t // chunk, chunk, -1))
                gw = parts.sum(0, dtype=torch.float32).to(dt_w)
            else:
                gw = (gy2.t() @ x2).to(dt_w)
        gb = gy2.sum(0, dtype=torch.float32).to(dt_b) if need_b and ctx.has_bias else None
        return gx, gw, gb


def _compute_dtype(x: torch.Tensor) -> torch.dtype:
    """The dtype a linear layer computes in: the autocast dtype when autocast is on."""
    return torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else x.dtype


def token_linear(x: torch.Tensor, layer: nn.Linear) -> torch.Tensor:
    """``layer(x)``: in bf16 on this package's GEMM kernels (bias gradient fused into the weight
    gradient), otherwise through the library GEMM with the token-split weight gradient."""
    if x.is_cuda and _compute_dtype(x) == torch.bfloat16 and x.shape[-1] % 8 == 0 and layer.weight.shape[0] % 8 == 0:
        return linear(x.to(torch.bfloat16), layer.weight, layer.bias)
    return _TokenLinear.apply(x, layer.weight, layer.bias)


def windows(x: torch.Tensor, window: int) -> torch.Tensor:
    """Cut a tile ``(B, h, w, C)`` into windows ``(B, nW, window*window, C)``
    (examples/swin.py:85-89)."""
    b, h, w, c = x.shape
    x = x.view(b, h // window, window, w // window, window, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, -1, window * window, c)


def unwindows(x: torch.Tensor, h: int, w: int, window: int) -> torch.Tensor:
    """Inverse of :func:`windows` (examples/swin.py:92-96)."""
    b, c = x.shape[0], x.shape[-1]
    x = x.view(b, h // window, w // window, window, window, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, h, w, c)


def relative_position_index(window: int) -> torch.Tensor:
    """Index into the bias table for every pair of positions inside a window
    (examples/swin.py:99-104)."""
    ij = torch.stack(torch.meshgrid(*[torch.arange(window)] * 2, indexing="ij")).flatten(1)
    rel = ij[:, :, None] - ij[:, None, :] + (window - 1)
    return rel[0] * (2 * window - 1) + rel[1]


def shift_mask(h: int, w: int, window: int, shift: int, groups: tuple) -> torch.Tensor:
    """Mask ``(nW, N, N)`` of this tile's windows after rolling the token grid by
    ``-shift``: tokens from the two sides of the image border must not attend to
    each other; the border lies at the GLOBAL position, so the region of a token
    follows from where the tile sits (examples/swin.py:107-126)."""

    def region(local_size: int, group: Any) -> torch.Tensor:
        size = local_size * group.size()
        idx = group.rank() * local_size + torch.arange(local_size)
        return (idx >= size - window).long() + (idx >= size - shift).long()

    rows, cols = region(h, groups[0]), region(w, groups[1])
    ids = (rows[:, None] * 3 + cols[None, :])[None, :, :, None]
    ids = windows(ids, window).squeeze(-1).squeeze(0)
    same = ids[:, :, None] == ids[:, None, :]
    return torch.zeros(same.shape).masked_fill(~same, float("-inf"))


class WindowAttention(nn.Module):
    """Multi-head attention inside windows with a learned relative-position bias
    (examples/swin.py:129-170); the attention core is this package's kernel."""

    def __init__(self, dim: int, heads: int, window: int, tile: tuple, shift: int, groups: tuple, device) -> None:
        super().__init__()
        self.heads, self.window = heads, window
        self.qkv = nn.Linear(dim, 3 * dim, device=device)
        self.proj = nn.Linear(dim, dim, device=device)
        self.bias_table = nn.Parameter(torch.zeros((2 * window - 1) ** 2, heads, device=device))
        nn.init.trunc_normal_(self.bias_table, std=0.02)
        self.register_buffer("index", relative_position_index(window).to(device), persistent=False)
        # The gather bias_table[index] as a product with a one-hot matrix (N*N, table rows): the same
        # numbers (1 * v plus zeros), and its backward is a small GEMM instead of a sorted scatter-add.
        onehot = torch.nn.functional.one_hot(self.index.view(-1), (2 * window - 1) ** 2).to(torch.float32)
        self.register_buffer("onehot", onehot, persistent=False)
        if shift:
            self.register_buffer("mask", shift_mask(*tile, window, shift, groups).to(device), persistent=False)
        else:
            self.mask = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        b, h, w, c = x.shape
        x = windows(x, self.window)
        n = x.shape[2]
        fused = x.dtype == torch.bfloat16  # the projections write / read the head layout themselves
        if fused:
            q, k, v = qkv_projection(x, self.qkv.weight, self.qkv.bias, self.heads).unbind(0)
        else:
            qkv = token_linear(x, self.qkv).view(b, -1, n, 3, self.heads, c // self.heads)
            q, k, v = (t.contiguous() for t in qkv.permute(3, 0, 1, 4, 2, 5).unbind(0))  # (B, nW, heads, N, d)
        with torch.autocast("cuda", enabled=False):
            bias = (self.onehot @ self.bias_table.float()).view(n, n, -1).permute(2, 0, 1)
        if self.mask is not None:
            bias = bias[None] + self.mask[:, None]  # (nW, heads, N, N)
        out = window_attention(q, k, v, bias.contiguous())
        if fused:
            return unwindows(heads_projection(out, self.proj.weight, self.proj.bias), h, w, self.window)
        out = out.transpose(2, 3).reshape(b, -1, n, c)
        return unwindows(token_linear(out, self.proj), h, w, self.window)


class SwinBlock(nn.Module):
    """``x + attn(norm(x))`` then ``x + mlp(norm(x))``; the windows may be shifted
    (examples/swin.py:173-210). ``groups`` are the two spatial groups of the tile
    (objects with ``size()`` / ``rank()``), ``comm_halo_1d_fn`` the 1-D exchange the
    roll uses (``RollConfig.comm_halo_1d_fn`` in the reference)."""

    def __init__(self, dim: int, heads: int, window: int, tile: tuple, groups: tuple = None,
                 comm_halo_1d_fn: Callable | None = None, shift: int = 0, device=None, eps: float = 1e-5) -> None:
        super().__init__()
        groups = groups or (TileGroup(1, 0), TileGroup(1, 0))
        self.groups, self.comm, self.shift_by, self.eps = groups, comm_halo_1d_fn, shift, eps
        self.norm1 = nn.LayerNorm(dim, eps=eps, device=device)
        self.attn = WindowAttention(dim, heads, window, tile, shift, groups, device)
        self.norm2 = nn.LayerNorm(dim, eps=eps, device=device)
        self.mlp = nn.Sequential(nn.Linear(dim, 4 * dim, device=device), nn.GELU(), nn.Linear(4 * dim, dim, device=device))

    def _roll(self, x: torch.Tensor, shift: int) -> torch.Tensor:
        if not shift:
            return x
        dist_dims = tuple(d for d, g in zip((1, 2), self.groups) if g.size() > 1)
        dist_groups = tuple(g for g in self.groups if g.size() > 1)
        return _Roll.apply(x.contiguous(), (shift, shift), (1, 2), dist_dims, dist_groups, self.comm)

    def _norm(self, ln: nn.LayerNorm, x: torch.Tensor) -> torch.Tensor:
        # Both LayerNorms feed a linear layer (through pure copies), which under autocast rounds
        # its input to the autocast dtype: asking for that dtype here gives the same numbers
        # without the fp32 tensor in between.
        return plain_layer_norm(x, ln.weight, ln.bias, self.eps, out_dtype=_compute_dtype(x))

    # The block in stages, so that a single-process harness can run several ranks
    # in lockstep (the two rolls are the only stages that talk to other ranks).
    def pre_attention(self, x: torch.Tensor) -> torch.Tensor:
        return self._norm(self.norm1, x)

    def shift(self, y: torch.Tensor) -> torch.Tensor:
        return self._roll(y, -self.shift_by)

    def unshift(self, y: torch.Tensor) -> torch.Tensor:
        return self._roll(y, self.shift_by)

    def finish(self, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        x = x + y.to(x.dtype)
        y = token_linear(self._norm(self.norm2, x), self.mlp[0])
        return x + token_linear(self.mlp[1](y), self.mlp[2])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = self.unshift(self.attn(self.shift(self.pre_attention(x))))
        return self.finish(x, y)


__all__ = ["SwinBlock", "WindowAttention", "relative_position_index", "shift_mask", "unwindows", "windows"]
