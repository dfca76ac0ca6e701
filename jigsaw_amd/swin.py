"""One rank's share of a Swin block on the GPU kernels of this package.

Mirrors the example model of the reference (examples/swin.py:64-210): tokens are
channels-last ``(B, h, w, C)`` tiles of a 2-D token grid; a block is
``x + unshift(attn(shift(norm1(x))))`` followed by ``x + mlp(norm2(x))``. The
LayerNorms (not sharded in the example) run on the fused unsharded-LayerNorm kernels,
the shift / unshift on the DistributedRoll kernels, the windowed attention with its
relative-position bias and shift mask on the attention core with an additive
bias. The linear layers are ``nn.Linear`` parameters (as in the reference example);
they run on this package's projection GEMMs (head split / merge and bias gradient fused
in): bf16 on the matrix cores, other dtypes on the FMA kernel with the same addressing.
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch
import torch.nn as nn

from . import _lib
from .attention import _SwinGridAttention, swin_grid_attention_packed, window_attention
from .conv import TileGroup
from .layernorm import _PlainLayerNormFork, plain_layer_norm, plain_layer_norm_fork
from .projection import (
    _GeluMlp,
    _HeadsProjection,
    _QkvProjection,
    gelu_mlp,
    heads_projection,
    linear,
    mlp_fusable,
    qkv_projection,
    fresh_casts,
)
from .roll import _Roll


def _compute_dtype(x: torch.Tensor) -> torch.dtype:
    """The dtype a linear layer computes in: the autocast dtype when autocast is on."""
    return torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled() else x.dtype


def token_linear(x: torch.Tensor, layer: nn.Linear) -> torch.Tensor:
    """``layer(x)`` on this package's GEMM kernels in the compute dtype (bf16 on the matrix
    cores, other dtypes on the FMA kernel with the same addressing); the bias gradient is
    summed inside the weight-gradient GEMM."""
    return linear(x.to(_compute_dtype(x)), layer.weight, layer.bias)


def windows(x: torch.Tensor, window: int) -> torch.Tensor:
    """Cut a tile ``(B, h, w, C)`` into windows ``(B, nW, window*window, C)``, windows and the
    tokens inside a window both in row-major order (examples/swin.py:85-89)."""
    b, h, w, c = x.shape
    x = x.view(b, h // window, window, w // window, window, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, -1, window * window, c)


def unwindows(x: torch.Tensor, h: int, w: int, window: int) -> torch.Tensor:
    """Inverse of :func:`windows` (examples/swin.py:92-96)."""
    b, c = x.shape[0], x.shape[-1]
    x = x.view(b, h // window, w // window, window, window, c)
    return x.permute(0, 1, 3, 2, 4, 5).reshape(b, h, w, c)


def relative_position_index(window: int) -> torch.Tensor:
    """``(N, N)`` row of the bias table for a (query, key) pair of one window: the table is
    a ``(2W-1) x (2W-1)`` grid of displacements, row-major, displacement = query - key
    shifted to start at 0 (what examples/swin.py:99-104 computes)."""
    token = torch.arange(window * window)
    ty, tx = token // window, token % window
    dy = ty[:, None] - ty[None, :] + (window - 1)
    dx = tx[:, None] - tx[None, :] + (window - 1)
    return dy * (2 * window - 1) + dx


def border_sides(h: int, w: int, window: int, shift: int, groups: tuple) -> torch.Tensor:
    """``(nW, N)`` integer code per token of the rolled tile: bit 1 set when the roll by
    ``-shift`` carried the token across the lower image border, bit 0 when across the right
    one. A token at rolled GLOBAL position ``g`` came from ``g + shift``; it crossed iff that
    lies beyond the grid. The grid size and the tile's place in it come from the two spatial
    groups (objects with ``size()`` and ``rank()``)."""

    def crossed(local: int, group: Any) -> torch.Tensor:
        g = group.rank() * local + torch.arange(local)
        return g + shift >= local * group.size()

    code = crossed(h, groups[0])[:, None].long() * 2 + crossed(w, groups[1])[None, :].long()
    return windows(code[None, :, :, None], window)[0, :, :, 0]


def shift_mask(h: int, w: int, window: int, shift: int, groups: tuple) -> torch.Tensor:
    """Additive mask ``(nW, N, N)`` of this tile's windows after rolling the token grid by
    ``-shift``: 0 where query and key lie on the same side of the image borders, ``-inf``
    where the roll brought them together across one (the pairs examples/swin.py:107-126
    masks; a window holds tokens from both sides only if it touches the border of the
    GLOBAL grid, so the mask depends on where the tile sits)."""
    side = border_sides(h, w, window, shift, groups)
    apart = side[:, :, None] != side[:, None, :]
    return torch.zeros(apart.shape).masked_fill(apart, float("-inf"))


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
            side = border_sides(*tile, window, shift, groups).to(torch.uint8)
            self.register_buffer("side", side.contiguous().to(device), persistent=False)
        else:
            self.mask = self.side = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        b, h, w, c = x.shape
        dt = _compute_dtype(x)
        if dt == torch.bfloat16 and c // self.heads == 32 and self.window == 8 and h % 8 == 0 and w % 8 == 0:
            # the kernel addresses the windows on the token grid and forms bias and mask itself:
            # no window partition, no (nW, heads, N, N) bias tensor
            qkv = qkv_projection(x.to(dt).view(b, h * w, c), self.qkv.weight, self.qkv.bias, self.heads)
            out = swin_grid_attention_packed(qkv, self.bias_table, self.side, (h, w))
            return heads_projection(out, self.proj.weight, self.proj.bias).view(b, h, w, c)
        x = windows(x, self.window).to(dt)
        n = x.shape[2]
        # the projections write / read the (B, nW, heads, N, d) head layout themselves
        q, k, v = qkv_projection(x, self.qkv.weight, self.qkv.bias, self.heads).unbind(0)
        with torch.autocast("cuda", enabled=False):
            bias = (self.onehot @ self.bias_table.float()).view(n, n, -1).permute(2, 0, 1)
        if self.mask is not None:
            bias = bias[None] + self.mask[:, None]  # (nW, heads, N, N)
        out = window_attention(q, k, v, bias.contiguous())
        return unwindows(heads_projection(out, self.proj.weight, self.proj.bias), h, w, self.window)


class _Stage:
    """What one of the block's autograd functions keeps for its backward when the whole block is a
    single autograd function: the part of a ``ctx`` those functions use."""

    needs_input_grad = (True,) * 8
    saved_tensors: tuple = ()

    def save_for_backward(self, *tensors) -> None:
        self.saved_tensors = tensors


class _WholeBlock(torch.autograd.Function):
    """The block of :class:`SwinBlock` as ONE node of the autograd graph: the same launches in the
    same order as the functions it is made of (their ``forward`` / ``backward`` are called as they
    are, each with a :class:`_Stage` for its ``ctx``), so the numbers are theirs bit for bit. What
    goes is the bookkeeping of eight nodes per step, forward and in the engine's backward walk, which
    on a slow host is a third of the step's wall clock."""

    @staticmethod
    def forward(ctx, x, n1w, n1b, qkv_w, qkv_b, table, proj_w, proj_b, n2w, n2b, w1, b1, w2, b2, block):  # noqa: D102
        b, h, w, c = x.shape
        dt, eps, heads = _compute_dtype(x), block.eps, block.attn.heads
        st = [_Stage() for _ in range(8)]
        # what each part has to differentiate: its parameters as autograd asks for them here (a frozen parameter
        # gets no gradient kernel where the part looks at the flag); the inputs between the parts always, x itself
        # only when it wants a gradient
        nig = tuple(ctx.needs_input_grad) if hasattr(ctx, "needs_input_grad") else (True,) * 15
        pad = (False,) * 6
        st[0].needs_input_grad = (nig[0], nig[1], nig[2]) + pad
        st[1].needs_input_grad = (True,) + pad
        st[2].needs_input_grad = (True, nig[3], nig[4]) + pad
        st[3].needs_input_grad = (True, nig[5]) + pad
        st[4].needs_input_grad = (True, nig[6], nig[7]) + pad
        st[5].needs_input_grad = (True,) + pad
        st[6].needs_input_grad = (True, nig[8], nig[9]) + pad
        st[7].needs_input_grad = (True, nig[10], nig[11], nig[12], nig[13], True) + pad
        roll_args = block._roll_args()
        y = _PlainLayerNormFork.forward(st[0], x, n1w, n1b, eps, dt)[0]
        if block.shift_by:
            y = _Roll.forward(st[1], y.contiguous(), (-block.shift_by,) * 2, (1, 2), *roll_args)
        qkv = _QkvProjection.forward(st[2], y.view(b, h * w, c), qkv_w, qkv_b, heads)
        out = _SwinGridAttention.forward(st[3], qkv, table, block.attn.side, (h, w))
        a = _HeadsProjection.forward(st[4], out, proj_w, proj_b).view(b, h, w, c)
        if block.shift_by:
            a = _Roll.forward(st[5], a.contiguous(), (block.shift_by,) * 2, (1, 2), *roll_args)
        x1 = x + a.to(x.dtype)
        y2 = _PlainLayerNormFork.forward(st[6], x1, n2w, n2b, eps, dt)[0]
        result = _GeluMlp.forward(st[7], y2, w1, b1, w2, b2, x1)
        ctx.stages, ctx.shifted, ctx.branch_dtype, ctx.grid = st, bool(block.shift_by), a.dtype, (b, h, w, c)
        return result

    @staticmethod
    def backward(ctx, grad):  # noqa: D102
        if ctx.stages is None:
            raise RuntimeError(
                "SwinBlock (one autograd node): backward was called a second time, but the tensors the first pass "
                "kept were released when it finished (they are not held through save_for_backward, so "
                "retain_graph=True does not keep them). Run the forward again, or build the block with one_node=False."
            )
        st, (b, h, w, c) = ctx.stages, ctx.grid
        gy2, gw1, gb1, gw2, gb2, over = _GeluMlp.backward(st[7], grad)
        gx1, gn2w, gn2b = _PlainLayerNormFork.backward(st[6], gy2, over)[:3]
        ga = gx1.to(ctx.branch_dtype)
        if ctx.shifted:
            ga = _Roll.backward(st[5], ga)[0]
        gout, gpw, gpb = _HeadsProjection.backward(st[4], ga.view(b, h * w, c))[:3]
        dqkv, dtable = _SwinGridAttention.backward(st[3], gout)[:2]
        gy, gqw, gqb = _QkvProjection.backward(st[2], dqkv)[:3]
        gy = gy.view(b, h, w, c)
        if ctx.shifted:
            gy = _Roll.backward(st[1], gy)[0]
        gx, gn1w, gn1b = _PlainLayerNormFork.backward(st[0], gy, gx1)[:3]
        ctx.stages = None
        return gx, gn1w, gn1b, gqw, gqb, dtable, gpw, gpb, gn2w, gn2b, gw1, gb1, gw2, gb2, None


class CapturedStep:
    """One forward + backward of a :class:`SwinBlock` as a HIP graph (see ``SwinBlock.captured_step``).

    ``x`` / ``grad_out``: the input buffers. After :meth:`replay`: ``y`` the block's output, ``grad_x``
    the gradient of ``x``, ``grads`` the gradients of the parameters by name (fresh values at every
    replay, not accumulated into ``.grad``). A replay only enqueues work on the current stream."""

    _NAMES = ("norm1.weight", "norm1.bias", "attn.qkv.weight", "attn.qkv.bias", "attn.bias_table", "attn.proj.weight",
              "attn.proj.bias", "norm2.weight", "norm2.bias", "mlp.0.weight", "mlp.0.bias", "mlp.2.weight", "mlp.2.bias")

    def __init__(self, block: "SwinBlock", x: torch.Tensor, grad_out: torch.Tensor, warmup: int):
        self.x, self.grad_out = x, grad_out
        named = dict(block.named_parameters())
        params = [named[n].detach() for n in self._NAMES]

        def step():
            ctx = _Stage()
            ctx.needs_input_grad = (True,) * 15
            # the bf16 copies of the fp32 parameters are made inside the step, so a replay reads the parameters
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16), fresh_casts():
                y = _WholeBlock.forward(ctx, self.x, *params, block)
                return y, _WholeBlock.backward(ctx, self.grad_out)

        # first calls outside the capture: one-time set-up of the kernels (LDS reservations, lookup tables)
        # and the allocator's pool for the capturing stream
        side = torch.cuda.Stream(device=x.device)
        side.wait_stream(torch.cuda.current_stream(x.device))
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                step()
        torch.cuda.current_stream(x.device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            self.y, grads = step()
        self.grad_x = grads[0]
        self.grads = dict(zip(self._NAMES, grads[1:14]))

    def replay(self) -> None:
        self.graph.replay()


class SwinBlock(nn.Module):
    """``x + attn(norm(x))`` then ``x + mlp(norm(x))``; the windows may be shifted
    (examples/swin.py:173-210). ``groups`` are the two spatial groups of the tile
    (objects with ``size()`` / ``rank()``), ``comm_halo_1d_fn`` the 1-D exchange the
    roll uses (``RollConfig.comm_halo_1d_fn`` in the reference)."""

    def __init__(self, dim: int, heads: int, window: int, tile: tuple, groups: tuple = None,
                 comm_halo_1d_fn: Callable | None = None, shift: int = 0, device=None, eps: float = 1e-5,
                 one_node: bool = True) -> None:
        super().__init__()
        groups = groups or (TileGroup(1, 0), TileGroup(1, 0))
        self.groups, self.comm, self.shift_by, self.eps = groups, comm_halo_1d_fn, shift, eps
        self.one_node = one_node  # the whole block as one autograd function where its fused kernels apply
        self.norm1 = nn.LayerNorm(dim, eps=eps, device=device)
        self.attn = WindowAttention(dim, heads, window, tile, shift, groups, device)
        self.norm2 = nn.LayerNorm(dim, eps=eps, device=device)
        self.mlp = nn.Sequential(nn.Linear(dim, 4 * dim, device=device), nn.GELU(), nn.Linear(4 * dim, dim, device=device))

    def _roll_args(self) -> tuple:
        dist_dims = tuple(d for d, g in zip((1, 2), self.groups) if g.size() > 1)
        dist_groups = tuple(g for g in self.groups if g.size() > 1)
        return dist_dims, dist_groups, self.comm

    def _roll(self, x: torch.Tensor, shift: int) -> torch.Tensor:
        if not shift:
            return x
        return _Roll.apply(x.contiguous(), (shift, shift), (1, 2), *self._roll_args())

    def _one_node(self, x: torch.Tensor) -> bool:
        """Whether the block runs as one autograd function: the shapes all of its fused kernels take."""
        if not self.one_node or x.dim() != 4 or not x.is_cuda or x.numel() == 0:
            return False
        if x.dtype != torch.bfloat16 or _compute_dtype(x) != torch.bfloat16:
            return False
        b, h, w, c = x.shape
        attn, fc1, fc2 = self.attn, self.mlp[0], self.mlp[2]
        if c % attn.heads or c // attn.heads != 32 or attn.window != 8 or h % 8 or w % 8:
            return False
        if not _lib.load().jg_ln_plain_supported(c) or any(t is None for t in (attn.qkv.bias, attn.proj.bias, fc1.bias, fc2.bias)):
            return False
        return mlp_fusable(x, fc1.weight, fc2.weight, x)

    def captured_step(self, x: torch.Tensor, grad_out: torch.Tensor, warmup: int = 3) -> "CapturedStep":
        """Forward + backward of the block for these shapes, recorded once in a HIP graph.

        The launches are those of the one-node form (bf16 tokens, 8 x 8 windows, heads of 32), issued
        by calling its ``forward`` / ``backward`` directly, with no autograd engine in between: no
        worker thread, no accumulation nodes, nothing a stream capture refuses. ``x`` and
        ``grad_out`` become the graph's input buffers (copy new values into them before a replay),
        the block's parameters are read where they lie at every replay, and the results are written to
        the same tensors every time. The roll's ``comm_fn`` runs while the graph is recorded, on the
        capturing stream: whatever it launches there is replayed with the rest."""
        if not self._one_node_ok(x):
            raise NotImplementedError("captured_step needs the shapes of the one-node block: bf16 tokens, 8 x 8 windows, "
                                      "heads of 32, biases present")
        if grad_out.shape != x.shape or grad_out.dtype != x.dtype:
            raise ValueError(f"grad_out {tuple(grad_out.shape)} {grad_out.dtype} does not match x {tuple(x.shape)} {x.dtype}")
        return CapturedStep(self, x.detach(), grad_out.detach(), warmup)

    def _one_node_ok(self, x: torch.Tensor) -> bool:
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return self._one_node(x)

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
        fc1, fc2 = self.mlp[0], self.mlp[2]
        return gelu_mlp(self._norm(self.norm2, x), fc1.weight, fc1.bias, fc2.weight, fc2.bias, residual=x)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # x + f(norm(x)) twice; the rows that go round a branch come out of the LayerNorm call beside
        # the normalised ones, so that the backward adds the two gradients of x inside its kernel
        dt = _compute_dtype(x)
        if self._one_node(x):
            attn, fc1, fc2 = self.attn, self.mlp[0], self.mlp[2]
            return _WholeBlock.apply(x, self.norm1.weight, self.norm1.bias, attn.qkv.weight, attn.qkv.bias, attn.bias_table,
                                     attn.proj.weight, attn.proj.bias, self.norm2.weight, self.norm2.bias, fc1.weight, fc1.bias,
                                     fc2.weight, fc2.bias, self)
        y, x = plain_layer_norm_fork(x, self.norm1.weight, self.norm1.bias, self.eps, out_dtype=dt)
        x = x + self.unshift(self.attn(self.shift(y))).to(x.dtype)
        y, x = plain_layer_norm_fork(x, self.norm2.weight, self.norm2.bias, self.eps, out_dtype=dt)
        fc1, fc2 = self.mlp[0], self.mlp[2]
        return gelu_mlp(y, fc1.weight, fc1.bias, fc2.weight, fc2.bias, residual=x)


__all__ = ["SwinBlock", "WindowAttention", "border_sides", "relative_position_index", "shift_mask", "unwindows", "windows"]
