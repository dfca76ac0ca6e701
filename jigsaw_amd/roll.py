"""DistributedRoll on the GPU: local cyclic roll + wrapped-slab pack / unpack.

Host-side mirror of jigsaw/modules/roll/_distributed_roll.py and the autograd
function of jigsaw/modules/roll/_functional.py. Signatures follow the reference
so that ``distributed_roll`` can stand where the reference's does; the exchange
itself stays an injected callable (``RollConfig.comm_halo_1d_fn``,
jigsaw/modules/roll/_config.py:26-27).
"""

from __future__ import annotations

from collections.abc import Callable, Sequence
from typing import Any

import torch

from . import _lib


def roll(x: torch.Tensor, shifts: Sequence[int], dims: Sequence[int]) -> torch.Tensor:
    """``torch.roll(x, shifts, dims)`` through ``jg_roll`` (one gather pass)."""
    _lib.require_gpu(x)
    if len(shifts) != len(dims):
        raise RuntimeError(f"shifts and dimensions must align. shifts: {len(shifts)}, dims:{len(dims)}")
    x = x.contiguous()
    per_axis = [0] * x.dim()
    for s, d in zip(shifts, dims):
        per_axis[d % x.dim()] += int(s)  # torch.roll applies repeated dims one after another
    out = torch.empty_like(x)
    if x.numel() == 0:
        return out
    if x.dim() > 6:
        raise NotImplementedError("roll: more than 6 axes")
    rc = _lib.load().jg_roll(
        _lib.ptr(out),
        _lib.ptr(x),
        x.dim(),
        _lib.i64_array(x.shape),
        _lib.i64_array(per_axis),
        x.element_size(),
        _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "jg_roll")
    return out


def slab_pack(x: torch.Tensor, dim: int, window_size: int) -> torch.Tensor:
    """``x[sl].contiguous()`` for the wrapped slab of ``exchange_halo_1d``."""
    _lib.require_gpu(x)
    if not x.is_contiguous():
        raise ValueError("slab_pack: x must be contiguous")
    dim %= x.dim()
    shape = list(x.shape)
    shape[dim] = abs(int(window_size))
    strip = torch.empty(shape, dtype=x.dtype, device=x.device)
    rc = _lib.load().jg_roll_pack(
        _lib.ptr(strip), _lib.ptr(x), x.dim(), _lib.i64_array(x.shape), dim, int(window_size),
        x.element_size(), _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "jg_roll_pack")
    return strip


def slab_unpack_(x: torch.Tensor, strip: torch.Tensor, dim: int, window_size: int) -> torch.Tensor:
    """``x[sl] = strip`` in place for the wrapped slab of ``exchange_halo_1d``."""
    _lib.require_gpu(x, strip)
    if not x.is_contiguous():
        raise ValueError("slab_unpack_: x must be contiguous")
    dim %= x.dim()
    shape = list(x.shape)
    shape[dim] = abs(int(window_size))
    strip = strip.to(dtype=x.dtype).contiguous()
    if list(strip.shape) != shape:
        raise ValueError(f"slab_unpack_: strip shape {tuple(strip.shape)} != {tuple(shape)}")
    rc = _lib.load().jg_roll_unpack(
        _lib.ptr(x), _lib.ptr(strip), x.dim(), _lib.i64_array(x.shape), dim, int(window_size),
        x.element_size(), _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "jg_roll_unpack")
    return x


def exchange_halo_1d(
    x: torch.Tensor,
    dim: int,
    window_size: int,
    group: Any,
    comm_halo_1d_fn: Callable,
) -> torch.Tensor:
    """Swap the wrapped slab of ``x`` along ``dim`` with the ring neighbour.

    Same contract as jigsaw/modules/roll/_distributed_roll.py:9-60: a positive
    ``window_size`` sends the leading slab with ``direction = +1`` and writes the
    received one in its place, a negative one the trailing slab with
    ``direction = -1``. ``x`` is modified in place.
    """
    if window_size == 0:
        return x
    halo_to_send = slab_pack(x, dim, window_size)
    recv = torch.zeros_like(halo_to_send)
    offset = 1 if window_size > 0 else -1
    recv, _ = comm_halo_1d_fn(halo_to_send, recv, offset, group=group, async_op=False)
    return slab_unpack_(x, recv, dim, window_size)


def _fused_steps_ok(x: torch.Tensor, per_axis: list, axes: list) -> bool:
    """Whether the one-pass kernels take this roll: distinct slab axes, and behind the last rolled
    axis and the last slab axis a run of whole 16-byte words."""
    if x.numel() == 0 or x.dim() > 5 or x.element_size() not in (2, 4) or len(set(axes)) != len(axes):
        return False
    rolled = [a for a, s in enumerate(per_axis) if s % x.shape[a] != 0]
    tail_from = max([*rolled, *axes]) + 1
    run = 1
    for n in x.shape[tail_from:]:
        run *= n
    return (run * x.element_size()) % 16 == 0 and x.data_ptr() % 16 == 0


def distributed_roll(
    x: torch.Tensor,
    shifts: tuple,
    dims: tuple,
    distributed_dims: list,
    spatial_process_groups: list,
    exchange_halo_1d_fn: Callable,
) -> torch.Tensor:
    """Roll the local tile and exchange the wrapped slabs of its distributed dims.

    Same contract and error behaviour as ``distributed_roll`` of
    jigsaw/modules/roll/_distributed_roll.py:63-113 (``exchange_halo_1d_fn`` is,
    as there, the 1-D communication function). Where the layout allows, the passes between
    two exchanges are one launch each: roll + cut of the first slab + clearing of its receive
    buffer; write-back of a received slab + cut of the next one; the last write-back.
    """
    if len(shifts) != len(dims):
        raise RuntimeError(f"shifts and dimensions must align. shifts: {len(shifts)}, dims:{len(dims)}")
    nd = x.dim()
    dim_to_shift = {d % nd: s for d, s in zip(dims, shifts)}
    if len(distributed_dims) != len(spatial_process_groups):
        raise ValueError("distributed_dims and spatial_process_groups differ in length")
    steps = []
    for d, pg in zip(distributed_dims, spatial_process_groups):
        if d % nd not in dim_to_shift:
            raise ValueError(f"distributed dim {d} not in dims {dims}")
        if dim_to_shift[d % nd] != 0:
            steps.append((d % nd, int(dim_to_shift[d % nd]), pg))
    per_axis = [0] * nd
    for s, d in zip(shifts, dims):
        per_axis[d % nd] += int(s)
    x = x.contiguous()
    if not steps or not _fused_steps_ok(x, per_axis, [a for a, _, _ in steps]):
        x = roll(x, shifts, dims)
        for axis, window, pg in steps:
            x = exchange_halo_1d(x, dim=axis, window_size=window, group=pg, comm_halo_1d_fn=exchange_halo_1d_fn)
        return x

    _lib.require_gpu(x)
    lib = _lib.load()
    shape, esize, stream = _lib.i64_array(x.shape), x.element_size(), _lib.stream_ptr(x.device)

    def buffers(axis, window):
        slab = list(x.shape)
        slab[axis] = abs(window)
        return torch.empty(slab, dtype=x.dtype, device=x.device), torch.empty(slab, dtype=x.dtype, device=x.device)

    out = torch.empty_like(x)
    axis, window, pg = steps[0]
    if abs(window) > x.shape[axis]:
        raise ValueError(f"|window| = {abs(window)} exceeds the local size {x.shape[axis]} along dim {axis}")
    strip, recv = buffers(axis, window)
    rc = lib.jg_roll_pack_fused(_lib.ptr(out), _lib.ptr(strip), _lib.ptr(recv), _lib.ptr(x), nd, shape,
                                _lib.i64_array(per_axis), axis, window, esize, stream)
    _lib.check(rc, "jg_roll_pack_fused")
    recv, _ = exchange_halo_1d_fn(strip, recv, 1 if window > 0 else -1, group=pg, async_op=False)
    for axis2, window2, pg2 in steps[1:]:
        if abs(window2) > x.shape[axis2]:
            raise ValueError(f"|window| = {abs(window2)} exceeds the local size {x.shape[axis2]} along dim {axis2}")
        strip2, recv2 = buffers(axis2, window2)
        recv = recv.to(dtype=x.dtype).contiguous()
        rc = lib.jg_roll_unpack_pack(_lib.ptr(out), _lib.ptr(recv), axis, window, _lib.ptr(strip2), _lib.ptr(recv2),
                                     axis2, window2, nd, shape, esize, stream)
        _lib.check(rc, "jg_roll_unpack_pack")
        recv, _ = exchange_halo_1d_fn(strip2, recv2, 1 if window2 > 0 else -1, group=pg2, async_op=False)
        axis, window = axis2, window2
    return slab_unpack_(out, recv, axis, window)


class _Roll(torch.autograd.Function):
    """Autograd function of the distributed roll (jigsaw/modules/roll/_functional.py:30-117):
    the backward is the same roll with negated shifts."""

    @staticmethod
    def forward(ctx, x, shifts, dims, distributed_dims, spatial_groups, comm_halo_1d_fn):  # noqa: D102
        ctx.args = (tuple(shifts), tuple(dims), tuple(distributed_dims), tuple(spatial_groups), comm_halo_1d_fn)
        return distributed_roll(x, tuple(shifts), tuple(dims), list(distributed_dims), list(spatial_groups), comm_halo_1d_fn)

    @staticmethod
    def backward(ctx, grad_output):  # noqa: D102
        shifts, dims, distributed_dims, spatial_groups, comm = ctx.args
        neg = tuple(-s for s in shifts)
        g = distributed_roll(grad_output.contiguous(), neg, dims, list(distributed_dims), list(spatial_groups), comm)
        return g, None, None, None, None, None


__all__ = ["_Roll", "distributed_roll", "exchange_halo_1d", "roll", "slab_pack", "slab_unpack_"]
