"""Oracle for the distributed transposed convolution. Test infrastructure only.

All ranks of a spatial mesh are simulated in one process; the exchanges of the
reference become list indexing. Follows jigsaw/modules/convolution/_conv_transpose/
halo.py (spans, reduce, expand) and distributed.py:212-283 (axis order, local padding).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .halo import _lines

_CONVT = {1: F.conv_transpose1d, 2: F.conv_transpose2d, 3: F.conv_transpose3d}


def produced_output_span(rank, group_size, local_in_size, kernel, stride, padding, dilation):
    """``(base, wloc, out_local, global_out)`` of a rank's raw local output
    (_conv_transpose/halo.py:53-71)."""
    extent = dilation * (kernel - 1) + 1
    global_in = group_size * local_in_size
    global_out = (global_in - 1) * stride - 2 * padding + extent
    if global_out % group_size != 0:
        raise NotImplementedError(f"global output size {global_out} not divisible by group size {group_size}")
    out_local = global_out // group_size
    base = rank * local_in_size * stride - padding
    wloc = (local_in_size - 1) * stride + extent
    return base, wloc, out_local, global_out


def reduce_axis(raws, local_in_size, kernel, stride, padding, dilation, axis):
    """Sum the overlapping raw outputs of one spatial group onto their owners along
    ``axis`` (transpose_halo_reduce, _conv_transpose/halo.py:111-160): a zero shard, then
    for every peer in rank order the part of the peer's raw span that lands in the shard
    is added; columns outside the global output are dropped."""
    G = len(raws)
    out = []
    for rank in range(G):
        _, _, out_local, global_out = produced_output_span(rank, G, local_in_size, kernel, stride, padding, dilation)
        keep_lo = rank * out_local
        shape = list(raws[rank].shape)
        shape[axis] = out_local
        y = raws[rank].new_zeros(shape)
        for peer in range(G):
            pb, pw, _, _ = produced_output_span(peer, G, local_in_size, kernel, stride, padding, dilation)
            r0 = max(keep_lo, pb, 0)
            cnt = max(min(keep_lo + out_local, pb + pw, global_out) - r0, 0)
            if cnt > 0:
                y.narrow(axis, r0 - keep_lo, cnt).add_(raws[peer].narrow(axis, r0 - pb, cnt))
        out.append(y.contiguous())
    return out


def expand_axis(grads, local_in_size, kernel, stride, padding, dilation, axis):
    """Reverse of :func:`reduce_axis` (transpose_halo_expand, _conv_transpose/halo.py:196-258):
    the gradient of every rank's raw span, gathered from the owners; zero outside the
    global output."""
    G = len(grads)
    out = []
    for rank in range(G):
        base, wloc, out_local, global_out = produced_output_span(rank, G, local_in_size, kernel, stride, padding, dilation)
        shape = list(grads[rank].shape)
        shape[axis] = wloc
        raw = grads[rank].new_zeros(shape)
        for peer in range(G):
            peer_lo = peer * out_local
            r0 = max(base, peer_lo, 0)
            cnt = max(min(base + wloc, peer_lo + out_local, global_out) - r0, 0)
            if cnt > 0:
                raw.narrow(axis, r0 - base, cnt).copy_(grads[peer].narrow(axis, r0 - peer_lo, cnt))
        out.append(raw.contiguous())
    return out


def _over_lines(tensors, mesh_shape, k, fn):
    out = dict(tensors)
    for line in _lines(mesh_shape, k):
        res = fn([out[c] for c in line])
        for c, t in zip(line, res):
            out[c] = t
    return out


def reduce_mesh(raws, mesh_shape, local_in_spatial, kernel, stride, padding, dilation):
    """All split axes in forward order (distributed.py:226-238); ``raws`` maps mesh coordinate -> tensor."""
    ns = len(mesh_shape)
    out = dict(raws)
    for k in range(ns):
        if mesh_shape[k] > 1:
            out = _over_lines(out, mesh_shape, k, lambda ts, k=k: reduce_axis(
                ts, local_in_spatial[k], kernel[k], stride[k], padding[k], dilation[k], axis=k - ns))
    return out


def expand_mesh(grads, mesh_shape, local_in_spatial, kernel, stride, padding, dilation):
    """All split axes in reverse order (distributed.py:260-271)."""
    ns = len(mesh_shape)
    out = dict(grads)
    for k in reversed(range(ns)):
        if mesh_shape[k] > 1:
            out = _over_lines(out, mesh_shape, k, lambda ts, k=k: expand_axis(
                ts, local_in_spatial[k], kernel[k], stride[k], padding[k], dilation[k], axis=k - ns))
    return out


def local_forward(x, w, stride, local_padding, dilation):
    """Raw local output: the native transposed conv with padding 0 on split axes
    (distributed.py:240-246; bias is added after the reduction, channel_comm.py:164-168)."""
    return _CONVT[w.dim() - 2](x, w, None, stride=stride, padding=local_padding, dilation=dilation)
