"""Oracle for the halo exchange of the distributed convolution.

All ranks of a spatial group are simulated in one process: the uneven
all-to-all of the reference becomes list indexing, everything else (span
arithmetic, zero fill, placement, add order) follows the reference line by line
in meaning. Test infrastructure only.
"""

from __future__ import annotations

import itertools

import torch


def needed_input_span(rank, group_size, local_in_size, kernel, stride, padding, dilation):
    """``(lo, hi, need, out_local)`` of a rank's output block.

    Follows jigsaw/modules/convolution/_conv/halo.py:49-63.
    """
    extent = dilation * (kernel - 1) + 1
    global_in = group_size * local_in_size
    global_out = (global_in + 2 * padding - extent) // stride + 1
    if global_out % group_size != 0:
        raise NotImplementedError(
            f"global output size {global_out} not divisible by group size {group_size}"
        )
    out_local = global_out // group_size
    lo = rank * out_local * stride - padding
    need = (out_local - 1) * stride + extent
    return lo, lo + need, need, out_local


def gather_axis(tiles, kernel, stride, padding, dilation, axis):
    """Halo-padded slice of every rank of one spatial group along ``axis``.

    ``tiles[r]`` is rank r's local tensor. Follows halo_gather,
    jigsaw/modules/convolution/_conv/halo.py:101-156: a zero tensor of the need
    span (:112-114), then for every peer (own rank included) the rows the peer
    owns inside the span are copied in (:134-154); out-of-domain rows stay 0.
    """
    G = len(tiles)
    n = tiles[0].shape[axis]
    out = []
    for rank in range(G):
        lo, hi, need, _ = needed_input_span(rank, G, n, kernel, stride, padding, dilation)
        shape = list(tiles[rank].shape)
        shape[axis] = need
        x_need = tiles[rank].new_zeros(shape)
        for peer in range(G):
            r0 = max(lo, peer * n, 0)
            cnt = max(min(hi, (peer + 1) * n, G * n) - r0, 0)
            if cnt > 0:
                x_need.narrow(axis, r0 - lo, cnt).copy_(tiles[peer].narrow(axis, r0 - peer * n, cnt))
        out.append(x_need.contiguous())
    return out


def scatter_add_axis(grads, kernel, stride, padding, dilation, local_in_size, axis):
    """Fold the padded gradients of one spatial group back onto the owners.

    ``grads[r]`` is rank r's gradient of its need span. Follows
    halo_scatter_add, jigsaw/modules/convolution/_conv/halo.py:195-251:
    ``g_local = zeros`` (:207), then ``g_local[off:off+n] += recv[peer]`` for
    peer = 0..G-1 in that order (:247-249), where recv[peer] is the part of the
    peer's span this rank owns (:232-238), the rank's own span included.
    """
    G = len(grads)
    n = local_in_size
    spans = [needed_input_span(r, G, n, kernel, stride, padding, dilation) for r in range(G)]
    out = []
    for rank in range(G):
        shape = list(grads[rank].shape)
        shape[axis] = n
        g_local = grads[rank].new_zeros(shape)
        for peer in range(G):
            p_lo, p_hi = spans[peer][0], spans[peer][1]
            r0 = max(p_lo, rank * n, 0)
            cnt = max(min(p_hi, (rank + 1) * n, G * n) - r0, 0)
            if cnt > 0:
                g_local.narrow(axis, r0 - rank * n, cnt).add_(grads[peer].narrow(axis, r0 - p_lo, cnt))
        out.append(g_local)
    return out


def _lines(mesh_shape, k):
    """Index tuples of every 1-D line of ranks along mesh axis ``k``."""
    others = [range(s) if i != k else [None] for i, s in enumerate(mesh_shape)]
    for idx in itertools.product(*others):
        yield [tuple(r if j is None else j for j in idx) for r in range(mesh_shape[k])]


def gather_mesh(tiles, mesh_shape, kernel, stride, padding, dilation):
    """Padded tile of every rank of an N-D spatial mesh.

    ``tiles`` maps a mesh coordinate (one entry per spatial axis) to the local
    ``(N, C, *spatial)`` tensor. Axes with a group of size 1 are not exchanged;
    the split axes run first to last (H, then W), as the ``_halo_fn`` loop of
    jigsaw/modules/convolution/_conv/distributed.py:264-275 over ``_split_axes``
    (_common/spatial_split.py:9-16).
    """
    ns = len(mesh_shape)
    cur = dict(tiles)
    for k in range(ns):
        if mesh_shape[k] <= 1:
            continue
        axis = k - ns
        for line in _lines(mesh_shape, k):
            res = gather_axis([cur[c] for c in line], kernel[k], stride[k], padding[k], dilation[k], axis)
            for c, t in zip(line, res):
                cur[c] = t
    return cur


def scatter_add_mesh(grads, mesh_shape, kernel, stride, padding, dilation, local_in_spatial):
    """Owned-gradient of every rank from the padded gradients of the mesh.

    Split axes are folded last to first (W, then H), as
    jigsaw/modules/convolution/_conv/distributed.py:378-389.
    """
    ns = len(mesh_shape)
    cur = dict(grads)
    for k in reversed(range(ns)):
        if mesh_shape[k] <= 1:
            continue
        axis = k - ns
        for line in _lines(mesh_shape, k):
            res = scatter_add_axis(
                [cur[c] for c in line], kernel[k], stride[k], padding[k], dilation[k], local_in_spatial[k], axis
            )
            for c, t in zip(line, res):
                cur[c] = t
    return cur


def local_padding(padding, mesh_shape):
    """Padding of the local conv: zero on split axes.

    Follows _local_padding, jigsaw/modules/convolution/_common/spatial_split.py:75-82.
    """
    return tuple(0 if g > 1 else p for p, g in zip(padding, mesh_shape))


def split_global(x, mesh_shape):
    """Cut a global ``(N, C, *spatial)`` tensor into equal tiles per mesh coordinate."""
    ns = len(mesh_shape)
    tiles = {}
    for c in itertools.product(*[range(s) for s in mesh_shape]):
        t = x
        for k in range(ns):
            n = x.shape[k - ns] // mesh_shape[k]
            t = t.narrow(k - ns, c[k] * n, n)
        tiles[c] = t.contiguous()
    return tiles
