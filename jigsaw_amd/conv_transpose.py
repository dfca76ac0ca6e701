"""One rank's share of the distributed transposed convolution on the GPU.

Host-side mirror of jigsaw/modules/convolution/_conv_transpose/: the hooks of
``ConvTransposeNdConfig`` (config.py:67-84) and the contracts of
``conv_transpose_halo_nway`` / ``conv_transpose_halo_nway_backward``
(distributed.py:212-283) and ``_ConvTransposeNd`` (functional.py).

The transposed convolution is the convolution's mirror image, and so is its data flow:
the raw local output is the input gradient of a convolution (``conv_nd_input``), the
overlap of neighbouring raw outputs is summed onto the owners by the same fold that the
convolution's backward uses (``transpose_halo_reduce`` == ``halo_scatter_add`` on the
raw span), the backward gathers the output gradient over the raw span (``halo_assemble``)
and then runs a plain convolution for the input gradient and the weight-gradient kernel
with the two operands exchanged. Every kernel is one the convolution already has.
"""

from __future__ import annotations

from typing import Any

import torch

from .conv import (
    _cast_to_autocast_dtype,
    _HipLayerConfig,
    _local_padding,
    _mesh_position,
    _present_offsets,
    conv_nd,
    conv_nd_input,
    conv_nd_input_fold,
    conv_nd_weight,
)
from .halo import HaloGeometry, halo_assemble, halo_fold, halo_fold_border_, halo_pack, neighbour_widths


def produced_output_span(rank, group_size, local_in_size, kernel, stride, padding, dilation):
    """``(base, wloc, out_local, global_out)``: local column ``i`` of a rank's raw output
    is global column ``base + i``; the rank keeps ``out_local`` of the ``global_out``
    columns (_conv_transpose/halo.py:14-71)."""
    extent = dilation * (kernel - 1) + 1
    global_in = group_size * local_in_size
    global_out = (global_in - 1) * stride - 2 * padding + extent
    if global_out % group_size != 0:
        raise NotImplementedError(
            "Distributed ConvTranspose with a halo exchange needs the "
            f"global output size along the split axis ({global_out}) to be "
            f"divisible by the spatial group size ({group_size})."
        )
    out_local = global_out // group_size
    base = rank * local_in_size * stride - padding
    wloc = (local_in_size - 1) * stride + extent
    return base, wloc, out_local, global_out


def raw_span_widths(rank, group_size, local_in_size, kernel, stride, padding, dilation):
    """``(left, right, out_local)``: how many raw output columns of a rank lie before and
    behind the block it keeps. They change from rank to rank when ``extent != stride +
    2 * padding`` (the raw spans drift against the blocks). Accepted: the raw span covers
    the kept block and reaches at most one block to either side, so that every overlap
    is with an adjacent rank; anything else raises ``NotImplementedError``."""
    base, wloc, out_local, _ = produced_output_span(rank, group_size, local_in_size, kernel, stride, padding, dilation)
    left = rank * out_local - base
    right = wloc - left - out_local
    if left < 0 or right < 0:
        raise NotImplementedError(
            f"transposed conv on a split axis: the raw span [{base}, {base + wloc}) of rank {rank} does not cover "
            f"the block it keeps [{rank * out_local}, {(rank + 1) * out_local})"
        )
    if left > out_local or right > out_local:
        raise NotImplementedError(
            f"transposed conv on a split axis: the raw span of rank {rank} reaches {left} / {right} columns past its "
            f"block of {out_local}: overlaps with non-adjacent ranks"
        )
    return left, right, out_local


def transpose_geometry(local_in_spatial, kernel, stride, padding, dilation, ranks, group_sizes) -> HaloGeometry:
    """The raw span of a rank as a halo geometry: the owned output block with ``lo`` raw
    columns before it and ``hi`` after, and the neighbours' widths where the spans drift
    (_conv_transpose/halo.py:14-71 and the per-peer overlaps of :134-152). Axes with a
    group of one carry no halo (the local transposed conv applies their padding itself)."""
    size, lo, hi, tlo, thi = [], [], [], [], []
    for a, n in enumerate(local_in_spatial):
        k, s, p, d = kernel[a], stride[a], padding[a], dilation[a]
        if group_sizes[a] <= 1:
            size.append((n - 1) * s - 2 * p + d * (k - 1) + 1)
            for w in (lo, hi, tlo, thi):
                w.append(0)
            continue
        args = (group_sizes[a], n, k, s, p, d)
        l, h, tl, th = neighbour_widths(lambda r: raw_span_widths(r, *args), ranks[a], group_sizes[a])  # noqa: B023
        size.append(raw_span_widths(ranks[a], *args)[2])
        lo.append(l)
        hi.append(h)
        tlo.append(tl)
        thi.append(th)
    return HaloGeometry(tuple(size), tuple(lo), tuple(hi), tuple(tlo), tuple(thi))


def conv_transpose_nd(x, w, b=None, *, stride=1, padding=0, dilation=1, groups=1) -> torch.Tensor:
    """``F.conv_transpose{1,2,3}d(x, w, b, stride, padding, 0, groups, dilation)`` — the
    ``conv_transpose_fn`` hook (config.py:67-68). ``w`` is ``(C_in, C_out, *k)``."""
    n = w.dim() - 2
    tup = lambda v: (v,) * n if isinstance(v, int) else tuple(v)  # noqa: E731
    s, p, d = tup(stride), tup(padding), tup(dilation)
    raw = tuple((x.shape[2 + a] - 1) * s[a] - 2 * p[a] + d[a] * (w.shape[2 + a] - 1) + 1 for a in range(n))
    y = conv_nd_input((x.shape[0], w.shape[1] * groups, *raw), w, x, stride=s, padding=p, dilation=d, groups=groups)
    if b is not None:
        y += b.to(y.dtype).view((1, -1) + (1,) * n)
    return y


def conv_transpose_halo_nway(x, w, b, stride, padding, dilation, spatial_groups, channel_group, config):
    """Transposed convolution with a halo reduction on every split axis; returns ``(y, x)``.

    Same contract as ``conv_transpose_halo_nway`` (distributed.py:212-257) for a
    channel-local layer: raw local output, overlaps summed onto the owners, bias added
    after the reduction (channel_comm.py:164-168)."""
    if channel_group is not None and channel_group.size() != 1:
        raise NotImplementedError("channel-sharded convolution is outside this package (col must be 1)")
    n = config.n_spatial
    ranks, sizes = _mesh_position(spatial_groups)
    x = x.contiguous()
    geom = transpose_geometry(x.shape[-n:], w.shape[-n:], stride, padding, dilation, ranks, sizes)
    present = _present_offsets(geom, ranks, sizes)
    kwargs = {"stride": stride, "padding": _local_padding(padding, sizes), "dilation": dilation, "groups": int(getattr(config, "groups_local", 1))}
    fused = conv_nd_input_fold(geom, w, x, present=present, **kwargs) if getattr(config, "fused_fold", False) else None
    if fused is not None:
        y, send = fused
        recv = config.halo_exchange.forward(send) if present else {}
        halo_fold_border_(y, recv, geom)
    else:
        y_raw = conv_nd_input((x.shape[0], w.shape[1] * kwargs["groups"], *geom.padded), w, x, **kwargs)
        send = halo_pack(y_raw, geom, from_padded=True, present=present) if present else {}
        recv = config.halo_exchange.forward(send) if present else {}
        y = halo_fold(y_raw, recv, geom)
    if b is not None:
        y += b.to(y.dtype).view((1, -1) + (1,) * n)
    # the input kept for the backward pass; detached, as it is handed out non-differentiable
    return y, x.detach()


def conv_transpose_halo_nway_backward(
    grad_output, x_aug, weight, stride, padding, dilation, local_in_spatial, spatial_groups, channel_group, config,
    need=(True, True),
):
    """Gradients of the halo-reduction transposed convolution; ``(g_x or None, g_w or None)``.

    Same contract as ``conv_transpose_halo_nway_backward`` (distributed.py:260-283): the
    output gradient is gathered over the raw span, then the input gradient is a plain
    convolution of it and the weight gradient pairs it with the saved input."""
    n = config.n_spatial
    ranks, sizes = _mesh_position(spatial_groups)
    need_x, need_w = need[0], need[1]
    g = grad_output.to(weight.dtype).contiguous()
    geom = transpose_geometry(local_in_spatial, weight.shape[-n:], stride, padding, dilation, ranks, sizes)
    present = _present_offsets(geom, ranks, sizes)
    send = halo_pack(g, geom, from_padded=False, present=present) if present else {}
    recv = config.halo_exchange.backward(send) if present else {}
    g_raw = halo_assemble(g, recv, geom)
    kwargs = {"stride": stride, "padding": _local_padding(padding, sizes), "dilation": dilation, "groups": int(getattr(config, "groups_local", 1))}
    g_x = conv_nd(g_raw, weight, None, **kwargs) if need_x else None
    g_w = conv_nd_weight(g_raw, weight.shape, x_aug.to(weight.dtype), **kwargs) if need_w else None
    return g_x, g_w


class HipConvTransposeNdConfig(_HipLayerConfig):
    """Kernel table of one distributed transposed convolution layer: built like the
    reference's ``ConvTransposeNdConfig`` (_conv_transpose/config.py:47-84) and carrying
    the attributes the layer, ``_ConvTransposeNd`` and the two ``dist_conv_transpose_*``
    functions read from it, ``_layer_key`` included, plus ``halo_exchange``."""

    _OPTIONS = ("halo_exchange", "fused_fold")
    fused_fold = True

    def __init__(self, channel_group: Any, bias: Any, kernel_size, stride, device: Any = None,
                 channel_comm: Any = "auto", groups: int = 1, **options: Any) -> None:
        super().__init__(channel_group, bias, kernel_size, stride, device, channel_comm, groups, **options)
        self.conv_transpose_fn = conv_transpose_nd
        self.native_conv_transpose_fn = conv_transpose_nd
        self.dist_conv_transpose_fn = conv_transpose_halo_nway
        self.dist_conv_transpose_backward_fn = conv_transpose_halo_nway_backward


class _ConvTransposeNd(torch.autograd.Function):
    """Autograd function of the distributed transposed convolution
    (jigsaw/modules/convolution/_conv_transpose/functional.py), HIP kernels inside."""

    @staticmethod
    def forward(ctx, x, weight, bias, stride, padding, dilation, spatial_groups, channel_group, config):  # noqa: D102
        xc, wc, bc = _cast_to_autocast_dtype(x, weight, bias)
        y, x_aug = config.dist_conv_transpose_fn(
            xc, wc, bc, stride=stride, padding=padding, dilation=dilation, spatial_groups=spatial_groups,
            channel_group=channel_group, config=config,
        )
        ctx.mark_non_differentiable(x_aug)
        ctx.save_for_backward(x_aug, weight)
        ctx.spatial_groups, ctx.channel_group = spatial_groups, channel_group
        ctx.local_in_spatial = tuple(x.shape[-config.n_spatial :])
        ctx.stride, ctx.padding, ctx.dilation, ctx.config = stride, padding, dilation, config
        ctx.has_bias = bias is not None
        return y, x_aug

    @staticmethod
    def backward(ctx, grad_output, grad_x_aug):  # noqa: D102
        x_aug, weight = ctx.saved_tensors
        config = ctx.config
        need_x, need_w, need_b = ctx.needs_input_grad[:3]
        g_b = config.grad_bias(grad_output.contiguous()) if (need_b and ctx.has_bias) else None
        g_x, g_w = config.dist_conv_transpose_backward_fn(
            grad_output, x_aug, weight, ctx.stride, ctx.padding, ctx.dilation, ctx.local_in_spatial,
            ctx.spatial_groups, ctx.channel_group, config, need=(need_x, need_w),
        )
        return g_x, g_w, g_b, None, None, None, None, None, None


__all__ = [
    "HipConvTransposeNdConfig",
    "_ConvTransposeNd",
    "conv_transpose_halo_nway",
    "conv_transpose_halo_nway_backward",
    "conv_transpose_nd",
    "produced_output_span",
    "raw_span_widths",
    "transpose_geometry",
]
