"""Sharded LayerNorm on the GPU.

Host-side mirror of ``_LayerNorm`` (jigsaw/modules/normalization/_functional.py:13-177):
same call signature ``apply(x, weight, bias, channel_group, eps)`` and the same
four outputs, so it can be assigned to ``DistributedLayerNorm.layernorm``
(jigsaw/modules/normalization/_layer_norm.py:90-94). The partial statistics, the
normalise + affine epilogue and the backward partials run in HIP kernels; the
two all-reduces per direction over the channel group stay here.
"""

from __future__ import annotations

from typing import Any

import torch
import torch.distributed as dist

from . import _lib


def _group_size(group: Any) -> int:
    if group is None:
        return 1
    return int(group.size())


def _all_reduce(t: torch.Tensor, op: str, group: Any) -> None:
    """AVG / SUM all-reduce of ``t`` over the channel group, in place.

    ``group`` is a ``torch.distributed`` process group, ``None`` (no sharding), or
    any object with ``size()`` and ``all_reduce(tensor, op)`` (a single-process
    stand-in that already holds the other shards' contributions).
    """
    if _group_size(group) == 1:
        return
    if hasattr(group, "all_reduce"):
        group.all_reduce(t, op)
        return
    red = dist.ReduceOp.AVG if op == "avg" else dist.ReduceOp.SUM
    dist.all_reduce(t, op=red, group=group)


def partial_stats(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 ``(mean, biased var)`` over the last (local) axis, shape ``(..., 1)``."""
    _lib.require_gpu(x)
    x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    mean = torch.empty(x.shape[:-1] + (1,), dtype=torch.float32, device=x.device)
    var = torch.empty_like(mean)
    rc = _lib.load().jg_ln_partial_fwd(
        _lib.ptr(mean), _lib.ptr(var), _lib.ptr(x), rows, cols, _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device)
    )
    _lib.check(rc, "jg_ln_partial_fwd")
    return mean, var


def _compute_dtype(x: torch.Tensor) -> torch.dtype:
    # promote_to_fp32_under_autocast (jigsaw/_core/autocast.py:83-107): norms run in
    # fp32 when autocast is on, otherwise in the input dtype.
    if torch.is_autocast_enabled():
        return torch.float32
    return x.dtype


class _LayerNorm(torch.autograd.Function):
    """Autograd function of the distributed LayerNorm (HIP kernels inside)."""

    @staticmethod
    def forward(x, weight, bias, channel_group, eps):  # noqa: D102
        _lib.require_gpu(x, weight, bias)
        cdt = _compute_dtype(x)
        x = x.contiguous()
        w = weight.to(cdt).contiguous()
        b = None if bias is None else bias.to(cdt).contiguous()
        cols = x.shape[-1]
        rows = x.numel() // cols
        local_mean, local_var = partial_stats(x)

        mean = local_mean.clone()
        _all_reduce(mean, "avg", channel_group)
        var = local_var + (local_mean - mean) ** 2 if _group_size(channel_group) > 1 else local_var
        _all_reduce(var, "avg", channel_group)

        y = torch.empty(x.shape, dtype=cdt, device=x.device)
        x_norm = torch.empty_like(y)
        rc = _lib.load().jg_ln_apply(
            _lib.ptr(y), _lib.ptr(x_norm), None, _lib.ptr(x), _lib.ptr(mean), _lib.ptr(var),
            _lib.ptr(w), _lib.ptr(b), rows, cols, float(eps),
            _lib.dtype_code(x.dtype), _lib.dtype_code(cdt), _lib.stream_ptr(x.device),
        )
        _lib.check(rc, "jg_ln_apply")
        # an input returned as-is cannot be saved by setup_context: hand out a view
        return y, x_norm, (w.view_as(w) if w is weight else w), (var + eps).to(cdt)

    @staticmethod
    def setup_context(ctx, inputs, output):  # noqa: D102
        x, weight, bias, channel_group, eps = inputs
        _, x_norm, w, var = output
        ctx.mark_non_differentiable(x_norm, w, var)
        ctx.channel_group = channel_group
        ctx.has_bias = bias is not None
        ctx.param_dtypes = (weight.dtype, None if bias is None else bias.dtype)
        ctx.in_dtype = x.dtype
        # sqrt(var + eps), as the reference saves it (_functional.py:75); fp32 for the kernels
        ctx.save_for_backward(x_norm, w, torch.sqrt(var.to(torch.float32)))

    @staticmethod
    def backward(ctx, grad_output, x_norm_grad, weight_grad, var_grad):  # noqa: D102
        x_norm, w, std = ctx.saved_tensors
        g = grad_output.to(x_norm.dtype).contiguous()
        group = ctx.channel_group
        cols = x_norm.shape[-1]
        rows = x_norm.numel() // cols
        n_global = cols * _group_size(group)
        lib = _lib.load()
        dev = g.device

        mean_gxn = torch.empty_like(std)
        dot = torch.empty_like(std)
        need_w = ctx.needs_input_grad[1]
        need_b = ctx.has_bias and ctx.needs_input_grad[2]
        gw = torch.empty(cols, dtype=torch.float32, device=dev) if need_w else None
        gb = torch.empty(cols, dtype=torch.float32, device=dev) if need_b else None
        ws_bytes = int(lib.jg_ln_bwd_workspace_bytes(rows, cols)) if (need_w or need_b) else 0
        ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=dev)
        rc = lib.jg_ln_partial_bwd(
            _lib.ptr(mean_gxn), _lib.ptr(dot), _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(g), _lib.ptr(x_norm),
            _lib.ptr(w), rows, cols, _lib.dtype_code(g.dtype), _lib.ptr(ws), ws_bytes, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "jg_ln_partial_bwd")

        grad_x = None
        if ctx.needs_input_grad[0]:
            _all_reduce(mean_gxn, "avg", group)
            _all_reduce(dot, "sum", group)
            grad_x = torch.empty_like(g)
            rc = lib.jg_ln_bwd_apply(
                _lib.ptr(grad_x), _lib.ptr(g), _lib.ptr(x_norm), _lib.ptr(w), _lib.ptr(mean_gxn), _lib.ptr(dot),
                _lib.ptr(std), rows, cols, n_global, _lib.dtype_code(g.dtype), _lib.stream_ptr(dev),
            )
            _lib.check(rc, "jg_ln_bwd_apply")
            grad_x = grad_x.to(ctx.in_dtype)
        wdt, bdt = ctx.param_dtypes
        grad_w = gw.to(wdt) if need_w else None
        grad_b = gb.to(bdt) if need_b else None
        return grad_x, grad_w, grad_b, None, None


def layer_norm(x, weight, bias, channel_group=None, eps: float = 1e-5) -> torch.Tensor:
    """``DistributedLayerNorm.forward``'s call: ``_LayerNorm.apply(...)[0]``
    (jigsaw/modules/normalization/_layer_norm.py:363-368)."""
    return _LayerNorm.apply(x, weight, bias, channel_group, eps)[0]


class _PlainLayerNorm(torch.autograd.Function):
    """``nn.LayerNorm`` over rows one rank holds whole: one fused kernel forward, one backward
    (plus the column reduction) that recomputes ``x_hat`` from ``(x, mean, rstd)``."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps, out_dtype):  # noqa: D102
        _lib.require_gpu(x, weight, bias)
        xc = x.contiguous()
        cols = xc.shape[-1]
        rows = xc.numel() // cols
        w = weight.to(torch.float32).contiguous()
        b = None if bias is None else bias.to(torch.float32).contiguous()
        y = torch.empty(xc.shape, dtype=out_dtype, device=x.device)
        mean = torch.empty(rows, dtype=torch.float32, device=x.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
        rc = _lib.load().jg_ln_plain_fwd(_lib.ptr(y), _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(xc), _lib.ptr(w), _lib.ptr(b),
                                         rows, cols, float(eps), _lib.dtype_code(xc.dtype), _lib.dtype_code(out_dtype),
                                         _lib.stream_ptr(x.device))
        _lib.check(rc, "jg_ln_plain_fwd")
        ctx.save_for_backward(xc, mean, rstd, w)
        ctx.has_bias = bias is not None
        ctx.param_dtypes = (weight.dtype, None if bias is None else bias.dtype)
        return y

    @staticmethod
    def backward(ctx, grad, past=None):  # noqa: D102
        xc, mean, rstd, w = ctx.saved_tensors
        cols = xc.shape[-1]
        rows = xc.numel() // cols
        g = grad.contiguous()
        if g.dtype != xc.dtype and torch.float32 not in (g.dtype, xc.dtype):
            g = g.to(xc.dtype)
        dev = g.device
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_b = ctx.has_bias and ctx.needs_input_grad[2]
        gx = torch.empty_like(xc) if need_x else None
        gw = torch.empty(cols, dtype=torch.float32, device=dev) if need_w else None
        gb = torch.empty(cols, dtype=torch.float32, device=dev) if need_b else None
        lib = _lib.load()
        nbytes = int(lib.jg_ln_plain_bwd_workspace_bytes(rows, cols)) if (need_w or need_b) else 0
        ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev)
        if past is not None and need_x:
            past = past.to(xc.dtype).contiguous()
            rc = lib.jg_ln_plain_bwd_add(_lib.ptr(gx), _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(g), _lib.ptr(xc), _lib.ptr(mean),
                                         _lib.ptr(rstd), _lib.ptr(w), rows, cols, _lib.dtype_code(g.dtype),
                                         _lib.dtype_code(xc.dtype), _lib.ptr(ws), nbytes, _lib.ptr(past), _lib.stream_ptr(dev))
            _lib.check(rc, "jg_ln_plain_bwd_add")
        else:
            rc = lib.jg_ln_plain_bwd(_lib.ptr(gx), _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(g), _lib.ptr(xc), _lib.ptr(mean),
                                     _lib.ptr(rstd), _lib.ptr(w), rows, cols, _lib.dtype_code(g.dtype), _lib.dtype_code(xc.dtype),
                                     _lib.ptr(ws), nbytes, _lib.stream_ptr(dev))
            _lib.check(rc, "jg_ln_plain_bwd")
        wdt, bdt = ctx.param_dtypes
        return gx, (gw.to(wdt) if need_w else None), (gb.to(bdt) if need_b else None), None, None


class _PlainLayerNormFork(torch.autograd.Function):
    """``(LayerNorm(x), x)``: the normalised rows for a branch and the rows themselves for the
    residual connection around it (``x + f(norm(x))``, examples/swin.py:206-209). The backward adds
    the gradient that arrives over the connection inside the LayerNorm backward kernel, where
    autograd would otherwise add the two gradient tensors of ``x`` in a pass of its own."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps, out_dtype):  # noqa: D102
        y = _PlainLayerNorm.forward(ctx, x, weight, bias, eps, out_dtype)
        return y, x.view_as(x)

    @staticmethod
    def backward(ctx, grad, past):  # noqa: D102
        if grad is None:  # the branch was not used
            return past, None, None, None, None
        return _PlainLayerNorm.backward(ctx, grad, past)


def plain_layer_norm_fork(x, weight, bias, eps: float = 1e-5, out_dtype: torch.dtype | None = None):
    """``(plain_layer_norm(x, ...), x)`` for a pre-norm residual block: use the second result where
    the block adds ``x`` back, and the sum of the two gradients of ``x`` is formed inside the
    LayerNorm backward (see :class:`_PlainLayerNormFork`). Falls back to the two separate results
    where :func:`plain_layer_norm` itself does."""
    odt = out_dtype or _compute_dtype(x)
    if x.numel() == 0 or not _lib.load().jg_ln_plain_supported(x.shape[-1]):
        return plain_layer_norm(x, weight, bias, eps, out_dtype), x
    return _PlainLayerNormFork.apply(x, weight, bias, eps, odt)


def plain_layer_norm(x, weight, bias, eps: float = 1e-5, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``F.layer_norm(x, (x.shape[-1],), weight, bias, eps)`` for rows that are not split over a
    channel group (the ``nn.LayerNorm`` of examples/swin.py:186-188). ``out_dtype`` defaults to
    what torch yields: fp32 under autocast, else ``x.dtype``; a caller whose next layer rounds to the
    autocast dtype anyway may ask for that dtype here and save the fp32 round trip. Widths the fused
    kernels do not take (not a multiple of 8, above 2048) go through :func:`layer_norm`."""
    odt = out_dtype or _compute_dtype(x)
    if x.numel() == 0:  # nothing to launch; torch keeps the (empty) graph connected
        return torch.nn.functional.layer_norm(x.to(odt), x.shape[-1:], weight.to(odt),
                                              None if bias is None else bias.to(odt), eps)
    if not _lib.load().jg_ln_plain_supported(x.shape[-1]):
        return layer_norm(x, weight, bias, None, eps).to(odt)
    return _PlainLayerNorm.apply(x, weight, bias, eps, odt)


__all__ = ["_LayerNorm", "layer_norm", "partial_stats", "plain_layer_norm", "plain_layer_norm_fork"]
