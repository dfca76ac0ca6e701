"""GroupNorm over a spatially sharded input on the GPU.

Host-side mirror of ``_GroupNorm`` (jigsaw/modules/normalization/_functional.py:317-468):
same call signature ``apply(x, num_groups, weight, bias, spatial_groups, eps)`` and the
same four outputs ``(y, x_norm, rstd, n)``, so it can stand where
``DistributedGroupNorm.forward`` calls ``functional._GroupNorm.apply``
(jigsaw/modules/normalization/_group_norm.py:287-289). The per-(sample, group) partial
sums, the normalise + affine pass and the backward run in HIP kernels; the sum
all-reduces over the spatial process groups (one of (count, sum), one of the centred
squares; backward one of the two sums) stay here.
"""

from __future__ import annotations

from collections.abc import Sequence
from typing import Any

import torch
import torch.distributed as dist

from . import _lib


def _all_reduce_sum(t: torch.Tensor, groups: Sequence[Any]) -> None:
    """Sum ``t`` in place over every group in turn (_functional.py:311-314). A group is a
    ``torch.distributed`` process group or any object with ``size()`` and
    ``all_reduce(tensor, "sum")`` (a single-process stand-in that holds the other shards'
    contributions)."""
    for g in groups or ():
        if g is None or int(g.size()) == 1:
            continue
        if hasattr(g, "all_reduce"):
            g.all_reduce(t, "sum")
        else:
            dist.all_reduce(t, op=dist.ReduceOp.SUM, group=g)


def _compute_dtype(x: torch.Tensor) -> torch.dtype:
    # promote_to_fp32_under_autocast (jigsaw/_core/autocast.py:83-107)
    if torch.is_autocast_enabled() and x.dtype in (torch.float16, torch.bfloat16):
        return torch.float32
    return x.dtype


def _dims(x: torch.Tensor) -> tuple[int, int, int]:
    n, c = x.shape[0], x.shape[1]
    return n, c, (x.numel() // (n * c) if n * c else 0)


def _workspace(lib, n: int, c: int, s: int, dev) -> tuple[torch.Tensor, int]:
    nbytes = int(lib.jg_gn_workspace_bytes(n, c, s))
    return torch.empty(nbytes, dtype=torch.uint8, device=dev), nbytes


def partial_sum(x: torch.Tensor, num_groups: int) -> torch.Tensor:
    """fp32 ``(N, num_groups)`` sums of ``x`` over each group's channels and the local positions."""
    _lib.require_gpu(x)
    x = x.contiguous()
    n, c, s = _dims(x)
    lib = _lib.load()
    out = torch.empty(n, num_groups, dtype=torch.float32, device=x.device)
    ws, nbytes = _workspace(lib, n, c, s, x.device)
    rc = lib.jg_gn_partial_sum(_lib.ptr(out), _lib.ptr(x), n, c, s, num_groups, _lib.dtype_code(x.dtype),
                               _lib.ptr(ws), nbytes, _lib.stream_ptr(x.device))
    _lib.check(rc, "jg_gn_partial_sum")
    return out


def partial_sqdev(x: torch.Tensor, mean: torch.Tensor, num_groups: int) -> torch.Tensor:
    """fp32 ``(N, num_groups)`` sums of ``(x - mean)^2`` with the global ``mean (N, num_groups)``."""
    _lib.require_gpu(x, mean)
    x = x.contiguous()
    n, c, s = _dims(x)
    lib = _lib.load()
    mean = mean.to(torch.float32).contiguous()
    out = torch.empty(n, num_groups, dtype=torch.float32, device=x.device)
    ws, nbytes = _workspace(lib, n, c, s, x.device)
    rc = lib.jg_gn_partial_sqdev(_lib.ptr(out), _lib.ptr(x), _lib.ptr(mean), n, c, s, num_groups,
                                 _lib.dtype_code(x.dtype), _lib.ptr(ws), nbytes, _lib.stream_ptr(x.device))
    _lib.check(rc, "jg_gn_partial_sqdev")
    return out


class _GroupNorm(torch.autograd.Function):
    """Autograd function of the GroupNorm over a spatially sharded input (HIP kernels inside)."""

    @staticmethod
    def forward(ctx, x, num_groups, weight, bias, spatial_groups, eps):  # noqa: D102
        _lib.require_gpu(x, weight, bias)
        if x.shape[1] % num_groups != 0:
            raise ValueError(f"{x.shape[1]} channels do not divide into {num_groups} groups")
        cdt = _compute_dtype(x)
        x = x.to(cdt).contiguous()
        w = None if weight is None else weight.to(cdt).contiguous()
        b = None if bias is None else bias.to(cdt).contiguous()
        n, c, s = _dims(x)
        lib = _lib.load()
        dev = x.device

        # global count and sum per (sample, group) in one collective per process group
        local = partial_sum(x, num_groups)
        stats = torch.stack([torch.full_like(local, float(c // num_groups * s)), local], dim=-1)
        _all_reduce_sum(stats, spatial_groups)
        count, total = stats.unbind(dim=-1)
        mean = (total / count).contiguous()
        # centred on the global mean before squaring (two-pass variance)
        var = partial_sqdev(x, mean, num_groups)
        _all_reduce_sum(var, spatial_groups)
        rstd = torch.rsqrt(var / count + eps).contiguous()

        y = torch.empty_like(x)
        x_norm = torch.empty_like(x)
        rc = lib.jg_gn_apply(_lib.ptr(y), _lib.ptr(x_norm), _lib.ptr(x), _lib.ptr(mean), _lib.ptr(rstd),
                             _lib.ptr(w), _lib.ptr(b), n, c, s, num_groups, _lib.dtype_code(cdt),
                             _lib.stream_ptr(dev))
        _lib.check(rc, "jg_gn_apply")

        count = count.contiguous()
        ctx.num_groups = num_groups
        ctx.spatial_groups = spatial_groups
        ctx.has_weight, ctx.has_bias = weight is not None, bias is not None
        ctx.dtypes = (None if weight is None else weight.dtype, None if bias is None else bias.dtype)
        ctx.save_for_backward(x_norm, rstd, count, w)
        rstd_out, n_out = rstd.unsqueeze(-1).to(cdt), count.unsqueeze(-1).to(cdt)
        ctx.mark_non_differentiable(x_norm, rstd_out, n_out)
        return y, x_norm, rstd_out, n_out

    @staticmethod
    def backward(ctx, grad_output, x_norm_grad, rstd_grad, n_grad):  # noqa: D102
        x_norm, rstd, count, w = ctx.saved_tensors
        g = grad_output.to(x_norm.dtype).contiguous()
        n, c, s = _dims(x_norm)
        groups = ctx.num_groups
        lib = _lib.load()
        dev = g.device
        need_x = ctx.needs_input_grad[0]
        need_w = ctx.has_weight and ctx.needs_input_grad[2]
        need_b = ctx.has_bias and ctx.needs_input_grad[3]

        gsum = torch.empty(n, groups, dtype=torch.float32, device=dev)
        gxsum = torch.empty_like(gsum)
        gw = torch.empty(c, dtype=torch.float32, device=dev) if need_w else None
        gb = torch.empty(c, dtype=torch.float32, device=dev) if need_b else None
        ws, nbytes = _workspace(lib, n, c, s, dev)
        rc = lib.jg_gn_partial_bwd(_lib.ptr(gsum), _lib.ptr(gxsum), _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(g),
                                   _lib.ptr(x_norm), _lib.ptr(w), n, c, s, groups, _lib.dtype_code(g.dtype),
                                   _lib.ptr(ws), nbytes, _lib.stream_ptr(dev))
        _lib.check(rc, "jg_gn_partial_bwd")

        grad_x = None
        if need_x:
            # both per-group reductions in one collective per process group
            sums = torch.stack([gsum, gxsum], dim=-1)
            _all_reduce_sum(sums, ctx.spatial_groups)
            gsum, gxsum = (t.contiguous() for t in sums.unbind(dim=-1))
            grad_x = torch.empty_like(g)
            rc = lib.jg_gn_bwd_apply(_lib.ptr(grad_x), _lib.ptr(g), _lib.ptr(x_norm), _lib.ptr(w), _lib.ptr(rstd),
                                     _lib.ptr(gsum), _lib.ptr(gxsum), _lib.ptr(count), n, c, s, groups,
                                     _lib.dtype_code(g.dtype), _lib.stream_ptr(dev))
            _lib.check(rc, "jg_gn_bwd_apply")
        # the weight and bias gradients are local; the layer sums them over its replicas
        dt_w, dt_b = ctx.dtypes
        return (grad_x, None, gw.to(dt_w) if need_w else None, gb.to(dt_b) if need_b else None, None, None)


def group_norm(x, num_groups, weight=None, bias=None, spatial_groups=(), eps=1e-5):
    """``_GroupNorm.apply(...)[0]``, the call of ``DistributedGroupNorm.forward``."""
    return _GroupNorm.apply(x, num_groups, weight, bias, spatial_groups, eps)[0]


__all__ = ["_GroupNorm", "group_norm", "partial_sqdev", "partial_sum"]
