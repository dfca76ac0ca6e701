"""Token projections around the attention core with the head split / merge fused in.

Host-side mirror of the pre- and post-processing of ``DistributedAttention.forward``
(jigsaw/modules/attention/_attention.py:881-918):

* :func:`qkv_projection` stands for ``self.qkv(x)`` followed by
  ``rearrange(qkv, "... n s (three h d) -> three ... n h s d")``: the GEMM writes q, k
  and v straight into their ``(..., h, s, d)`` places, no rearrange copy;
* :func:`heads_projection` stands for
  ``rearrange(out, "... n h s d -> ... n s (h d)").contiguous()`` followed by
  ``self.head_concat(out)``: the GEMM reads the attention output where it lies.

Both are ``autograd`` functions; their backward reads and writes the head layouts the
same way (input gradient: the same GEMM with the transposed weight; weight and bias
gradient: one GEMM contracted over the tokens). The weights are the rank's local
``nn.Linear`` parameters ``(out_features, in_features)``.
"""

from __future__ import annotations

import contextlib
import math

import torch

from . import _lib


def _nt(out, a, w, bias, rows, n_out, k_in, a_heads, out_heads, dims) -> None:
    lib = _lib.load()
    b, h, s, d = dims
    rc = lib.jg_proj_nt(_lib.ptr(out), _lib.ptr(a), _lib.ptr(w), _lib.ptr(bias), _lib.dtype_code(a.dtype), rows, n_out,
                        k_in, int(a_heads), int(out_heads), b, h, s, d, _lib.stream_ptr(a.device))
    _lib.check(rc, "jg_proj_nt")


_remember_casts = False


def remember_casts(on: bool = True) -> bool:
    """Switch the remembering of parameter casts on or off for the process; returns the previous setting.

    Off (the default), every forward casts the fp32 parameters to the compute dtype anew and every
    backward transposes the saved cast: always right. On, the copies are kept on the parameter and reused
    until the parameter changes, which saves a dozen small launches per Swin block step. A change is
    recognised by the tensor's version counter (every in-place operation on the parameter itself, an
    optimizer step included, bumps it) and by its storage address, device and dtype. A write through
    ``param.data`` (``p.data.normal_()``, ``dist.broadcast(p.data, ...)``, an EMA swap that copies into
    ``p.data``) bumps no counter and keeps the address: after such a write call :func:`invalidate_casts`
    on the module or parameter, or leave remembering off."""
    global _remember_casts
    before, _remember_casts = _remember_casts, bool(on)
    return before


def invalidate_casts(*targets) -> None:
    """Drop the remembered casts of the given parameters / tensors or of every parameter and buffer of the
    given modules (after a write through ``.data``, which the version counter does not see)."""
    for t in targets:
        if isinstance(t, torch.nn.Module):
            invalidate_casts(*t.parameters(), *t.buffers())
        elif isinstance(t, torch.Tensor) and getattr(t, "_jg_casts", None) is not None:
            try:
                del t._jg_casts
            except AttributeError:
                pass


@contextlib.contextmanager
def fresh_casts():
    """Inside, the casts of the parameters are made anew and not remembered: for work that is recorded
    in a HIP graph, where a remembered copy would be read at every replay in place of the parameter."""
    global _remember_casts
    before, _remember_casts = _remember_casts, False
    try:
        yield
    finally:
        _remember_casts = before


def _cast_key(t: torch.Tensor) -> tuple:
    return (t._version, t.data_ptr(), t.device, t.dtype, tuple(t.shape), tuple(t.stride()))


def _cast_cached(t: torch.Tensor | None, dtype: torch.dtype, transposed: bool = False) -> torch.Tensor | None:
    """``t`` in ``dtype``, contiguous (optionally its transpose). With :func:`remember_casts` on, the copy is
    kept on the tensor until its version counter, storage address, device, dtype or layout changes: under
    autocast the parameters are fp32 and every forward and backward would otherwise launch a cast (and the
    input gradient a transpose copy) per layer."""
    if t is None:
        return None
    if not transposed and t.dtype == dtype and t.is_contiguous():
        return t
    if not _remember_casts:
        src = t.detach()
        return (src.t() if transposed else src).to(dtype).contiguous()
    key = (dtype, transposed)
    cache = getattr(t, "_jg_casts", None)
    stamp = _cast_key(t)
    if cache is None or cache[0] != stamp:
        cache = (stamp, {})
        try:
            t._jg_casts = cache
        except AttributeError:  # a tensor subclass without a __dict__: no cache
            pass
    got = cache[1].get(key)
    if got is None:
        src = t.detach()
        got = (src.t() if transposed else src).to(dtype).contiguous()
        cache[1][key] = got
    return got


def _transposed(ctx, w: torch.Tensor) -> torch.Tensor:
    """The transposed weight of the input-gradient GEMM: the remembered copy of the parameter when casts
    are remembered and the parameter is still the one the forward saw, else a transpose of the saved cast."""
    ref = getattr(ctx, "weight_ref", None)
    if _remember_casts and ref is not None and ref._version == ctx.weight_version:
        return _cast_cached(ref, w.dtype, transposed=True)
    return w.t().contiguous()


def _grad_dtype(compute: torch.dtype, dtypes) -> torch.dtype:
    """fp32 when every parameter that gets a gradient is fp32 (autocast), else the compute dtype."""
    return torch.float32 if all(dt in (None, torch.float32) for dt in dtypes) else compute


def _tn(g, x, rows, n, c, g_heads, x_heads, dims, want_bias, grad_dtype=None):
    lib = _lib.load()
    b, h, s, d = dims
    gdt = grad_dtype or g.dtype
    gw = torch.empty(n, c, dtype=gdt, device=g.device)
    gb = torch.empty(n, dtype=gdt, device=g.device) if want_bias else None
    nbytes = int(lib.jg_proj_tn_workspace(rows, n, c))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=g.device)
    rc = lib.jg_proj_tn(_lib.ptr(gw), _lib.ptr(gb), _lib.ptr(g), _lib.ptr(x), _lib.dtype_code(g.dtype),
                        _lib.dtype_code(gdt), rows, n, c,
                        int(g_heads), int(x_heads), b, h, s, d, _lib.ptr(ws), nbytes, _lib.stream_ptr(g.device))
    _lib.check(rc, "jg_proj_tn")
    return gw, gb


class _QkvProjection(torch.autograd.Function):
    """``(*lead, s, C) -> (3, *lead, h, s, d)`` with ``weight (3 h d, C)``."""

    @staticmethod
    def forward(ctx, x, weight, bias, heads):  # noqa: D102
        _lib.require_gpu(x, weight, bias)
        if x.dim() < 2:
            raise ValueError("x must be (..., seq, channels)")
        n_out, c = weight.shape
        if x.shape[-1] != c:
            raise ValueError(f"x has {x.shape[-1]} channels, the weight takes {c}")
        if n_out % (3 * heads) != 0:
            raise ValueError(f"{n_out} output features do not split into 3 x {heads} heads")
        d = n_out // (3 * heads)
        lead, s = tuple(x.shape[:-2]), x.shape[-2]
        b = math.prod(lead)
        xc = x.contiguous()
        w = _cast_cached(weight, x.dtype)
        bs = _cast_cached(bias, x.dtype)
        out = torch.empty((3, *lead, heads, s, d), dtype=x.dtype, device=x.device)
        if b * s:
            _nt(out, xc, w, bs, b * s, n_out, c, False, True, (b, heads, s, d))
        ctx.save_for_backward(xc, w)
        ctx.weight_ref, ctx.weight_version = weight, weight._version
        ctx.dims = (b, heads, s, d)
        ctx.has_bias = bias is not None
        ctx.dtypes = (weight.dtype, None if bias is None else bias.dtype)
        return out

    @staticmethod
    def backward(ctx, grad):  # noqa: D102
        xc, w = ctx.saved_tensors
        b, h, s, d = ctx.dims
        n_out, c = w.shape
        g = grad.to(xc.dtype).contiguous()
        gx = gw = gb = None
        if b * s == 0:
            gx = torch.zeros_like(xc) if ctx.needs_input_grad[0] else None
            gw = torch.zeros_like(w) if ctx.needs_input_grad[1] else None
            gb = torch.zeros(n_out, dtype=w.dtype, device=w.device) if ctx.has_bias and ctx.needs_input_grad[2] else None
        else:
            if ctx.needs_input_grad[0]:
                gx = torch.empty_like(xc)
                _nt(gx, g, _transposed(ctx, w), None, b * s, c, n_out, True, False, ctx.dims)
            need_b = ctx.has_bias and ctx.needs_input_grad[2]
            if ctx.needs_input_grad[1] or need_b:
                gw, gb = _tn(g, xc, b * s, n_out, c, True, False, ctx.dims, need_b, _grad_dtype(g.dtype, ctx.dtypes))
        dt_w, dt_b = ctx.dtypes
        return (gx, None if gw is None or not ctx.needs_input_grad[1] else gw.to(dt_w),
                None if gb is None else gb.to(dt_b), None)


class _HeadsProjection(torch.autograd.Function):
    """``(*lead, h, s, d) -> (*lead, s, n_out)`` with ``weight (n_out, h d)``."""

    @staticmethod
    def forward(ctx, out, weight, bias):  # noqa: D102
        _lib.require_gpu(out, weight, bias)
        if out.dim() < 3:
            raise ValueError("out must be (..., heads, seq, head_dim)")
        n_out, k = weight.shape
        h, s, d = out.shape[-3:]
        if h * d != k:
            raise ValueError(f"heads x head_dim = {h * d}, the weight takes {k}")
        lead = tuple(out.shape[:-3])
        b = math.prod(lead)
        oc = out.contiguous()
        w = _cast_cached(weight, out.dtype)
        bs = _cast_cached(bias, out.dtype)
        y = torch.empty((*lead, s, n_out), dtype=out.dtype, device=out.device)
        if b * s:
            _nt(y, oc, w, bs, b * s, n_out, k, True, False, (b, h, s, d))
        ctx.save_for_backward(oc, w)
        ctx.weight_ref, ctx.weight_version = weight, weight._version
        ctx.dims = (b, h, s, d)
        ctx.has_bias = bias is not None
        ctx.dtypes = (weight.dtype, None if bias is None else bias.dtype)
        return y

    @staticmethod
    def backward(ctx, grad):  # noqa: D102
        oc, w = ctx.saved_tensors
        b, h, s, d = ctx.dims
        n_out, k = w.shape
        g = grad.to(oc.dtype).contiguous()
        go = gw = gb = None
        if b * s == 0:
            go = torch.zeros_like(oc) if ctx.needs_input_grad[0] else None
            gw = torch.zeros_like(w) if ctx.needs_input_grad[1] else None
            gb = torch.zeros(n_out, dtype=w.dtype, device=w.device) if ctx.has_bias and ctx.needs_input_grad[2] else None
        else:
            if ctx.needs_input_grad[0]:
                go = torch.empty_like(oc)
                _nt(go, g, _transposed(ctx, w), None, b * s, k, n_out, False, True, ctx.dims)
            need_b = ctx.has_bias and ctx.needs_input_grad[2]
            if ctx.needs_input_grad[1] or need_b:
                gw, gb = _tn(g, oc, b * s, n_out, k, False, True, ctx.dims, need_b, _grad_dtype(g.dtype, ctx.dtypes))
        dt_w, dt_b = ctx.dtypes
        return (go, None if gw is None or not ctx.needs_input_grad[1] else gw.to(dt_w),
                None if gb is None else gb.to(dt_b))


class _Linear(torch.autograd.Function):
    """``(*lead, k) -> (*lead, n)`` with ``weight (n, k)``: ``F.linear`` on the same GEMM kernels,
    the bias gradient summed inside the weight-gradient GEMM."""

    @staticmethod
    def forward(ctx, x, weight, bias):  # noqa: D102
        _lib.require_gpu(x, weight, bias)
        n_out, k = weight.shape
        if x.dim() < 1 or x.shape[-1] != k:
            raise ValueError(f"x has {x.shape[-1] if x.dim() else 0} features, the weight takes {k}")
        xc = x.contiguous()
        rows = xc.numel() // k
        w = _cast_cached(weight, x.dtype)
        bs = _cast_cached(bias, x.dtype)
        y = torch.empty((*x.shape[:-1], n_out), dtype=x.dtype, device=x.device)
        if rows:
            _nt(y, xc, w, bs, rows, n_out, k, False, False, (1, 1, 1, 1))
        ctx.save_for_backward(xc, w)
        ctx.weight_ref, ctx.weight_version = weight, weight._version
        ctx.has_bias = bias is not None
        ctx.dtypes = (weight.dtype, None if bias is None else bias.dtype)
        return y

    @staticmethod
    def backward(ctx, grad):  # noqa: D102
        xc, w = ctx.saved_tensors
        n_out, k = w.shape
        rows = xc.numel() // k
        g = grad.to(xc.dtype).contiguous()
        gx = gw = gb = None
        need_b = ctx.has_bias and ctx.needs_input_grad[2]
        if rows == 0:
            gx = torch.zeros_like(xc) if ctx.needs_input_grad[0] else None
            gw = torch.zeros_like(w) if ctx.needs_input_grad[1] else None
            gb = torch.zeros(n_out, dtype=w.dtype, device=w.device) if need_b else None
        else:
            if ctx.needs_input_grad[0]:
                gx = torch.empty_like(xc)
                _nt(gx, g, _transposed(ctx, w), None, rows, k, n_out, False, False, (1, 1, 1, 1))
            if ctx.needs_input_grad[1] or need_b:
                gw, gb = _tn(g, xc, rows, n_out, k, False, False, (1, 1, 1, 1), need_b, _grad_dtype(g.dtype, ctx.dtypes))
        dt_w, dt_b = ctx.dtypes
        return (gx, None if gw is None or not ctx.needs_input_grad[1] else gw.to(dt_w),
                None if gb is None else gb.to(dt_b))


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` in ``x.dtype`` on this package's GEMM kernels (the MLP and any
    other token-wise layer around the attention core); its backward forms the weight and the bias
    gradient in one pass over the output gradient."""
    return _Linear.apply(x, weight, bias)


EPI_GELU, EPI_DGELU, EPI_ADD = 1, 2, 3


def _nt_fused(out, aux, epilogue, a, w, bias, rows, n_out, k_in) -> None:
    rc = _lib.load().jg_proj_nt_fused(_lib.ptr(out), _lib.ptr(aux), epilogue, _lib.ptr(a), _lib.ptr(w), _lib.ptr(bias),
                                      _lib.dtype_code(a.dtype), rows, n_out, k_in, _lib.stream_ptr(a.device))
    _lib.check(rc, "jg_proj_nt_fused")


def mlp_fusable(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, residual: torch.Tensor | None) -> bool:
    """Whether :func:`gelu_mlp` runs on the fused epilogues: bf16 tokens, feature counts that are
    multiples of 8 (16-byte rows), a bf16 residual of the output's shape."""
    ok = x.dtype == torch.bfloat16 and x.numel() > 0 and all(n % 8 == 0 for n in (*w1.shape, *w2.shape))
    return ok and (residual is None or (residual.dtype == torch.bfloat16 and residual.shape[:-1] == x.shape[:-1]))


class _GeluMlp(torch.autograd.Function):
    """``residual + F.linear(F.gelu(F.linear(x, w1, b1)), w2, b2)`` (examples/swin.py:190-194 with the
    residual sum of 206-209) as four GEMM launches forward and backward apart from the weight
    gradients: GELU leaves the first GEMM beside the pre-activation, the residual is added on the way
    out of the second, and in the backward the GELU derivative multiplies the input gradient of the
    second layer on its way out."""

    @staticmethod
    def forward(ctx, x, w1, b1, w2, b2, residual):  # noqa: D102
        _lib.require_gpu(x, w1, b1, w2, b2, residual)
        hid, k = w1.shape
        n_out = w2.shape[0]
        xc = x.contiguous()
        rows = xc.numel() // k
        dt = x.dtype
        w1c, b1c, w2c, b2c = (_cast_cached(t, dt) for t in (w1, b1, w2, b2))
        pre = torch.empty((*x.shape[:-1], hid), dtype=dt, device=x.device)
        act = torch.empty_like(pre)
        _nt_fused(pre, act, EPI_GELU, xc, w1c, b1c, rows, hid, k)
        out = torch.empty((*x.shape[:-1], n_out), dtype=dt, device=x.device)
        if residual is None:
            _nt(out, act, w2c, b2c, rows, n_out, hid, False, False, (1, 1, 1, 1))
        else:
            _nt_fused(out, residual.contiguous(), EPI_ADD, act, w2c, b2c, rows, n_out, hid)
        ctx.save_for_backward(xc, pre, act, w1c, w2c)
        ctx.refs = ((w1, w1._version), (w2, w2._version))
        ctx.dtypes = tuple(None if t is None else t.dtype for t in (w1, b1, w2, b2))
        ctx.has_residual = residual is not None
        return out

    @staticmethod
    def backward(ctx, grad):  # noqa: D102
        xc, pre, act, w1c, w2c = ctx.saved_tensors
        hid, k = w1c.shape
        n_out = w2c.shape[0]
        rows = xc.numel() // k
        g = grad.to(xc.dtype).contiguous()
        dt_w1, dt_b1, dt_w2, dt_b2 = ctx.dtypes

        def transposed(i, wc):
            ref, version = ctx.refs[i]
            return _cast_cached(ref, wc.dtype, transposed=True) if _remember_casts and ref._version == version else wc.t().contiguous()

        gw2, gb2 = _tn(g, act, rows, n_out, hid, False, False, (1, 1, 1, 1), dt_b2 is not None,
                       _grad_dtype(g.dtype, (dt_w2, dt_b2)))
        dpre = torch.empty_like(pre)  # dL/d(pre-activation) = (g W2) * gelu'(pre)
        _nt_fused(dpre, pre, EPI_DGELU, g, transposed(1, w2c), None, rows, hid, n_out)
        gw1, gb1 = _tn(dpre, xc, rows, hid, k, False, False, (1, 1, 1, 1), dt_b1 is not None,
                       _grad_dtype(g.dtype, (dt_w1, dt_b1)))
        gx = None
        if ctx.needs_input_grad[0]:
            gx = torch.empty_like(xc)
            _nt(gx, dpre, transposed(0, w1c), None, rows, k, hid, False, False, (1, 1, 1, 1))
        return (gx, gw1.to(dt_w1), None if gb1 is None else gb1.to(dt_b1), gw2.to(dt_w2),
                None if gb2 is None else gb2.to(dt_b2), g if ctx.has_residual else None)


def gelu_mlp(x, w1, b1, w2, b2, residual=None):
    """``(residual +) linear(gelu(linear(x, w1, b1)), w2, b2)``; GELU, its derivative and the residual
    sum ride on the GEMMs when :func:`mlp_fusable`, else the same from separate steps."""
    if mlp_fusable(x, w1, w2, residual):
        return _GeluMlp.apply(x, w1, b1, w2, b2, residual)
    y = linear(torch.nn.functional.gelu(linear(x, w1, b1)), w2, b2)
    return y if residual is None else residual + y.to(residual.dtype)


def qkv_projection(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, heads: int) -> torch.Tensor:
    """``rearrange(F.linear(x, weight, bias), "... s (three h d) -> three ... h s d", three=3, h=heads)``
    without the intermediate ``(..., s, 3 h d)`` tensor (_attention.py:881-890)."""
    return _QkvProjection.apply(x, weight, bias, heads)


def heads_projection(out: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``F.linear(rearrange(out, "... h s d -> ... s (h d)"), weight, bias)`` without the
    contiguous copy of the rearranged tensor (_attention.py:909-916)."""
    return _HeadsProjection.apply(out, weight, bias)


__all__ = ["gelu_mlp", "heads_projection", "invalidate_casts", "linear", "mlp_fusable", "qkv_projection", "remember_casts"]
