"""Ring-attention step on the GPU: attention core, log-sum-exp merge, ring loops.

Host-side mirror of

* the attention-core contract ``forward(q, k, v, scale, dropout_p, seed=None, *,
  layout) -> (out, logsumexp, rng_state)`` and ``backward(grad_out, q, k, v, out,
  logsumexp, scale, *extra, ...) -> (dq, dk, dv)``
  (jigsaw/modules/attention/_functional/cores/__init__.py:1-15), i.e. what
  ``RingAttentionConfig.attn_core_forward_fn / attn_core_backward_fn`` hold
  (jigsaw/modules/attention/_config.py:459-464);
* the fused merge hook ``fused_online_softmax_merge_``
  (jigsaw/modules/attention/_functional/_merge_kernel.py:88-172);
* the per-rank loops of ``ring_forward`` / ``ring_backward``
  (jigsaw/modules/attention/_functional/forward.py:160-199, backward.py:176-270)
  over K/V chunks that are already local. Circulating the chunks between ranks is
  outside this module.
"""

from __future__ import annotations

import ctypes
import math
from collections.abc import Sequence

import torch

from . import _lib

_SUPPORTED_O = (torch.float16, torch.bfloat16, torch.float32)


# --------------------------------------------------------------------------- #
# merge hook
# --------------------------------------------------------------------------- #
def fused_online_softmax_merge_(o1, l1, o2, l2, layout):
    """HIP stand-in for the Triton merge: mutates ``o1``, returns ``(o1, l_new)``.

    Returns ``None`` for anything the kernel does not cover, exactly where the
    reference's hook does (_merge_kernel.py:117-138), so the caller's eager
    fallback stays reachable.
    """
    if not o1.is_cuda:
        return None
    if layout not in ("bhsd", "bshd"):
        return None
    if o1.dtype not in _SUPPORTED_O or o2.dtype not in _SUPPORTED_O:
        return None
    if o1.shape != o2.shape or not o1.is_contiguous() or not o2.is_contiguous():
        return None
    if l1.shape != l2.shape or l1.dim() != 3 or not l1.is_contiguous() or not l2.is_contiguous():
        return None
    if o1.dtype != torch.float32 and o1.dtype != o2.dtype:
        return None
    is_bshd = layout == "bshd"
    b, s1, s2, d = o1.shape
    n = s1 if is_bshd else s2
    h = s2 if is_bshd else s1
    if l1.shape != (b, h, n) or l1.dtype != torch.float32:
        return None
    l2f = l2 if l2.dtype == torch.float32 else l2.to(torch.float32)
    l_new = torch.empty_like(l1, dtype=torch.float32)
    rc = _lib.load().jg_lse_merge(
        _lib.ptr(o1), _lib.ptr(l1), _lib.ptr(o2), _lib.ptr(l2f), _lib.ptr(l_new), b, h, n, d, int(is_bshd),
        _lib.dtype_code(o1.dtype), _lib.dtype_code(o2.dtype), _lib.stream_ptr(o1.device),
    )
    _lib.check(rc, "jg_lse_merge")
    return o1, l_new


# --------------------------------------------------------------------------- #
# attention core
# --------------------------------------------------------------------------- #
def _flat(t: torch.Tensor) -> tuple[int, int, int]:
    if t.dim() < 3:
        raise ValueError(f"expected (..., s, d), got shape {tuple(t.shape)}")
    batch = 1
    for s in t.shape[:-2]:
        batch *= int(s)
    return batch, int(t.shape[-2]), int(t.shape[-1])


def _check_qkv(q, k, v):
    _lib.require_gpu(q, k, v)
    if not (q.dtype == k.dtype == v.dtype):
        raise RuntimeError(f"q, k, v must share a dtype, got {q.dtype}, {k.dtype}, {v.dtype}")
    if k.shape != v.shape or q.shape[:-2] != k.shape[:-2] or q.shape[-1] != k.shape[-1]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")


def _bias_args(bias, batch, sq, sk):
    if bias is None:
        return None, 0
    bias = bias.to(torch.float32).contiguous()
    if bias.dim() < 2 or tuple(bias.shape[-2:]) != (sq, sk):
        raise ValueError(f"bias must end in ({sq}, {sk}), got {tuple(bias.shape)}")
    period = bias.numel() // (sq * sk)
    if period == 0 or batch % period:
        raise ValueError(f"bias with {period} matrices does not tile a batch of {batch}")
    return bias, period


# --------------------------------------------------------------------------- #
# Shapes the MFMA kernels do not take as they are (head sizes other than 64, 96 and 128 -- the
# "widths" below; fp16 has kernels for 96 and 128 only --, sequence lengths that are not multiples
# of 128) are brought to them on the host, in bf16 / fp16 and without a bias:
#   * head size: zero columns are appended to q, k, v (they add nothing to the scores and give
#     zero output columns);
#   * queries: zero rows are appended and their results dropped;
#   * keys, head size below its width: rows are appended whose first spare column holds -c, against
#     a column of c in q, c = sqrt(30000 / scale) (a value fp16 can hold): their scores are
#     -30000, their probabilities 0;
#   * keys, head size equal to its width (no spare column): the multiple of 128 goes through the MFMA kernels, the
#     remaining keys through the one-thread-per-row kernel, and the two (out, lse) pairs are merged
#     like two ring steps; the backward treats the two key ranges like two ring chunks, the short
#     one filled up with zero keys (which the backward's arithmetic ignores by itself).
# Half of the matrix-core work on zeros is still tens of times faster than the FMA kernel.
# --------------------------------------------------------------------------- #
_MASKED_SCORE = -30000.0


def _width(d: int, dtype: torch.dtype) -> int:
    """Head size of the MFMA kernels that take a head of ``d`` columns (fp16: 96 and 128 only)."""
    return 64 if d <= 64 and dtype == torch.bfloat16 else 96 if d <= 96 else 128


_KERNEL_HEAD_SIZES = (8, 16, 32, 64, 96, 128)


_F32_MFMA_HEAD_SIZES = (32, 64, 128)


def _kernel_head_size(d: int, dtype=None, has_bias: bool = False) -> int:
    """Smallest head size the kernels are built for that holds ``d`` columns (zero columns change
    neither scores nor the other outputs); ``d`` itself beyond the largest. fp32 without a bias
    goes to the sizes of its matrix-core kernels, everything else to those of the
    one-thread-per-row kernels."""
    sizes = _F32_MFMA_HEAD_SIZES if dtype == torch.float32 and not has_bias else _KERNEL_HEAD_SIZES
    return next((n for n in sizes if n >= d), d)


def _shapeable(q, k, bias) -> bool:
    d, sq, sk = q.shape[-1], q.shape[-2], k.shape[-2]
    if bias is not None or q.dtype not in (torch.bfloat16, torch.float16) or d > 128 or sq == 0 or sk < 128:
        return False
    return d != _width(d, q.dtype) or sq % 128 != 0 or sk % 128 != 0


def _pad_last(t: torch.Tensor, to: int) -> torch.Tensor:
    return t if t.shape[-1] == to else torch.nn.functional.pad(t, (0, to - t.shape[-1]))


def _pad_rows(t: torch.Tensor, to: int) -> torch.Tensor:
    return t if t.shape[-2] == to else torch.nn.functional.pad(t, (0, 0, 0, to - t.shape[-2]))


def _up128(n: int) -> int:
    return (n + 127) // 128 * 128


def _shape_qkv(q, k, v, scale):
    """q, k, v as the MFMA kernels take them: ``(q, k, v, key ranges)``; a key range is
    ``(start, stop)`` in the (possibly padded) k / v, the first one a multiple of 128 long."""
    d, sq, sk = q.shape[-1], q.shape[-2], k.shape[-2]
    w = _width(d, q.dtype)
    qp = _pad_rows(_pad_last(q, w), _up128(sq))
    kp, vp = _pad_last(k, w), _pad_last(v, w)
    if sk % 128 == 0:
        return qp, kp, vp, [(0, sk)]
    if d < w:
        c = math.sqrt(-_MASKED_SCORE / float(scale))
        qp[..., d] = c
        kp, vp = _pad_rows(kp, _up128(sk)), _pad_rows(vp, _up128(sk))
        kp[..., sk:, d] = -c
        return qp, kp, vp, [(0, _up128(sk))]
    main = sk // 128 * 128
    return qp, kp, vp, [(0, main), (main, sk)]


def _shaped_forward(q, k, v, scale):
    d, sq = q.shape[-1], q.shape[-2]
    qp, kp, vp, ranges = _shape_qkv(q, k, v, scale)
    out, lse = _core_forward(qp, kp[..., ranges[0][0]:ranges[0][1], :], vp[..., ranges[0][0]:ranges[0][1], :], scale)
    if len(ranges) == 2:
        o2, l2 = _core_forward(qp, kp[..., ranges[1][0]:ranges[1][1], :], vp[..., ranges[1][0]:ranges[1][1], :], scale)
        rows, w = qp.shape[-2], qp.shape[-1]
        merged = fused_online_softmax_merge_(out.float().reshape(1, -1, rows, w), lse.reshape(1, -1, rows),
                                             o2.reshape(1, -1, rows, w), l2.reshape(1, -1, rows), "bhsd")
        out, lse = merged[0].to(q.dtype).reshape(out.shape), merged[1].reshape(lse.shape)
    return out[..., :sq, :d].contiguous(), lse[..., :sq].contiguous()


def _shaped_backward(grad_out, q, k, v, out, lse, scale):
    d, sq, sk = q.shape[-1], q.shape[-2], k.shape[-2]
    qp, kp, vp, ranges = _shape_qkv(q, k, v, scale)
    rows, w = qp.shape[-2], qp.shape[-1]
    gp, op = _pad_rows(_pad_last(grad_out, w), rows), _pad_rows(_pad_last(out, w), rows)
    lp = lse if lse.shape[-1] == rows else torch.nn.functional.pad(lse, (0, rows - lse.shape[-1]))
    dq, dks, dvs = None, [], []
    for lo, hi in ranges:
        # A key range shorter than a tile is filled up with zero keys: with the global out / lse a
        # zero key adds nothing to dq (its k is zero) and its own dk / dv rows are dropped, so the
        # backward needs no mask.
        kj, vj = _pad_rows(kp[..., lo:hi, :], _up128(hi - lo)), _pad_rows(vp[..., lo:hi, :], _up128(hi - lo))
        dq_j, dk_j, dv_j = _core_backward(gp, qp, kj, vj, op, lp, scale)
        dq = dq_j.float() if dq is None else dq + dq_j.float()
        dks.append(dk_j[..., : hi - lo, :])
        dvs.append(dv_j[..., : hi - lo, :])
    dk = dks[0] if len(dks) == 1 else torch.cat(dks, dim=-2)
    dv = dvs[0] if len(dvs) == 1 else torch.cat(dvs, dim=-2)
    return (dq[..., :sq, :d].to(q.dtype).contiguous(), dk[..., :sk, :d].contiguous(), dv[..., :sk, :d].contiguous())


def core_forward(q, k, v, scale, bias=None, out_acc=None, lse_acc=None, want_out=True):
    """One attention core call; optionally merges into ``(out_acc, lse_acc)`` in place.

    Returns ``(out, lse)`` (``None`` each when ``want_out`` is false).
    """
    _check_qkv(q, k, v)
    if out_acc is None and lse_acc is None and want_out and _shapeable(q, k, bias):
        return _shaped_forward(q, k, v, scale)
    d, dp = q.shape[-1], _kernel_head_size(q.shape[-1], q.dtype, bias is not None)
    if dp != d and out_acc is None and lse_acc is None:
        out, lse = _core_forward(_pad_last(q, dp), _pad_last(k, dp), _pad_last(v, dp), scale, bias, None, None, want_out)
        return (out[..., :d].contiguous() if want_out else None), lse
    return _core_forward(q, k, v, scale, bias, out_acc, lse_acc, want_out)


def _core_forward(q, k, v, scale, bias=None, out_acc=None, lse_acc=None, want_out=True):
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    batch, sq, d = _flat(q)
    sk = int(k.shape[-2])
    bias_t, period = _bias_args(bias, batch, sq, sk)
    out = torch.empty_like(q) if want_out else None
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device) if want_out else None
    rc = _lib.load().jg_attn_fwd(
        _lib.ptr(out), _lib.ptr(lse), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), batch, sq, sk, d, float(scale),
        _lib.ptr(bias_t), period, _lib.ptr(out_acc), _lib.ptr(lse_acc), _lib.dtype_code(q.dtype),
        _lib.stream_ptr(q.device),
    )
    _lib.check(rc, "jg_attn_fwd")
    return out, lse


def forward(q, k, v, scale=0.0, dropout_p=0.0, seed=None, *, layout="bhsd"):
    """Attention core forward with the reference's signature
    (cores/math.py:31-78, cores/sdpa.py:17-85): ``(out, logsumexp, rng_state)``."""
    if layout != "bhsd":
        raise NotImplementedError(f"the HIP core is bhsd-only; got layout={layout!r}")
    if dropout_p != 0.0:
        raise NotImplementedError("attention dropout is not supported by the HIP core")
    scale = scale or (q.size(-1) ** -0.5)
    out, lse = core_forward(q, k, v, scale)
    return out, lse, None


def core_backward(grad_out, q, k, v, out, logsumexp, scale, bias=None, want_dbias=False):
    """``(dq, dk, dv[, dbias])`` of one chunk from the global ``out`` / ``logsumexp``."""
    _check_qkv(q, k, v)
    _lib.require_gpu(grad_out, out, logsumexp)
    if not want_dbias and _shapeable(q, k, bias):
        return _shaped_backward(grad_out.to(q.dtype), q, k, v, out.to(q.dtype), logsumexp.to(torch.float32), scale)
    d, dp = q.shape[-1], _kernel_head_size(q.shape[-1], q.dtype, bias is not None)
    if dp != d:
        res = _core_backward(_pad_last(grad_out, dp), _pad_last(q, dp), _pad_last(k, dp), _pad_last(v, dp),
                             _pad_last(out, dp), logsumexp, scale, bias, want_dbias)
        return tuple(t[..., :d].contiguous() for t in res[:3]) + tuple(res[3:])
    return _core_backward(grad_out, q, k, v, out, logsumexp, scale, bias, want_dbias)


def _core_backward(grad_out, q, k, v, out, logsumexp, scale, bias=None, want_dbias=False):
    dt = q.dtype
    grad_out, out = grad_out.to(dt).contiguous(), out.to(dt).contiguous()
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    lse = logsumexp.to(torch.float32).contiguous()
    batch, sq, d = _flat(q)
    sk = int(k.shape[-2])
    bias_t, period = _bias_args(bias, batch, sq, sk)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dbias = torch.empty(q.shape[:-1] + (sk,), dtype=torch.float32, device=q.device) if want_dbias else None
    lib = _lib.load()
    nbytes = int(lib.jg_attn_bwd_workspace_bytes(batch, sq, sk, d))
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=q.device)
    rc = lib.jg_attn_bwd(
        _lib.ptr(dq), _lib.ptr(dk), _lib.ptr(dv), _lib.ptr(grad_out), _lib.ptr(q), _lib.ptr(k), _lib.ptr(v),
        _lib.ptr(out), _lib.ptr(lse), batch, sq, sk, d, float(scale), _lib.ptr(bias_t), period, _lib.ptr(dbias),
        _lib.dtype_code(dt), _lib.ptr(ws), nbytes, _lib.stream_ptr(q.device),
    )
    _lib.check(rc, "jg_attn_bwd")
    if want_dbias:
        return dq, dk, dv, dbias
    return dq, dk, dv


def backward(grad_out, q, k, v, out, logsumexp, scale, *args, dropout_p=0.0, seed=None, rng_state=None,
             layout="bhsd", **kwargs):
    """Attention core backward with the reference's signature
    (cores/math.py:81-149, cores/sdpa.py:88-165): ``(dq, dk, dv)`` in ``grad_out.dtype``."""
    if layout != "bhsd":
        raise NotImplementedError(f"the HIP core is bhsd-only; got layout={layout!r}")
    if dropout_p != 0.0:
        raise NotImplementedError("attention dropout is not supported by the HIP core")
    dq, dk, dv = core_backward(grad_out, q, k, v, out, logsumexp, scale)
    gd = grad_out.dtype
    return dq.to(gd), dk.to(gd), dv.to(gd)


# --------------------------------------------------------------------------- #
# per-rank ring loops over local chunks
# --------------------------------------------------------------------------- #
def _fused_ok(q, k) -> bool:
    """Whether one launch attends the chunk AND merges into the running accumulators: the 16-bit MFMA
    kernels at head sizes 64 / 96 / 128 with lengths in multiples of 128, and the fp32 matrix-core
    kernel at head sizes 32 / 64 / 128 (any lengths, 16-byte aligned tensors)."""
    d = q.shape[-1]
    if q.dtype == torch.float32:
        return d in (32, 64, 128) and all(t.data_ptr() % 16 == 0 for t in (q, k))
    return (
        q.dtype in (torch.bfloat16, torch.float16) and d in (64, 96, 128) and d == _width(d, q.dtype)
        and q.shape[-2] % 128 == 0 and k.shape[-2] % 128 == 0
    )


def attend_step_(q, kj, vj, scale, out, lse):
    """One ring step: attend chunk ``(kj, vj)`` and merge into the running fp32
    ``(out, lse)`` in place (``_attend_step``, forward.py:64-96). Uses the fused
    kernel when it covers the shape, the core + merge kernels otherwise."""
    kj, vj = kj.contiguous(), vj.contiguous()
    if (_fused_ok(q, kj) and q.is_contiguous() and vj.data_ptr() % 16 == 0 and out.dtype == torch.float32
            and out.is_contiguous() and lse.is_contiguous() and out.data_ptr() % 16 == 0):
        core_forward(q, kj, vj, scale, out_acc=out, lse_acc=lse, want_out=False)
        return out, lse
    out_j, l_j = core_forward(q, kj, vj, scale)
    fused = fused_online_softmax_merge_(out, lse, out_j, l_j, "bhsd")
    if fused is None:
        raise NotImplementedError("merge of these dtypes / layouts is not covered by the HIP kernel")
    return fused


def ring_forward(q, k_chunks: Sequence[torch.Tensor], v_chunks: Sequence[torch.Tensor], scale, rank: int = 0):
    """``(out, lse)`` of one rank's queries over all P chunks, visited in ring order
    ``(rank + step) % P`` (forward_chunk_provider.py:190-192). The accumulator is
    fp32 and cast to ``q.dtype`` once at the end (forward.py:160-167, 199)."""
    P = len(k_chunks)
    acc = torch.promote_types(q.dtype, torch.float32)
    out = torch.zeros(q.shape, device=q.device, dtype=acc)
    lse = torch.full(q.shape[:-1], float("-inf"), device=q.device, dtype=acc)
    for step in range(P):
        j = (rank + step) % P
        out, lse = attend_step_(q, k_chunks[j].to(q.dtype), v_chunks[j].to(q.dtype), scale, out, lse)
    return out.to(q.dtype), lse


_MAX_CHUNKS_PER_CALL = 16


def backward_chunks(dout, q, out, lse, k_chunks, v_chunks, scale):
    """``(dq, [dk_j], [dv_j])`` over resident chunks in ONE pass (``jg_attn_bwd_chunks``): the dQ
    kernel walks every chunk with dQ in its registers (one launch, one rounding), the dK/dV kernel
    takes the chunk as a grid dimension. ``None`` where that entry point does not cover the call
    (anything but bf16 at head size 64 with lengths that are multiples of 128, up to 16 chunks of
    one shape)."""
    P = len(k_chunks)
    if not 1 <= P <= _MAX_CHUNKS_PER_CALL or len(v_chunks) != P:
        return None
    if q.dtype != torch.bfloat16 or q.shape[-1] != 64 or q.shape[-2] % 128 or k_chunks[0].shape[-2] % 128:
        return None
    if any(t.shape != k_chunks[0].shape or t.dtype != q.dtype or t.device != q.device for t in (*k_chunks, *v_chunks)):
        return None
    if k_chunks[0].shape[:-2] != q.shape[:-2] or not q.is_cuda:
        return None
    _lib.require_gpu(dout, q, out, lse)
    dout, out, q = dout.to(q.dtype).contiguous(), out.to(q.dtype).contiguous(), q.contiguous()
    lse = lse.to(torch.float32).contiguous()
    ks = [t.contiguous() for t in k_chunks]
    vs = [t.contiguous() for t in v_chunks]
    batch, sq, d = _flat(q)
    sk = int(ks[0].shape[-2])
    dq = torch.empty_like(q)
    # one allocation for all partials: chunk j's dK / dV are views of it
    dkv = torch.empty((2, P) + tuple(ks[0].shape), dtype=q.dtype, device=q.device)
    dks, dvs = list(dkv[0].unbind(0)), list(dkv[1].unbind(0))
    lib = _lib.load()
    nbytes = int(lib.jg_attn_bwd_workspace_bytes(batch, sq, sk, d))
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=q.device)
    arr = lambda ts: (ctypes.c_void_p * P)(*(t.data_ptr() for t in ts))  # noqa: E731
    rc = lib.jg_attn_bwd_chunks(
        _lib.ptr(dq), arr(dks), arr(dvs), _lib.ptr(dout), _lib.ptr(q), arr(ks), arr(vs), P, _lib.ptr(out), _lib.ptr(lse),
        batch, sq, sk, d, float(scale), _lib.dtype_code(q.dtype), _lib.ptr(ws), nbytes, _lib.stream_ptr(q.device),
    )
    if rc == -2:
        return None
    _lib.check(rc, "jg_attn_bwd_chunks")
    return dq, dks, dvs


def ring_backward(dout, q, out, lse, k_chunks, v_chunks, scale):
    """``(dq, [dk_j], [dv_j])``: this rank's contribution to every chunk's gradient.

    ``dq`` accumulates over the chunks (backward.py:184, 269; here in fp32, cast to
    ``q.dtype`` at the end — the reference accumulates in ``q.dtype``); the sum of
    dK/dV over the ranks that attended a chunk is the caller's collective. Chunks that are all
    resident go through one pass (:func:`backward_chunks`) where it covers them."""
    core = q.dtype
    one_pass = backward_chunks(dout, q, out, lse, [t.to(core) for t in k_chunks], [t.to(core) for t in v_chunks], scale)
    if one_pass is not None:
        return one_pass
    dout, out = dout.to(core), out.to(core)
    dq = torch.zeros(q.shape, device=q.device, dtype=torch.float32)
    dks, dvs = [], []
    for kj, vj in zip(k_chunks, v_chunks):
        dq_j, dk_j, dv_j = core_backward(dout, q, kj.to(core), vj.to(core), out, lse, scale)
        dq += dq_j
        dks.append(dk_j)
        dvs.append(dv_j)
    return dq.to(core), dks, dvs


# --------------------------------------------------------------------------- #
# windowed attention with an additive bias (Swin block)
# --------------------------------------------------------------------------- #
class _BiasedAttention(torch.autograd.Function):
    """``F.scaled_dot_product_attention(q, k, v, attn_mask=bias)`` as the Swin example
    calls it (examples/swin.py:146-151), differentiable in q, k, v and bias."""

    @staticmethod
    def forward(ctx, q, k, v, bias):  # noqa: D102
        scale = q.shape[-1] ** -0.5
        out, lse = core_forward(q, k, v, scale, bias=bias)
        ctx.save_for_backward(q, k, v, bias, out, lse)
        ctx.scale = scale
        return out

    @staticmethod
    def backward(ctx, grad_out):  # noqa: D102
        q, k, v, bias, out, lse = ctx.saved_tensors
        need_bias = bias is not None and ctx.needs_input_grad[3]
        res = core_backward(grad_out, q, k, v, out, lse, ctx.scale, bias=bias, want_dbias=need_bias)
        dq, dk, dv = res[:3]
        dbias = None
        if need_bias:
            # sum the per-batch-entry gradient over the entries that share a bias matrix
            sq, sk = q.shape[-2], k.shape[-2]
            period = bias.numel() // (sq * sk)
            per_entry = res[3].reshape(-1, period, sq, sk)
            dbias = (per_entry[0] if per_entry.shape[0] == 1 else per_entry.sum(0)).reshape(bias.shape).to(bias.dtype)
        return dq, dk, dv, dbias


def window_attention(q, k, v, bias=None):
    """softmax(q k^T / sqrt(d) + bias) v over the last two axes."""
    return _BiasedAttention.apply(q, k, v, bias)


SWIN_WINDOW, SWIN_HEAD_SIZE = 8, 32


def swin_grid_supported(q: torch.Tensor, grid: tuple, window: int) -> bool:
    """Whether :func:`swin_grid_attention` has a kernel for these tensors: bf16, head size 32,
    8 x 8 windows tiling the token grid."""
    return (
        q.dtype == torch.bfloat16 and q.shape[-1] == SWIN_HEAD_SIZE and window == SWIN_WINDOW
        and grid[0] % window == 0 and grid[1] % window == 0 and grid[0] * grid[1] == q.shape[-2]
    )


class _SwinGridAttention(torch.autograd.Function):
    """Attention inside the 8 x 8 windows of a token grid. ``qkv`` is (3, B, heads, gh * gw, 32), the
    tokens in grid order, as the qkv projection writes it; relative-position bias from ``table``
    (225, heads) and the shift mask from the per-token codes ``side`` (windows, 64) are formed inside
    the kernel (examples/swin.py:99-170). Differentiable in qkv and table; the gradient comes back
    as one (3, ...) tensor, so that nothing is stacked or split on the way to the projection."""

    @staticmethod
    def forward(ctx, qkv, table, side, grid):  # noqa: D102
        lib = _lib.load()
        qkv = qkv.contiguous()
        table = table.detach().float().contiguous()
        _, images, heads, tokens, d = qkv.shape
        gh, gw = grid
        scale = d ** -0.5
        out = torch.empty_like(qkv[0])
        lse = torch.empty(images * heads * tokens, dtype=torch.float32, device=qkv.device)
        rc = lib.jg_attn_swin_fwd(
            _lib.ptr(out), _lib.ptr(lse), _lib.ptr(qkv[0]), _lib.ptr(qkv[1]), _lib.ptr(qkv[2]), _lib.ptr(table),
            _lib.ptr(side), images, heads, gh, gw, d, float(scale), _lib.dtype_code(qkv.dtype),
            _lib.stream_ptr(qkv.device),
        )
        _lib.check(rc, "jg_attn_swin_fwd")
        ctx.save_for_backward(qkv, table, side, out, lse)
        ctx.grid, ctx.scale = (gh, gw), scale
        return out

    @staticmethod
    def backward(ctx, grad_out):  # noqa: D102
        lib = _lib.load()
        qkv, table, side, out, lse = ctx.saved_tensors
        _, images, heads, tokens, d = qkv.shape
        gh, gw = ctx.grid
        grad_out = grad_out.contiguous()
        dqkv = torch.empty_like(qkv)
        dtable = ws = None
        ws_bytes = 0
        if ctx.needs_input_grad[1]:
            dtable = torch.empty_like(table)
            ws_bytes = lib.jg_attn_swin_bwd_workspace_bytes(images, heads, gh, gw)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=qkv.device)
        rc = lib.jg_attn_swin_bwd(
            _lib.ptr(dqkv[0]), _lib.ptr(dqkv[1]), _lib.ptr(dqkv[2]), _lib.ptr(dtable), _lib.ptr(grad_out),
            _lib.ptr(qkv[0]), _lib.ptr(qkv[1]), _lib.ptr(qkv[2]), _lib.ptr(out), _lib.ptr(lse), _lib.ptr(table),
            _lib.ptr(side), images, heads, gh, gw, d, float(ctx.scale), _lib.dtype_code(qkv.dtype), _lib.ptr(ws),
            ws_bytes, _lib.stream_ptr(qkv.device),
        )
        _lib.check(rc, "jg_attn_swin_bwd")
        return dqkv, dtable, None, None


def swin_grid_attention_packed(qkv, table, side, grid):
    """:func:`swin_grid_attention` on the (3, B, heads, tokens, 32) tensor of the qkv projection."""
    if qkv.dim() != 5 or qkv.shape[0] != 3 or not swin_grid_supported(qkv[0], grid, SWIN_WINDOW):
        raise NotImplementedError("swin_grid_attention: (3, B, heads, tokens, 32) bf16 and 8 x 8 windows only")
    if side is not None and (side.dtype != torch.uint8 or side.numel() != qkv.shape[-2]):
        raise ValueError("side must be a uint8 code per token, (windows, 64)")
    if table.shape != (225, qkv.shape[2]):
        raise ValueError(f"table must be (225, heads = {qkv.shape[2]}), got {tuple(table.shape)}")
    return _SwinGridAttention.apply(qkv, table, side, grid)


def swin_grid_attention(q, k, v, table, side, grid):
    """Attention inside the 8 x 8 windows of a token grid for separate ``q, k, v`` of shape
    (B, heads, gh * gw, 32) (stacked here; see :func:`swin_grid_attention_packed`). ``side`` is a uint8
    tensor (windows, 64) or ``None``."""
    if not swin_grid_supported(q, grid, SWIN_WINDOW):
        raise NotImplementedError("swin_grid_attention: bf16, head size 32 and 8 x 8 windows only")
    return swin_grid_attention_packed(torch.stack((q, k, v)), table, side, grid)


__all__ = [
    "attend_step_",
    "backward",
    "backward_chunks",
    "core_backward",
    "core_forward",
    "forward",
    "fused_online_softmax_merge_",
    "ring_backward",
    "ring_forward",
    "swin_grid_attention",
    "swin_grid_attention_packed",
    "swin_grid_supported",
    "window_attention",
]
