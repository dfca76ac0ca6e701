"""Ring-attention step on the GPU: attention core, log-sum-exp merge, ring loops.

Host-side mirror of the attention-core contract
(jigsaw/modules/attention/_functional/cores/__init__.py:1-15) and of the fused
merge hook (jigsaw/modules/attention/_functional/_merge_kernel.py:88-172).
"""

from __future__ import annotations

import torch

from . import _lib

_SUPPORTED_O = (torch.float16, torch.bfloat16, torch.float32)


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


__all__ = ["fused_online_softmax_merge_"]
