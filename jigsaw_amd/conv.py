"""Local convolution and the halo-exchange convolution on the GPU.

Host-side mirror of the callables the reference keeps on ``ConvNdConfig``
(jigsaw/modules/convolution/_conv/config.py:82-95):

* ``conv_fn`` / ``conv_input_fn`` / ``conv_weight_fn`` / ``grad_bias`` with the
  signatures of ``F.conv{1,2,3}d``, ``torch.nn.grad.conv*_input``,
  ``conv*_weight`` and ``_sum_grad_bias``;
* ``dist_conv_fn`` / ``dist_conv_backward_fn`` with the signatures of
  ``conv_halo_nway`` / ``conv_halo_nway_backward``
  (jigsaw/modules/convolution/_conv/distributed.py:212-396);
* ``_ConvNd`` (jigsaw/modules/convolution/_conv/functional.py:28-169).

The reference pads one split axis at a time through a collective. Here a rank
packs all its strips once, hands them to ``config.halo_exchange`` (the only part
that talks to other ranks), and assembles the padded tile in one pass.
"""

from __future__ import annotations

import ctypes
import itertools
import math
from collections.abc import Sequence
from typing import Any, Protocol

import torch

from . import _lib
from .halo import (HaloGeometry, halo_assemble, halo_fold, halo_fold_border_, halo_gather_axis, halo_pack,
                   halo_scatter_add_axis, new_strips, spans_fit_the_strips, strip_table)

# --------------------------------------------------------------------------- #
# local primitives
# --------------------------------------------------------------------------- #


def _tup(v: int | Sequence[int], n: int, name: str) -> tuple:
    if isinstance(v, int):
        return (v,) * n
    v = tuple(int(i) for i in v)
    if len(v) == 1:
        return v * n
    if len(v) != n:
        raise ValueError(f"{name} must have {n} entries, got {v}")
    return v


def _desc(batch, c_in, c_out, in_spatial, kernel, stride, padding, dilation, groups) -> _lib.ConvDesc:
    n = len(kernel)
    d = _lib.ConvDesc()
    d.n_spatial, d.groups, d.batch, d.c_in, d.c_out = n, groups, batch, c_in, c_out
    lead = 3 - n
    for a in range(3):
        if a < lead:
            d.in_size[a], d.kernel[a], d.stride[a], d.padding[a], d.dilation[a] = 1, 1, 1, 0, 1
        else:
            i = a - lead
            d.in_size[a], d.kernel[a] = in_spatial[i], kernel[i]
            d.stride[a], d.padding[a], d.dilation[a] = stride[i], padding[i], dilation[i]
    return d


def _out_spatial(in_spatial, kernel, stride, padding, dilation) -> tuple:
    out = []
    for i, k, s, p, d in zip(in_spatial, kernel, stride, padding, dilation):
        span = i + 2 * p - d * (k - 1) - 1
        if span < 0:
            raise RuntimeError(
                f"Calculated padded input size per channel: ({i + 2 * p}). Kernel size: ({d * (k - 1) + 1}). "
                "Kernel size can't be greater than actual input size"
            )
        out.append(span // s + 1)
    return tuple(out)


def _workspace(desc: _lib.ConvDesc, op: int, dtype: torch.dtype, device, given: torch.Tensor | None = None
               ) -> tuple[torch.Tensor | None, int]:
    """The workspace of one launch: ``given`` when the caller brought one (checked for size), else a new one."""
    nbytes = int(_lib.load().jg_conv_workspace_bytes(desc, op, _lib.dtype_code(dtype)))
    if nbytes == 0:
        return None, 0
    if given is not None:
        if given.device != torch.device(device) or not given.is_contiguous() or given.numel() * given.element_size() < nbytes:
            raise ValueError(f"workspace: needs {nbytes} contiguous bytes on {device}")
        return given, nbytes
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def _out_tensor(out: torch.Tensor | None, shape, dtype: torch.dtype, device, what: str) -> torch.Tensor:
    """``out`` when given (shape, dtype and layout checked), else a new tensor."""
    if out is None:
        return torch.empty(shape, dtype=dtype, device=device)
    if tuple(out.shape) != tuple(shape) or out.dtype != dtype or out.device != torch.device(device) or not out.is_contiguous():
        raise ValueError(f"{what}: `out` must be a contiguous {dtype} tensor of shape {tuple(shape)} on {device}")
    return out


def _check_args(x_like, w, groups, padding):
    if isinstance(padding, str):
        raise NotImplementedError(f"string padding ({padding!r}) is not supported; pass per-axis integers")
    if not isinstance(groups, int) or groups < 1 or w.shape[0] % groups:
        raise ValueError(f"groups = {groups} must be a positive integer that divides the {w.shape[0]} output channels")
    n = w.dim() - 2
    if n not in (1, 2, 3):
        raise ValueError(f"weight must be (Cout, Cin, *kernel) with 1 to 3 spatial axes, got {tuple(w.shape)}")
    return n


# --------------------------------------------------------------------------- #
# Non-overlapping kernels (kernel == stride, no padding, no dilation: patch embeddings,
# 1 x 1 convolutions) are a GEMM over the patches: the patch matrix is laid out once and the
# MFMA projection kernels (jg_proj_nt / jg_proj_tn) do the arithmetic.
# --------------------------------------------------------------------------- #
def _patch_gemm_ok(dtype, c_in, c_out, kernel, stride, padding, dilation) -> bool:
    if dtype != torch.bfloat16:
        return False
    if any(k != s for k, s in zip(kernel, stride)) or any(padding) or any(d != 1 for d in dilation):
        return False
    k_elems = c_in
    for k in kernel:
        k_elems *= int(k)
    return k_elems % 8 == 0 and c_out % 8 == 0


def _patchify(x: torch.Tensor, kernel, out_sp) -> torch.Tensor:
    """``(N, C, *spatial) -> (N * prod(out), C * prod(kernel))``, features ordered as the weight's ``(C, *kernel)``."""
    n = len(kernel)
    x = x[(slice(None), slice(None)) + tuple(slice(0, o * k) for o, k in zip(out_sp, kernel))]
    shape = [x.shape[0], x.shape[1]]
    for o, k in zip(out_sp, kernel):
        shape += [o, k]
    x = x.reshape(shape)
    o_dims = [2 + 2 * i for i in range(n)]
    k_dims = [3 + 2 * i for i in range(n)]
    rows = x.shape[0]
    for o in out_sp:
        rows *= o
    return x.permute(0, *o_dims, 1, *k_dims).reshape(rows, -1)


def _unpatchify(p: torch.Tensor, input_shape, kernel, out_sp) -> torch.Tensor:
    """Inverse of :func:`_patchify`; cells no patch covers (a remainder of the extent) are zero."""
    n = len(kernel)
    batch, c = input_shape[0], input_shape[1]
    p = p.reshape(batch, *out_sp, c, *kernel)
    perm = [0, n + 1]
    for i in range(n):
        perm += [1 + i, n + 2 + i]
    covered = tuple(o * k for o, k in zip(out_sp, kernel))
    body = p.permute(perm).reshape(batch, c, *covered)
    if covered == tuple(input_shape[2:]):
        return body.contiguous()
    gx = torch.zeros(input_shape, dtype=p.dtype, device=p.device)
    gx[(slice(None), slice(None)) + tuple(slice(0, v) for v in covered)] = body
    return gx


def _proj_nt(a: torch.Tensor, w2: torch.Tensor, bias) -> torch.Tensor:
    rows, k = a.shape
    out = torch.empty(rows, w2.shape[0], dtype=a.dtype, device=a.device)
    if rows:
        rc = _lib.load().jg_proj_nt(_lib.ptr(out), _lib.ptr(a), _lib.ptr(w2), _lib.ptr(bias), _lib.dtype_code(a.dtype),
                                    rows, w2.shape[0], k, 0, 0, 1, 1, 1, 1, _lib.stream_ptr(a.device))
        _lib.check(rc, "jg_proj_nt")
    return out


def _tokens_of(g: torch.Tensor) -> torch.Tensor:
    """``(N, M, *out) -> (N * prod(out), M)``."""
    n = g.dim() - 2
    return g.permute(0, *range(2, 2 + n), 1).reshape(-1, g.shape[1])


# --------------------------------------------------------------------------- #
# Kernels with extents 1 or 3 per axis (1 x 1, 1 x 3, 3 x 1, ...) at stride 1 run on the 3 x 3 (x 3)
# MFMA kernels: the weights sit in the centre of a zero 3 x 3 (x 3) kernel and the padding grows
# by one on the axes that were 1. Same result (the added taps multiply zeros), and although most of
# the matrix-core work is on zeros it is far faster than the FMA kernels.
# --------------------------------------------------------------------------- #
def _embed3(kernel, stride, dilation):
    """Per-axis tap offset ((3 - k) / 2) when the kernel embeds into 3 x 3 (x 3), else ``None``."""
    n = len(kernel)
    if n not in (2, 3) or all(k == 3 for k in kernel):
        return None
    if any(k not in (1, 3) for k in kernel) or any(s != 1 for s in stride):
        return None
    if any(d != 1 and k != 1 for d, k in zip(dilation, kernel)):
        return None
    return tuple((3 - k) // 2 for k in kernel)


def _embed_weight(w: torch.Tensor, off) -> torch.Tensor:
    w3 = torch.zeros((w.shape[0], w.shape[1]) + (3,) * len(off), dtype=w.dtype, device=w.device)
    w3[(slice(None), slice(None)) + tuple(slice(o, 3 - o) for o in off)] = w
    return w3


# --------------------------------------------------------------------------- #
# Strided kernels with extents 1 or 3 (3 x 3 stride 2 down-sampling, ...): the stride-1 result
# sampled at the stride (forward), and the stride-1 gradients of the output gradient with zeros
# between its cells (backward). Costs prod(stride) times the matrix-core work of the strided
# layer and a copy, and still beats the FMA kernels by an order of magnitude.
# --------------------------------------------------------------------------- #
def _dense_stride_ok(kernel, stride, dilation, padding=None) -> bool:
    if len(kernel) not in (2, 3) or all(s == 1 for s in stride):
        return False
    if all(k == s for k, s in zip(kernel, stride)):  # kernel = stride has its own route
        return False
    ones = (1,) * len(kernel)
    if any(d != 1 for d in dilation):
        return padding is not None and (_dilated_ok(kernel, ones, padding, dilation) or _prepad(kernel, ones, padding, dilation) is not None)
    if any(k not in (1, 3) for k in kernel):
        return _big_kernel_ok(kernel, ones, dilation)
    return True


# --------------------------------------------------------------------------- #
# Dilated 3-tap kernels at stride 1 whose padding is a multiple of the dilation ("same" padding
# p = d, and the halo-padded tile with p = 0): output cell d * o + r reads input cells
# d * (o + t - p / d) + r, so the cells of one residue r form a plain 3-tap convolution of
# their own. The prod(dilation) residue images go into the batch, the undilated MFMA kernels
# run once over all of them, and the result is interleaved back: the same arithmetic, two
# permutation copies per tensor.
# --------------------------------------------------------------------------- #
def _dilated_ok(kernel, stride, padding, dilation) -> bool:
    if len(kernel) not in (2, 3) or any(s != 1 for s in stride):
        return False
    ones = (1,) * len(kernel)
    if any(k not in (1, 3) for k in kernel) and not _big_kernel_ok(kernel, ones, ones):
        return False  # the undilated layer of a residue image must have a route of its own
    if not any(d > 1 and k > 1 for k, d in zip(kernel, dilation)):
        return False
    return all(p % d == 0 for k, p, d in zip(kernel, padding, dilation) if d > 1 and k > 1)


def _phase_counts(kernel, dilation) -> tuple:
    return tuple(int(d) if k > 1 else 1 for k, d in zip(kernel, dilation))


def _prepad(kernel, stride, padding, dilation):
    """A padding that is no multiple of the dilation: the cells to lay around the input as zeros (per
    axis) so that what remains of the padding is one, or ``None`` where that opens no route."""
    if len(kernel) not in (2, 3) or any(s != 1 for s in stride):
        return None
    extra = tuple(p % d if d > 1 and k > 1 else 0 for k, p, d in zip(kernel, padding, dilation))
    if not any(extra):
        return None
    return extra if _dilated_ok(kernel, stride, tuple(p - e for p, e in zip(padding, extra)), dilation) else None


def _zero_rim(x: torch.Tensor, extra) -> torch.Tensor:
    pads = []
    for e in reversed(extra):
        pads += [e, e]
    return torch.nn.functional.pad(x, pads)


def _to_phases(t: torch.Tensor, phases, ext) -> torch.Tensor:
    """``(N, C, *spatial) -> (prod(phases) * N, C, *ext)``: image ``r`` of an axis holds the cells
    ``r, r + P, r + 2 P, ...`` of that axis, zero beyond the tensor's end."""
    n = len(phases)
    full = tuple(e * p for e, p in zip(ext, phases))
    if tuple(t.shape[2:]) != full:
        grown = torch.zeros((t.shape[0], t.shape[1], *full), dtype=t.dtype, device=t.device)
        keep = tuple(slice(0, min(a, b)) for a, b in zip(t.shape[2:], full))
        grown[(slice(None), slice(None)) + keep] = t[(slice(None), slice(None)) + keep]
        t = grown
    shape = [t.shape[0], t.shape[1]]
    for e, p in zip(ext, phases):
        shape += [e, p]
    t = t.reshape(shape)
    p_dims = [3 + 2 * i for i in range(n)]
    e_dims = [2 + 2 * i for i in range(n)]
    return t.permute(*p_dims, 0, 1, *e_dims).reshape(-1, shape[1], *ext)


def _from_phases(tb: torch.Tensor, phases, batch, sizes) -> torch.Tensor:
    """Inverse of :func:`_to_phases`, cut to ``sizes``."""
    n = len(phases)
    ext = tuple(tb.shape[2:])
    t = tb.reshape(*phases, batch, tb.shape[1], *ext)
    perm = [n, n + 1]
    for i in range(n):
        perm += [n + 2 + i, i]
    t = t.permute(perm).reshape(batch, tb.shape[1], *(e * p for e, p in zip(ext, phases)))
    return t[(slice(None), slice(None)) + tuple(slice(0, v) for v in sizes)].contiguous()


# --------------------------------------------------------------------------- #
# Kernels with more than three taps on an axis (5 x 5, 7 x 7, 4 x 4 at stride 1 ...): the taps of an
# axis, filled up in front with zeros to a multiple of three, are blocks of three, and tap 3 i + u
# of block i reads what tap u reads of the input moved by 3 i cells. The moved copies of the input
# (zero padding included) become channel blocks of ONE three-tap layer, which the MFMA kernels run
# without padding: the same products, summed in the same fp32 accumulators, at prod(blocks) times
# the input in memory. The input gradient is the forward of the output gradient under the
# transposed, reversed kernel; the weight gradient is that of the three-tap layer, put back in order.
# --------------------------------------------------------------------------- #
_MAX_TAP_BLOCKS = 9


def _tap_blocks(kernel) -> tuple:
    """Per axis ``(blocks of three taps, zero taps in front)``."""
    return tuple(((k + 2) // 3, (k + 2) // 3 * 3 - k) for k in kernel)


def _big_kernel_ok(kernel, stride, dilation) -> bool:
    if len(kernel) not in (2, 3) or any(s != 1 for s in stride) or any(d != 1 for d in dilation):
        return False
    # two taps are one block with a zero tap in front
    return any(k not in (1, 3) for k in kernel) and math.prod(b for b, _ in _tap_blocks(kernel)) <= _MAX_TAP_BLOCKS


_MOVED_COPY_BYTES = 8 << 30  # most that the moved copies of one call may take


def _tap_blocks_fit(dtype, batch, c_in, kernel, out_sp) -> bool:
    """Whether the three-tap layer the tap-block route builds is one the matrix-core kernels take (their per-image
    extent is bounded by 32-bit byte offsets: cells * 72 * element size < 2 ** 31, fp32 counted at 4 bytes) and its
    moved copies stay below ``_MOVED_COPY_BYTES``; otherwise the layer stays on the direct kernels as it is, where
    zero-padded taps and the copies would only cost."""
    if dtype not in (torch.bfloat16, torch.float16, torch.float32):
        return False
    es = 4 if dtype == torch.float32 else 2
    cells = math.prod(int(o) + 2 for o in out_sp)
    if cells * 72 * es >= 1 << 31:
        return False
    blocks = math.prod(b for b, _ in _tap_blocks(kernel))
    return int(batch) * int(c_in) * blocks * cells * (2 if dtype != torch.float32 else 4) <= _MOVED_COPY_BYTES


def _moved_copies(x: torch.Tensor, kernel, padding, out_sp) -> torch.Tensor:
    """``(N, C, *spatial) -> (N, prod(blocks) * C, *(out + 2))``: block ``(i, j, ..)`` holds the zero-padded
    input moved by ``(3 i, 3 j, ..)`` cells, cut to what a three-tap layer without padding needs."""
    blocks = _tap_blocks(kernel)
    pads = []
    for (_, lead), p in reversed(list(zip(blocks, padding))):  # F.pad counts from the last axis
        pads += [p + lead, p]
    xp = torch.nn.functional.pad(x, pads)
    parts = []
    for idx in itertools.product(*(range(b) for b, _ in blocks)):
        cut = tuple(slice(3 * i, 3 * i + o + 2) for i, o in zip(idx, out_sp))
        parts.append(xp[(slice(None), slice(None)) + cut])
    return torch.cat(parts, dim=1)


def _tap_block_weight(w: torch.Tensor) -> torch.Tensor:
    """``(M, C, *k) -> (M, prod(blocks) * C, 3, 3[, 3])``, channel blocks in the order of :func:`_moved_copies`."""
    n = w.dim() - 2
    blocks = _tap_blocks(w.shape[2:])
    pads = []
    for _, lead in reversed(blocks):
        pads += [lead, 0]
    w6 = torch.nn.functional.pad(w, pads)
    shape = [w.shape[0], w.shape[1]]
    for b, _ in blocks:
        shape += [b, 3]
    w6 = w6.reshape(shape)
    b_dims = [2 + 2 * i for i in range(n)]
    t_dims = [3 + 2 * i for i in range(n)]
    return w6.permute(0, *b_dims, 1, *t_dims).reshape(w.shape[0], -1, *(3,) * n).contiguous()


def _from_tap_blocks(gw3: torch.Tensor, weight_shape) -> torch.Tensor:
    """Inverse of :func:`_tap_block_weight` for a gradient: back to ``weight_shape``, the zero taps dropped."""
    n = len(weight_shape) - 2
    blocks = _tap_blocks(weight_shape[2:])
    m, c = weight_shape[0], weight_shape[1]
    g6 = gw3.reshape(m, *(b for b, _ in blocks), c, *(3,) * n)
    perm = [0, n + 1]
    for i in range(n):
        perm += [1 + i, n + 2 + i]
    g6 = g6.permute(perm).reshape(m, c, *(3 * b for b, _ in blocks))
    return g6[(slice(None), slice(None)) + tuple(slice(lead, None) for _, lead in blocks)].contiguous()


# Grouped layers: a group is an ungrouped layer of its own on a slice of the channels. Where a group has
# at least _GROUP_MIN channels on either side it runs as that layer (on the matrix cores where they
# cover it, through the routes above otherwise), at the price of a contiguous copy of each slice;
# narrower groups (depthwise layers) stay on the direct kernels, which walk a group per block.
_GROUP_MIN = 8


def _per_group_ok(groups: int, c_in_group: int, c_out_group: int, n_spatial: int) -> bool:
    return groups > 1 and n_spatial >= 2 and c_in_group >= _GROUP_MIN and c_out_group >= _GROUP_MIN


def _stuffed(g: torch.Tensor, dense_sp, stride) -> torch.Tensor:
    """``g`` with ``stride - 1`` zeros between its cells: the output gradient of the stride-1 layer."""
    up = torch.zeros((g.shape[0], g.shape[1], *dense_sp), dtype=g.dtype, device=g.device)
    up[(slice(None), slice(None)) + tuple(slice(0, (o - 1) * s + 1, s) for o, s in zip(g.shape[2:], stride))] = g
    return up


def _single_launch(dtype, c_in, weight_shape, stride, padding, dilation, groups) -> bool:
    """True where conv_nd / conv_nd_weight hand the tensors to the C entry point as they are (no route that
    re-shapes the layer, copies channel slices or lays out patches first)."""
    n = len(weight_shape) - 2
    kernel = tuple(int(k) for k in weight_shape[2:])
    stride, padding, dilation = _tup(stride, n, "stride"), _tup(padding, n, "padding"), _tup(dilation, n, "dilation")
    if groups != 1:
        return not _per_group_ok(groups, int(weight_shape[1]), int(weight_shape[0]) // groups, n)
    if _dense_stride_ok(kernel, stride, dilation, padding) or _prepad(kernel, stride, padding, dilation) is not None:
        return False
    if _dilated_ok(kernel, stride, padding, dilation) or _big_kernel_ok(kernel, stride, dilation):
        return False
    if _embed3(kernel, stride, dilation) is not None:
        return False
    return not _patch_gemm_ok(dtype, c_in, int(weight_shape[0]), kernel, stride, padding, dilation)


def conv_nd(x, w, b=None, *, stride=1, padding=0, dilation=1, groups=1, out=None, workspace=None) -> torch.Tensor:
    """``F.conv{1,2,3}d(x, w, b, stride, padding, dilation, groups)`` on the HIP kernels.

    ``out`` / ``workspace`` (the result tensor and ``jg_conv_workspace_bytes`` bytes of scratch) let a caller
    that runs the same layer again and again bring its own buffers, so that the call allocates nothing; they
    are honoured where the layer runs as one launch on the given tensors and refused on the routes that
    re-shape the layer first."""
    _lib.require_gpu(x, w, b)
    if (out is not None or workspace is not None) and not _single_launch(x.dtype, x.shape[1], w.shape, stride, padding, dilation, groups):
        raise NotImplementedError("conv_nd: `out` / `workspace` are taken only where the layer is one launch on the given tensors")
    n = _check_args(x, w, groups, padding)
    if x.dim() != n + 2:
        raise ValueError(f"expected a batched (N, C, *spatial) input with {n} spatial axes, got {tuple(x.shape)}")
    if x.dtype != w.dtype or (b is not None and b.dtype != x.dtype):
        raise RuntimeError(f"Input type ({x.dtype}) and weight / bias type ({w.dtype}) should be the same")
    if x.shape[1] != w.shape[1] * groups:
        raise RuntimeError(f"expected input to have {w.shape[1] * groups} channels, but got {x.shape[1]} channels instead")
    stride, padding, dilation = _tup(stride, n, "stride"), _tup(padding, n, "padding"), _tup(dilation, n, "dilation")
    if _per_group_ok(groups, w.shape[1], w.shape[0] // groups, n):
        cg, mg = w.shape[1], w.shape[0] // groups
        return torch.cat([
            conv_nd(x[:, i * cg:(i + 1) * cg].contiguous(), w[i * mg:(i + 1) * mg], None if b is None else b[i * mg:(i + 1) * mg],
                    stride=stride, padding=padding, dilation=dilation)
            for i in range(groups)], dim=1)
    plain = groups == 1  # the routes below re-shape ungrouped layers; narrow groups run the direct kernels as they are
    if plain and _dense_stride_ok(tuple(w.shape[2:]), stride, dilation, padding):
        out_sp = _out_spatial(x.shape[2:], w.shape[2:], stride, padding, dilation)
        dense = conv_nd(x, w, b, stride=1, padding=padding, dilation=dilation)
        return dense[(slice(None), slice(None)) + tuple(slice(0, (o - 1) * s + 1, s) for o, s in zip(out_sp, stride))].contiguous()
    extra = _prepad(tuple(w.shape[2:]), stride, padding, dilation) if plain else None
    if extra is not None:
        return conv_nd(_zero_rim(x, extra), w, b, stride=1, padding=tuple(p - e for p, e in zip(padding, extra)), dilation=dilation)
    if plain and _dilated_ok(tuple(w.shape[2:]), stride, padding, dilation):
        phases = _phase_counts(w.shape[2:], dilation)
        out_sp = _out_spatial(x.shape[2:], w.shape[2:], stride, padding, dilation)
        ext_in = tuple(-(-int(i) // p) for i, p in zip(x.shape[2:], phases))
        yb = conv_nd(_to_phases(x, phases, ext_in), w, b, stride=1, padding=tuple(pp // p for pp, p in zip(padding, phases)))
        return _from_phases(yb, phases, x.shape[0], out_sp)
    if (plain and _big_kernel_ok(tuple(w.shape[2:]), stride, dilation)
            and _tap_blocks_fit(x.dtype, x.shape[0], x.shape[1], w.shape[2:], _out_spatial(x.shape[2:], w.shape[2:], stride, padding, dilation))):
        out_sp = _out_spatial(x.shape[2:], w.shape[2:], stride, padding, dilation)
        return conv_nd(_moved_copies(x, w.shape[2:], padding, out_sp), _tap_block_weight(w), b, stride=1, padding=0)
    off = _embed3(tuple(w.shape[2:]), stride, dilation) if plain else None
    if off is not None:
        return conv_nd(x, _embed_weight(w, off), b, stride=1, padding=tuple(p + o for p, o in zip(padding, off)))
    x, w = x.contiguous(), w.contiguous()
    b = None if b is None else b.contiguous()
    out_sp = _out_spatial(x.shape[2:], w.shape[2:], stride, padding, dilation)
    if plain and _patch_gemm_ok(x.dtype, x.shape[1], w.shape[0], w.shape[2:], stride, padding, dilation):
        y_tok = _proj_nt(_patchify(x, w.shape[2:], out_sp), w.reshape(w.shape[0], -1), b)
        return y_tok.reshape(x.shape[0], *out_sp, w.shape[0]).permute(0, n + 1, *range(1, n + 1)).contiguous()
    y = _out_tensor(out, (x.shape[0], w.shape[0], *out_sp), x.dtype, x.device, "conv_nd")
    desc = _desc(x.shape[0], x.shape[1], w.shape[0], x.shape[2:], w.shape[2:], stride, padding, dilation, groups)
    ws, nbytes = _workspace(desc, 0, x.dtype, x.device, workspace)
    rc = _lib.load().jg_conv_fwd(
        _lib.ptr(y), _lib.ptr(x), _lib.ptr(w), _lib.ptr(b), desc, _lib.dtype_code(x.dtype), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "jg_conv_fwd")
    return y


def conv_nd_input(input_shape, w, g, *, stride=1, padding=0, dilation=1, groups=1) -> torch.Tensor:
    """``torch.nn.grad.conv{1,2,3}d_input(input_shape, w, g, ...)`` on the HIP kernels."""
    _lib.require_gpu(w, g)
    n = _check_args(g, w, groups, padding)
    input_shape = tuple(int(v) for v in input_shape)
    if len(input_shape) != n + 2:
        raise ValueError(f"input_shape must have {n + 2} entries, got {input_shape}")
    if g.dtype != w.dtype:
        raise RuntimeError(f"grad_output type ({g.dtype}) and weight type ({w.dtype}) should be the same")
    stride, padding, dilation = _tup(stride, n, "stride"), _tup(padding, n, "padding"), _tup(dilation, n, "dilation")
    if input_shape[1] != w.shape[1] * groups:
        raise ValueError(f"input_shape has {input_shape[1]} channels, the weight takes {w.shape[1] * groups}")
    if _per_group_ok(groups, w.shape[1], w.shape[0] // groups, n):
        cg, mg = w.shape[1], w.shape[0] // groups
        if g.shape[1] != w.shape[0]:
            raise ValueError(f"grad_output has {g.shape[1]} channels, the weight produces {w.shape[0]}")
        return torch.cat([
            conv_nd_input((input_shape[0], cg, *input_shape[2:]), w[i * mg:(i + 1) * mg], g[:, i * mg:(i + 1) * mg].contiguous(),
                          stride=stride, padding=padding, dilation=dilation)
            for i in range(groups)], dim=1)
    plain = groups == 1  # as in conv_nd
    if plain and _dense_stride_ok(tuple(w.shape[2:]), stride, dilation, padding):
        dense_sp = _out_spatial(input_shape[2:], w.shape[2:], (1,) * n, padding, dilation)
        return conv_nd_input(input_shape, w, _stuffed(g, dense_sp, stride), stride=1, padding=padding, dilation=dilation)
    extra = _prepad(tuple(w.shape[2:]), stride, padding, dilation) if plain else None
    if extra is not None:
        rimmed = input_shape[:2] + tuple(v + 2 * e for v, e in zip(input_shape[2:], extra))
        gxr = conv_nd_input(rimmed, w, g, stride=1, padding=tuple(p - e for p, e in zip(padding, extra)), dilation=dilation)
        return gxr[(slice(None), slice(None)) + tuple(slice(e, e + v) for v, e in zip(input_shape[2:], extra))].contiguous()
    if plain and _dilated_ok(tuple(w.shape[2:]), stride, padding, dilation):
        phases = _phase_counts(w.shape[2:], dilation)
        out_sp = _out_spatial(input_shape[2:], w.shape[2:], stride, padding, dilation)
        if tuple(g.shape) != (input_shape[0], w.shape[0], *out_sp):
            raise ValueError(f"grad_output shape {tuple(g.shape)} does not match the convolution of an input of shape {input_shape}")
        ext_in = tuple(-(-i // p) for i, p in zip(input_shape[2:], phases))
        pad0 = tuple(pp // p for pp, p in zip(padding, phases))
        ext_out = _out_spatial(ext_in, w.shape[2:], (1,) * n, pad0, (1,) * n)
        gxb = conv_nd_input((g.shape[0] * math.prod(phases), input_shape[1], *ext_in), w, _to_phases(g, phases, ext_out),
                            stride=1, padding=pad0)
        return _from_phases(gxb, phases, input_shape[0], input_shape[2:])
    if (plain and _big_kernel_ok(tuple(w.shape[2:]), stride, dilation) and all(p <= k - 1 for p, k in zip(padding, w.shape[2:]))
            and _tap_blocks_fit(g.dtype, g.shape[0], w.shape[0], w.shape[2:], input_shape[2:])):
        out_sp = _out_spatial(input_shape[2:], w.shape[2:], stride, padding, dilation)
        if tuple(g.shape) != (input_shape[0], w.shape[0], *out_sp):
            raise ValueError(f"grad_output shape {tuple(g.shape)} does not match the convolution of an input of shape {input_shape}")
        # the forward of g under the transposed kernel with its taps reversed, padded by k - 1 - p
        back = w.transpose(0, 1).flip(*range(2, 2 + n))
        return conv_nd(g, back, None, stride=1, padding=tuple(k - 1 - p for p, k in zip(padding, w.shape[2:])))
    off = _embed3(tuple(w.shape[2:]), stride, dilation) if plain else None
    if off is not None:
        return conv_nd_input(input_shape, _embed_weight(w, off), g, stride=1,
                             padding=tuple(p + o for p, o in zip(padding, off)))
    g, w = g.contiguous(), w.contiguous()
    out_sp = _out_spatial(input_shape[2:], w.shape[2:], stride, padding, dilation)
    if tuple(g.shape) != (input_shape[0], w.shape[0], *out_sp):
        raise ValueError(
            f"grad_output shape {tuple(g.shape)} does not match the convolution of an input of shape {input_shape} "
            f"(expected {(input_shape[0], w.shape[0], *out_sp)})"
        )
    if plain and _patch_gemm_ok(g.dtype, w.shape[1], w.shape[0], w.shape[2:], stride, padding, dilation):
        # gradient of every patch = g_tokens x W, then back to the image layout
        w2t = w.reshape(w.shape[0], -1).t().contiguous()
        return _unpatchify(_proj_nt(_tokens_of(g).contiguous(), w2t, None), input_shape, w.shape[2:], out_sp)
    gx = torch.empty(input_shape, dtype=g.dtype, device=g.device)
    desc = _desc(input_shape[0], input_shape[1], w.shape[0], input_shape[2:], w.shape[2:], stride, padding, dilation, groups)
    ws, nbytes = _workspace(desc, 1, g.dtype, g.device)
    rc = _lib.load().jg_conv_dgrad(
        _lib.ptr(gx), _lib.ptr(w), _lib.ptr(g), desc, _lib.dtype_code(g.dtype), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(g.device),
    )
    _lib.check(rc, "jg_conv_dgrad")
    return gx


def _framed_desc(x_tile, geom: HaloGeometry, w, stride, padding, dilation, groups):
    n = geom.n_spatial
    stride, padding, dilation = _tup(stride, n, "stride"), _tup(padding, n, "padding"), _tup(dilation, n, "dilation")
    if tuple(x_tile.shape[2:]) != tuple(geom.size):
        raise ValueError(f"own tile {tuple(x_tile.shape[2:])} does not match the geometry {geom.size}")
    desc = _desc(x_tile.shape[0], x_tile.shape[1], w.shape[0] if hasattr(w, "shape") else w[0], geom.padded,
                 (w.shape if hasattr(w, "shape") else w)[2:], stride, padding, dilation, groups)
    return desc, stride, padding, dilation


def frame_bands(x_tile, geom: HaloGeometry, weight_shape, *, stride=1, padding=0, dilation=1, groups=1):
    """``(band_lo, band_hi)`` per spatial axis: the frame of the padded tile that the framed
    convolution kernels read (everything else comes from the own tile), or ``None`` where
    only the unframed kernels cover the problem."""
    _lib.require_gpu(x_tile)
    weight_shape = tuple(int(v) for v in weight_shape)
    desc, *_ = _framed_desc(x_tile, geom, weight_shape, stride, padding, dilation, groups)
    lo, hi = (ctypes.c_int32 * 3)(), (ctypes.c_int32 * 3)()
    cg = geom.c_geom(int(x_tile.shape[0]) * int(x_tile.shape[1]))
    rc = _lib.load().jg_conv_frame_bands(desc, cg, _lib.dtype_code(x_tile.dtype), lo, hi)
    if rc == -2:
        return None
    _lib.check(rc, "jg_conv_frame_bands")
    pad = 3 - geom.n_spatial
    return tuple(lo[pad:]), tuple(hi[pad:])


def conv_nd_framed(x_frame, x_tile, geom: HaloGeometry, w, b=None, *, stride=1, padding=0, dilation=1, groups=1):
    """``conv_nd`` on the padded tile of which only the frame (``frame_bands``) holds data:
    windows inside the own tile are read from ``x_tile``. Same bits as ``conv_nd`` on the
    fully assembled tile. Returns ``None`` where only the unframed kernel exists."""
    _lib.require_gpu(x_frame, x_tile, w)
    n = _check_args(x_frame, w, groups, padding)
    x_tile, w = x_tile.contiguous(), w.contiguous()
    desc, stride, padding, dilation = _framed_desc(x_tile, geom, w, stride, padding, dilation, groups)
    if tuple(x_frame.shape) != (x_tile.shape[0], x_tile.shape[1], *geom.padded) or not x_frame.is_contiguous():
        raise ValueError("conv_nd_framed: x_frame must be the contiguous padded tensor of the geometry")
    if b is not None:
        b = b.contiguous()
    out_sp = _out_spatial(geom.padded, w.shape[2:], stride, padding, dilation)
    y = torch.empty((x_tile.shape[0], w.shape[0], *out_sp), dtype=x_tile.dtype, device=x_tile.device)
    ws, nbytes = _workspace(desc, 0, x_tile.dtype, x_tile.device)
    rc = _lib.load().jg_conv_fwd_framed(
        _lib.ptr(y), _lib.ptr(x_frame), _lib.ptr(x_tile), _lib.ptr(w), _lib.ptr(b), desc,
        geom.c_geom(int(x_tile.shape[0]) * int(x_tile.shape[1])), _lib.dtype_code(x_tile.dtype), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(x_tile.device),
    )
    if rc == -2:
        return None
    _lib.check(rc, "jg_conv_fwd_framed")
    return y


def conv_nd_weight_framed(x_frame, x_tile, geom: HaloGeometry, weight_shape, g, *, stride=1, padding=0, dilation=1,
                          groups=1, with_bias_grad=False):
    """``conv_nd_weight`` (optionally with the bias gradient) on a framed input, see
    ``conv_nd_framed``. Returns ``None`` where only the unframed kernel exists."""
    _lib.require_gpu(x_frame, x_tile, g)
    weight_shape = tuple(int(v) for v in weight_shape)
    if x_tile.dtype != g.dtype:
        raise RuntimeError(f"input type ({x_tile.dtype}) and grad_output type ({g.dtype}) should be the same")
    x_tile, g = x_tile.contiguous(), g.contiguous()
    desc, stride, padding, dilation = _framed_desc(x_tile, geom, weight_shape, stride, padding, dilation, groups)
    out_sp = _out_spatial(geom.padded, weight_shape[2:], stride, padding, dilation)
    if tuple(g.shape) != (x_tile.shape[0], weight_shape[0], *out_sp) or x_tile.shape[1] != weight_shape[1]:
        raise ValueError(f"grad_output {tuple(g.shape)} / tile {tuple(x_tile.shape)} do not match weight {weight_shape}")
    gw = torch.empty(weight_shape, dtype=g.dtype, device=g.device)
    gb = torch.empty(weight_shape[0], dtype=g.dtype, device=g.device) if with_bias_grad else None
    ws, nbytes = _workspace(desc, 2, g.dtype, g.device)
    rc = _lib.load().jg_conv_wgrad_framed(
        _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(x_frame), _lib.ptr(x_tile), _lib.ptr(g), desc,
        geom.c_geom(int(x_tile.shape[0]) * int(x_tile.shape[1])), _lib.dtype_code(g.dtype), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(g.device),
    )
    if rc == -2:
        return None
    _lib.check(rc, "jg_conv_wgrad_framed")
    return (gw, gb) if with_bias_grad else gw


def conv_nd_input_fold(geom: HaloGeometry, w, g, *, stride=1, padding=0, dilation=1, groups=1, present=None,
                       out=None, workspace=None):
    """Input gradient of the convolution on the halo-padded tile, written to its owners.

    Equivalent to ``conv_nd_input`` on the padded shape followed by
    ``halo_pack(from_padded=True)``, without the padded gradient reaching memory:
    returns ``(gx, send)`` where ``gx`` (N, Cin, *geom.size) holds ``0 + own`` in every
    cell and ``send[offset]`` is the halo block owned by that neighbour (only the
    offsets in ``present``, all by default). ``halo_fold_border_`` finishes the fold
    once the neighbours' blocks have arrived. Returns ``None`` where only the
    unfused kernels cover the problem. ``out = (gx, send)`` of an earlier call with the same
    arguments and ``workspace`` are written again instead of new tensors.
    """
    _lib.require_gpu(w, g)
    n = _check_args(g, w, groups, padding)
    if g.dtype != w.dtype:
        raise RuntimeError(f"grad_output type ({g.dtype}) and weight type ({w.dtype}) should be the same")
    if geom.n_spatial != n:
        raise ValueError(f"geometry has {geom.n_spatial} spatial axes, the convolution {n}")
    if g.dtype != torch.bfloat16 or groups != 1:  # the fold epilogue exists for ungrouped bf16 layers: say so before sizing a workspace
        return None
    stride, padding, dilation = _tup(stride, n, "stride"), _tup(padding, n, "padding"), _tup(dilation, n, "dilation")
    g, w = g.contiguous(), w.contiguous()
    batch, c_in = int(g.shape[0]), int(w.shape[1]) * groups
    padded = geom.padded
    out_sp = _out_spatial(padded, w.shape[2:], stride, padding, dilation)
    if tuple(g.shape) != (batch, w.shape[0], *out_sp):
        raise ValueError(
            f"grad_output shape {tuple(g.shape)} does not match the convolution of a padded tile {padded} "
            f"(expected {(batch, w.shape[0], *out_sp)})"
        )
    desc = _desc(batch, c_in, w.shape[0], padded, w.shape[2:], stride, padding, dilation, groups)
    ws, nbytes = _workspace(desc, 1, g.dtype, g.device, workspace)
    lead = (batch, c_in)
    offs = geom.offsets() if present is None else [tuple(o) for o in present]
    if out is None:
        send, tab = new_strips(geom, "pack_bwd", lead, offs, g.dtype, g.device)
        gx = torch.empty(lead + geom.size, dtype=g.dtype, device=g.device)
    else:
        gx, send = out
        gx = _out_tensor(gx, lead + geom.size, g.dtype, g.device, "conv_nd_input_fold")
        if set(send) != set(offs):
            raise ValueError("conv_nd_input_fold: `out` holds strips for other offsets than `present`")
        tab = strip_table(send, geom, "pack_bwd", lead, g)
    rc = _lib.load().jg_conv_dgrad_fold(
        _lib.ptr(gx), tab, _lib.ptr(w), _lib.ptr(g), desc, geom.c_geom(batch * c_in), _lib.dtype_code(g.dtype),
        _lib.ptr(ws), nbytes, _lib.stream_ptr(g.device),
    )
    if rc == -2:  # only the unfused kernels cover this geometry / dtype
        return None
    _lib.check(rc, "jg_conv_dgrad_fold")
    return gx, send


def conv_nd_weight(x, weight_shape, g, *, stride=1, padding=0, dilation=1, groups=1, with_bias_grad=False,
                   out=None, workspace=None):
    """``torch.nn.grad.conv{1,2,3}d_weight(x, weight_shape, g, ...)`` on the HIP kernels.

    ``with_bias_grad=True`` returns ``(gw, gb)`` with ``gb = g.sum`` over batch and pixels
    (config.py:117-120), from the same pass over ``g`` where the MFMA kernel covers the shape.
    ``out`` (``gw``, or ``(gw, gb)`` with the bias gradient) and ``workspace`` as for :func:`conv_nd`.
    """
    _lib.require_gpu(x, g)
    weight_shape = tuple(int(v) for v in weight_shape)
    n = len(weight_shape) - 2
    if (out is not None or workspace is not None) and not _single_launch(x.dtype, x.shape[1], weight_shape, stride, padding, dilation, groups):
        raise NotImplementedError("conv_nd_weight: `out` / `workspace` are taken only where the layer is one launch on the given tensors")
    out_w, out_b = (out if with_bias_grad else (out, None)) if out is not None else (None, None)
    if isinstance(padding, str):
        raise NotImplementedError(f"string padding ({padding!r}) is not supported; pass per-axis integers")
    if not isinstance(groups, int) or groups < 1 or weight_shape[0] % groups:
        raise ValueError(f"groups = {groups} must be a positive integer that divides the {weight_shape[0]} output channels")
    if x.dtype != g.dtype:
        raise RuntimeError(f"input type ({x.dtype}) and grad_output type ({g.dtype}) should be the same")
    stride, padding, dilation = _tup(stride, n, "stride"), _tup(padding, n, "padding"), _tup(dilation, n, "dilation")
    if _per_group_ok(groups, weight_shape[1], weight_shape[0] // groups, n):
        cg, mg = weight_shape[1], weight_shape[0] // groups
        if x.shape[1] != cg * groups or g.shape[1] != weight_shape[0]:
            raise ValueError(f"{x.shape[1]} input and {g.shape[1]} output channels do not fit a weight of shape {weight_shape} in {groups} groups")
        parts = [conv_nd_weight(x[:, i * cg:(i + 1) * cg].contiguous(), (mg, cg, *weight_shape[2:]), g[:, i * mg:(i + 1) * mg].contiguous(),
                                stride=stride, padding=padding, dilation=dilation, with_bias_grad=with_bias_grad)
                 for i in range(groups)]
        if with_bias_grad:
            return torch.cat([gw for gw, _ in parts], dim=0), torch.cat([gb for _, gb in parts], dim=0)
        return torch.cat(parts, dim=0)
    plain = groups == 1  # as in conv_nd
    if plain and _dense_stride_ok(weight_shape[2:], stride, dilation, padding):
        dense_sp = _out_spatial(x.shape[2:], weight_shape[2:], (1,) * n, padding, dilation)
        return conv_nd_weight(x, weight_shape, _stuffed(g, dense_sp, stride), stride=1, padding=padding, dilation=dilation,
                              with_bias_grad=with_bias_grad)
    extra = _prepad(weight_shape[2:], stride, padding, dilation) if plain else None
    if extra is not None:
        return conv_nd_weight(_zero_rim(x, extra), weight_shape, g, stride=1, padding=tuple(p - e for p, e in zip(padding, extra)),
                              dilation=dilation, with_bias_grad=with_bias_grad)
    if plain and _dilated_ok(weight_shape[2:], stride, padding, dilation):
        phases = _phase_counts(weight_shape[2:], dilation)
        out_sp = _out_spatial(x.shape[2:], weight_shape[2:], stride, padding, dilation)
        if tuple(g.shape) != (x.shape[0], weight_shape[0], *out_sp) or x.shape[1] != weight_shape[1]:
            raise ValueError(f"grad_output {tuple(g.shape)} / input {tuple(x.shape)} do not match weight {weight_shape}")
        ext_in = tuple(-(-int(i) // p) for i, p in zip(x.shape[2:], phases))
        pad0 = tuple(pp // p for pp, p in zip(padding, phases))
        ext_out = _out_spatial(ext_in, weight_shape[2:], (1,) * n, pad0, (1,) * n)
        # every residue image is one more batch entry of the undilated layer: the sum over the batch is the answer
        return conv_nd_weight(_to_phases(x, phases, ext_in), weight_shape, _to_phases(g, phases, ext_out), stride=1,
                              padding=pad0, with_bias_grad=with_bias_grad)
    if (plain and _big_kernel_ok(weight_shape[2:], stride, dilation)
            and _tap_blocks_fit(x.dtype, x.shape[0], x.shape[1], weight_shape[2:], _out_spatial(x.shape[2:], weight_shape[2:], stride, padding, dilation))):
        out_sp = _out_spatial(x.shape[2:], weight_shape[2:], stride, padding, dilation)
        if tuple(g.shape) != (x.shape[0], weight_shape[0], *out_sp) or x.shape[1] != weight_shape[1]:
            raise ValueError(f"grad_output {tuple(g.shape)} / input {tuple(x.shape)} do not match weight {weight_shape}")
        moved = _moved_copies(x, weight_shape[2:], padding, out_sp)
        res = conv_nd_weight(moved, (weight_shape[0], moved.shape[1]) + (3,) * n, g, stride=1, padding=0,
                             with_bias_grad=with_bias_grad)
        gw = _from_tap_blocks(res[0] if with_bias_grad else res, weight_shape)
        return (gw, res[1]) if with_bias_grad else gw
    off = _embed3(weight_shape[2:], stride, dilation) if plain else None
    if off is not None:
        # gradient of the 3 x 3 (x 3) kernel the weights sit in; its centre taps are the answer
        res = conv_nd_weight(x, weight_shape[:2] + (3,) * n, g, stride=1,
                             padding=tuple(p + o for p, o in zip(padding, off)), with_bias_grad=with_bias_grad)
        gw3 = res[0] if with_bias_grad else res
        gw = gw3[(slice(None), slice(None)) + tuple(slice(o, 3 - o) for o in off)].contiguous()
        return (gw, res[1]) if with_bias_grad else gw
    x, g = x.contiguous(), g.contiguous()
    out_sp = _out_spatial(x.shape[2:], weight_shape[2:], stride, padding, dilation)
    if tuple(g.shape) != (x.shape[0], weight_shape[0], *out_sp) or x.shape[1] != weight_shape[1] * groups:
        raise ValueError(f"grad_output {tuple(g.shape)} / input {tuple(x.shape)} do not match weight {weight_shape}")
    if plain and _patch_gemm_ok(x.dtype, weight_shape[1], weight_shape[0], weight_shape[2:], stride, padding, dilation):
        # gw = g_tokens^T x patches (contraction over the patches), the bias gradient from the same pass
        patches, g_tok = _patchify(x, weight_shape[2:], out_sp), _tokens_of(g).contiguous()
        rows, k = patches.shape
        lib = _lib.load()
        gw2 = torch.empty(weight_shape[0], k, dtype=x.dtype, device=x.device)
        gb = torch.empty(weight_shape[0], dtype=x.dtype, device=x.device) if with_bias_grad else None
        if rows:
            nb = int(lib.jg_proj_tn_workspace(rows, weight_shape[0], k))
            pws = torch.empty(max(nb, 16), dtype=torch.uint8, device=x.device)
            rc = lib.jg_proj_tn(_lib.ptr(gw2), _lib.ptr(gb), _lib.ptr(g_tok), _lib.ptr(patches), _lib.dtype_code(x.dtype),
                                _lib.dtype_code(x.dtype), rows, weight_shape[0], k, 0, 0, 1, 1, 1, 1, _lib.ptr(pws), nb, _lib.stream_ptr(x.device))
            _lib.check(rc, "jg_proj_tn")
        else:
            gw2.zero_()
            if gb is not None:
                gb.zero_()
        gw = gw2.reshape(weight_shape)
        return (gw, gb) if with_bias_grad else gw
    gw = _out_tensor(out_w, weight_shape, x.dtype, x.device, "conv_nd_weight")
    desc = _desc(x.shape[0], x.shape[1], weight_shape[0], x.shape[2:], weight_shape[2:], stride, padding, dilation, groups)
    ws, nbytes = _workspace(desc, 2, x.dtype, x.device, workspace)
    if with_bias_grad:
        # one pass over g for both gradients where the MFMA kernel covers the shape
        gb = _out_tensor(out_b, (weight_shape[0],), x.dtype, x.device, "conv_nd_weight (bias gradient)")
        rc = _lib.load().jg_conv_wgrad_bias(
            _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(x), _lib.ptr(g), desc, _lib.dtype_code(x.dtype), _lib.ptr(ws), nbytes,
            _lib.stream_ptr(x.device),
        )
        if rc != -2:
            _lib.check(rc, "jg_conv_wgrad_bias")
            return gw, gb
    rc = _lib.load().jg_conv_wgrad(
        _lib.ptr(gw), _lib.ptr(x), _lib.ptr(g), desc, _lib.dtype_code(x.dtype), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "jg_conv_wgrad")
    if with_bias_grad:
        gb_sep = sum_grad_bias(g, n)
        return gw, (gb_sep if out_b is None else out_b.copy_(gb_sep))
    return gw


def sum_grad_bias(g: torch.Tensor, n_spatial: int) -> torch.Tensor:
    """``grad_output.sum`` over batch and spatial axes (config.py:117-120)."""
    _lib.require_gpu(g)
    if g.dim() != n_spatial + 2:
        raise ValueError(f"expected (N, C, *spatial) with {n_spatial} spatial axes, got {tuple(g.shape)}")
    g = g.contiguous()
    batch, ch = g.shape[0], g.shape[1]
    spatial = 1
    for s in g.shape[2:]:
        spatial *= int(s)
    gb = torch.empty(ch, dtype=g.dtype, device=g.device)
    lib = _lib.load()
    nbytes = int(lib.jg_bias_grad_workspace_bytes(batch, ch, spatial))
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=g.device)
    rc = lib.jg_bias_grad(
        _lib.ptr(gb), _lib.ptr(g), batch, ch, spatial, _lib.dtype_code(g.dtype), _lib.ptr(ws), nbytes,
        _lib.stream_ptr(g.device),
    )
    _lib.check(rc, "jg_bias_grad")
    return gb


# --------------------------------------------------------------------------- #
# the distributed convolution of one rank
# --------------------------------------------------------------------------- #


class TileGroup:
    """One axis of the spatial mesh as seen from one rank: ``size()`` and ``rank()``,
    the two members of a process group the halo geometry needs."""

    def __init__(self, size: int, rank: int) -> None:
        if not 0 <= rank < size:
            raise ValueError(f"rank {rank} outside a group of {size}")
        self._size, self._rank = int(size), int(rank)

    def size(self) -> int:
        return self._size

    def rank(self) -> int:
        return self._rank


class HaloExchange(Protocol):
    """What moves strips between ranks. ``send`` maps a neighbour offset to the strip
    packed for it; the result maps the offset of each existing neighbour to the strip
    received from it. One implementation per transport; none lives in this module."""

    def forward(self, send: dict) -> dict: ...

    def backward(self, send: dict) -> dict: ...

    def along_axis(self, axis: int, send: list, backward: bool) -> list:
        """The exchange of ONE split axis for need spans the strips do not cover
        (``exchange_along_axis``, _common/halo.py:7-63): ``send[p]`` is the part cut for rank ``p`` of
        that axis' group (``None``: nothing, and always for the rank itself); returns what the peers cut
        for this rank, by peer. Only called where ``halo.spans_fit_the_strips`` says no."""
        ...


def _mesh_position(spatial_groups) -> tuple[tuple, tuple]:
    sizes = tuple(1 if g is None else int(g.size()) for g in spatial_groups)
    ranks = tuple(0 if g is None else int(g.rank()) for g in spatial_groups)
    return ranks, sizes


def _present_offsets(geom: HaloGeometry, ranks, sizes) -> list:
    out = []
    for o in geom.offsets():
        ok = True
        for a, v in enumerate(o):
            if v == 0:
                continue
            if sizes[a] <= 1 or not 0 <= ranks[a] + v < sizes[a]:
                ok = False
        if ok:
            out.append(o)
    return out


def _local_padding(padding, sizes) -> tuple:
    """Zero on split axes (jigsaw/modules/convolution/_common/spatial_split.py:75-82)."""
    return tuple(0 if s > 1 else p for p, s in zip(padding, sizes))


def _needs_halo(sizes, padding, dilation) -> bool:
    return any(s > 1 and (p != 0 or d != 1) for s, p, d in zip(sizes, padding, dilation))


def _frame_decision(config, x, geom: HaloGeometry, weight_shape, kwargs):
    """Bands of the frame when the framed kernels are asked for and cover the problem, else ``None``."""
    if not getattr(config, "framed", False) or config.conv_fn is not conv_nd or config.conv_weight_fn is not conv_nd_weight:
        return None
    if x.dtype != torch.bfloat16:
        return None
    return frame_bands(x, geom, weight_shape, **kwargs)


def conv_halo_nway(x, w, b, stride, padding, dilation, spatial_groups, channel_group, config):
    """Convolve with a halo exchange on every split axis; returns ``(y, x_aug)``.

    Same contract as ``conv_halo_nway``
    (jigsaw/modules/convolution/_conv/distributed.py:212-293) for a channel-local
    layer: ``x_aug`` is the halo-padded tile kept for the backward pass.
    """
    if not isinstance(padding, tuple):
        raise NotImplementedError(
            "Distributed ConvNd with a halo exchange does not support "
            f"string padding ({padding!r}); pass an explicit per-axis padding."
        )
    if channel_group is not None and channel_group.size() != 1:
        raise NotImplementedError("channel-sharded convolution is outside this package (col must be 1)")
    n = config.n_spatial
    ranks, sizes = _mesh_position(spatial_groups)
    x = x.contiguous()
    kwargs = {"stride": stride, "padding": _local_padding(padding, sizes), "dilation": dilation, "groups": int(getattr(config, "groups_local", 1))}
    if not spans_fit_the_strips(x.shape[-n:], w.shape[-n:], stride, padding, dilation, sizes):
        # need spans that leave out owned rows or reach past the adjacent rank: one split axis at a
        # time, first to last, every peer's overlap copied in (distributed.py:264-275, halo.py:101-156)
        x_aug = x
        for a in range(n):
            if sizes[a] <= 1:
                continue
            x_aug = halo_gather_axis(x_aug, a - n, ranks[a], sizes[a], w.shape[a - n], stride[a], padding[a], dilation[a],
                                     lambda send, a=a: config.halo_exchange.along_axis(a, send, False))
        y = config.conv_fn(x_aug, w, b, **kwargs) if b is not None else config.conv_fn(x_aug, w, **kwargs)
        return y, x_aug
    geom = HaloGeometry.for_conv(x.shape[-n:], w.shape[-n:], stride, padding, dilation, ranks, sizes)
    present = _present_offsets(geom, ranks, sizes)
    send = halo_pack(x, geom, from_padded=False, present=present) if present else {}
    recv = config.halo_exchange.forward(send) if present else {}
    bands = _frame_decision(config, x, geom, w.shape, kwargs)
    if bands is not None:
        # only the frame of the padded tile is built; the kernels read the tile itself elsewhere.
        # The padded tensor that is returned is then NOT a full copy: its consumer is
        # conv_halo_nway_backward with x_tile given (what _ConvNd of this module does).
        x_frame = halo_assemble(x, recv, geom, bands=bands)
        x_frame._jg_frame_only = True  # read by conv_halo_nway_backward: no weight gradient without the tile
        y = conv_nd_framed(x_frame, x, geom, w, b, **kwargs)
        if y is None:
            raise RuntimeError("framed forward: " + _lib.load().jg_last_error().decode())
        return y, x_frame
    x_aug = halo_assemble(x, recv, geom)
    y = config.conv_fn(x_aug, w, b, **kwargs) if b is not None else config.conv_fn(x_aug, w, **kwargs)
    return y, x_aug


def conv_halo_nway_backward(
    grad_output, x_aug, weight, stride, padding, dilation, local_in_spatial, spatial_groups, channel_group, config,
    need=(True, True), x_tile=None,
):
    """Gradients of the halo-exchange convolution; returns ``(g_x or None, g_w or None)``.

    Same contract as ``conv_halo_nway_backward``
    (jigsaw/modules/convolution/_conv/distributed.py:296-396): dgrad on the padded
    shape, wgrad, then the halo gradients are folded onto their owners.
    """
    n = config.n_spatial
    ranks, sizes = _mesh_position(spatial_groups)
    local_padding = _local_padding(padding, sizes)
    need_x, need_w = need[0], need[1]
    # a third entry asks for the bias gradient too; the result then has three entries
    want_b = len(need) > 2
    need_b = want_b and need[2]
    g = grad_output.to(weight.dtype)
    kwargs = {"stride": stride, "padding": local_padding, "dilation": dilation, "groups": int(getattr(config, "groups_local", 1))}
    g_w = g_b = None
    if x_tile is None and need_w and getattr(config, "framed", False) and getattr(x_aug, "_jg_frame_only", False):
        raise RuntimeError(
            "x_aug is the frame of a framed forward (config.framed) and its interior is undefined: the weight "
            "gradient needs the rank's tile as x_tile=. Use _ConvNd of this package, which keeps the tile, or "
            "build the config without framed=True."
        )
    if x_tile is not None:
        # x_aug is the frame that the framed forward built (conv_halo_nway with config.framed)
        if need_w:
            geom_w = HaloGeometry.for_conv(local_in_spatial, weight.shape[-n:], stride, padding, dilation, ranks, sizes)
            res = conv_nd_weight_framed(x_aug, x_tile, geom_w, weight.shape, g, with_bias_grad=need_b, **kwargs)
            if res is None:
                raise RuntimeError(
                    "the framed forward was used but the framed weight gradient does not cover this case: "
                    + _lib.load().jg_last_error().decode()
                )
            g_w, g_b = res if need_b else (res, None)
        elif need_b:
            g_b = config.grad_bias(g.contiguous())
    elif need_w and need_b and config.conv_weight_fn is conv_nd_weight:
        g_w, g_b = conv_nd_weight(x_aug, weight.shape, g, with_bias_grad=True, **kwargs)
    else:
        g_w = config.conv_weight_fn(x_aug, weight.shape, g, **kwargs) if need_w else None
        g_b = config.grad_bias(g.contiguous()) if need_b else None
    done = (lambda gx: (gx, g_w, g_b)) if want_b else (lambda gx: (gx, g_w))
    if not need_x:
        return done(None)
    if not spans_fit_the_strips(local_in_spatial, weight.shape[-n:], stride, padding, dilation, sizes):
        # the general spans of the forward: fold one split axis at a time, last to first, the peers'
        # parts added in rank order (distributed.py:378-389, halo.py:195-251)
        g_x = config.conv_input_fn(x_aug.shape, weight, g, **kwargs)
        for a in reversed(range(n)):
            if sizes[a] <= 1:
                continue
            g_x = halo_scatter_add_axis(g_x, a - n, ranks[a], sizes[a], weight.shape[a - n], stride[a], padding[a], dilation[a],
                                        local_in_spatial[a], lambda send, a=a: config.halo_exchange.along_axis(a, send, True))
        return done(g_x)
    geom = HaloGeometry.for_conv(local_in_spatial, weight.shape[-n:], stride, padding, dilation, ranks, sizes)
    present = _present_offsets(geom, ranks, sizes)
    if getattr(config, "fused_fold", False) and config.conv_input_fn is conv_nd_input:
        # dgrad writes the owned cells and the send strips itself; same bits as the
        # three separate steps below
        fused = conv_nd_input_fold(geom, weight, g, present=present, **kwargs)
        if fused is not None:
            g_x, send = fused
            recv = config.halo_exchange.backward(send) if present else {}
            return done(halo_fold_border_(g_x, recv, geom))
    g_x_need = config.conv_input_fn(x_aug.shape, weight, g, **kwargs)
    send = halo_pack(g_x_need, geom, from_padded=True, present=present) if present else {}
    recv = config.halo_exchange.backward(send) if present else {}
    g_x = halo_fold(g_x_need, recv, geom)
    return done(g_x)


_CHANNEL_COMMS = ("auto", "all_to_all", "isend", "batch_isend_irecv")


def _resolve_channel_comm(channel_comm: Any, device: Any) -> str:
    """The string a layer finds in ``config.channel_comm`` (and hands back when it rebuilds
    the config for a new channel group): ``"all_gather"`` is kept, ``"auto"`` becomes the
    transport of the device, unknown names raise ``ValueError``
    (jigsaw/modules/convolution/_common/channel_comm.py:25-58, jigsaw/_core/comm.py:101-137)."""
    if channel_comm == "all_gather":
        return "all_gather"
    name = str(getattr(channel_comm, "value", channel_comm)).lower()
    if name not in _CHANNEL_COMMS:
        raise ValueError(f"channel_comm must be 'all_gather' or one of {list(_CHANNEL_COMMS)}, got {channel_comm!r}")
    kind = getattr(device, "type", str(device).split(":")[0]) if device is not None else "cuda"
    if kind not in ("cuda", "cpu"):
        raise ValueError(f"Unsupported device {kind}")
    if name == "auto":
        return "all_to_all" if kind == "cuda" else "batch_isend_irecv"
    if name == "all_to_all" and kind != "cuda":
        raise ValueError(f"comm='all_to_all' needs a GPU, got device {kind!r}; use 'isend' or 'batch_isend_irecv'")
    return name


def layer_key(channel_group: Any, bias: Any, kernel_size, stride, groups: int) -> dict:
    """The properties of a layer a kernel table is built for; the reference's layers compare
    them entry by entry with their own and refuse a table built for another layer
    (jigsaw/modules/convolution/_common/config.py:9-43, jigsaw/_core/config.py:6-34)."""
    return {
        "n_spatial": len(kernel_size),
        "bias": bias is not None,
        "kernel_size == stride": tuple(kernel_size) == tuple(stride),
        "groups": groups,
        "channel group size": channel_group.size(),
    }


class _HipLayerConfig:
    """What the two kernel tables share: the constructor arguments of the reference's
    configs in their order (a layer rebuilds its config as
    ``type(config)(channel_group, bias, kernel_size, stride, device, channel_comm, groups)``,
    jigsaw/modules/convolution/_conv/base.py:572-580), the ``_layer_key`` the layer
    validates, and the options of this package, which live on the CLASS so that such a
    rebuild keeps them (see :meth:`bound`)."""

    vmapped = False
    halo_exchange: HaloExchange | None = None  # transport of the strips; None on a 1 x ... x 1 mesh

    def __init__(self, channel_group: Any, bias: Any, kernel_size, stride, device: Any = None,
                 channel_comm: Any = "auto", groups: int = 1, **options: Any) -> None:
        unknown = set(options) - set(self._OPTIONS)
        if unknown:
            raise TypeError(f"unknown option(s) {sorted(unknown)}; this config takes {list(self._OPTIONS)}")
        for name, value in options.items():
            setattr(self, name, value)
        kernel_size, stride = tuple(kernel_size), tuple(stride)
        if len(kernel_size) != len(stride):
            raise ValueError(f"kernel_size {kernel_size} and stride {stride} differ in length")
        self.n_spatial = len(kernel_size)
        self.channel_comm = _resolve_channel_comm(channel_comm, device)
        self.groups = int(groups)
        self._layer_key = layer_key(channel_group, bias, kernel_size, stride, groups)
        size = channel_group.size()
        self.channel_local = groups % size == 0
        self.groups_local = groups // size if self.channel_local else 1
        if size != 1:
            raise NotImplementedError(
                f"the HIP kernel table covers channel-local layers (channel group size {size}); "
                "channel-sharded convolution is outside this package"
            )
        self.grad_bias = self._no_bias if bias is None else self._sum_grad_bias

    @classmethod
    def bound(cls, **options: Any):
        """A subclass with ``options`` (``halo_exchange=...``, ...) as class attributes, for
        layers that rebuild their config from its type."""
        unknown = set(options) - set(cls._OPTIONS)
        if unknown:
            raise TypeError(f"unknown option(s) {sorted(unknown)}; this config takes {list(cls._OPTIONS)}")
        return type(cls.__name__, (cls,), dict(options))

    @classmethod
    def for_rank(cls, n_spatial: int, bias: Any, halo_exchange: HaloExchange | None = None, groups: int = 1,
                 **options: Any):
        """Short form for a channel-local layer whose kernel is not its stride (the layers
        that exchange halos): only the number of spatial axes, the bias and ``groups`` matter."""
        return cls(TileGroup(1, 0), bias, (3,) * int(n_spatial), (1,) * int(n_spatial), None, groups=groups,
                   halo_exchange=halo_exchange, **options)

    def _no_bias(self, *args: Any, **kwargs: Any) -> None:
        return None

    def _sum_grad_bias(self, grad_output: torch.Tensor) -> torch.Tensor:
        return sum_grad_bias(grad_output, self.n_spatial)


class HipConvNdConfig(_HipLayerConfig):
    """Kernel table of one distributed convolution layer, HIP edition: built like the
    reference's ``ConvNdConfig`` (config.py:32-95) and carrying the attributes the layer,
    ``_ConvNd`` and the two ``dist_conv_*`` functions read from it — ``_layer_key``,
    ``n_spatial``, ``channel_comm``, ``groups``, ``channel_local``, ``groups_local``,
    ``conv_fn``, ``native_conv_fn``, ``conv_input_fn``, ``conv_weight_fn``, ``grad_bias``,
    ``dist_conv_fn``, ``dist_conv_backward_fn`` — plus this package's options."""

    _OPTIONS = ("halo_exchange", "framed", "fused_fold", "fused_bias_grad")
    framed = False  # build only the frame of the padded tile (needs _ConvNd of this module, which keeps the tile)
    fused_fold = True  # dgrad + pack + fold in one pass where the MFMA kernel covers the shape
    fused_bias_grad = True  # bias gradient from the weight-gradient kernel's pass over g

    def __init__(self, channel_group: Any, bias: Any, kernel_size, stride, device: Any = None,
                 channel_comm: Any = "auto", groups: int = 1, **options: Any) -> None:
        super().__init__(channel_group, bias, kernel_size, stride, device, channel_comm, groups, **options)
        self.conv_fn = conv_nd
        self.native_conv_fn = conv_nd
        self.conv_input_fn = conv_nd_input
        self.conv_weight_fn = conv_nd_weight
        # kernel == stride tiles the domain without overlap; conv_halo_nway finds no strips
        # to exchange there and runs the local kernels only
        self.dist_conv_fn = conv_halo_nway
        self.dist_conv_backward_fn = conv_halo_nway_backward


def _cast_to_autocast_dtype(*tensors):
    """Matmul-family opt-in to autocast: cast down to the autocast dtype
    (jigsaw/_core/autocast.py:44-66)."""
    if not torch.is_autocast_enabled():
        return tensors
    dt = torch.get_autocast_dtype("cuda")
    return tuple(t if t is None or not t.is_floating_point() else t.to(dt) for t in tensors)


class _ConvNd(torch.autograd.Function):
    """Autograd function of the distributed convolution
    (jigsaw/modules/convolution/_conv/functional.py:28-169), HIP kernels inside."""

    @staticmethod
    def forward(x, weight, bias, stride, padding, dilation, spatial_groups, channel_group, config):  # noqa: D102
        x, weight, bias = _cast_to_autocast_dtype(x, weight, bias)
        return config.dist_conv_fn(
            x, weight, bias, stride=stride, padding=padding, dilation=dilation, spatial_groups=spatial_groups,
            channel_group=channel_group, config=config,
        )

    @staticmethod
    def setup_context(ctx, inputs, output):  # noqa: D102
        x, weight, bias, stride, padding, dilation, spatial_groups, channel_group, config = inputs
        _, x_aug = output
        ctx.mark_non_differentiable(x_aug)
        # the same decision conv_halo_nway took: x_aug is a frame only, so the tile is kept
        ctx.framed = False
        n = config.n_spatial
        ranks, sizes = _mesh_position(spatial_groups)
        if (getattr(config, "framed", False) and isinstance(padding, tuple)
                and spans_fit_the_strips(x.shape[-n:], weight.shape[-n:], stride, padding, dilation, sizes)):
            geom = HaloGeometry.for_conv(x.shape[-n:], weight.shape[-n:], stride, padding, dilation, ranks, sizes)
            kwargs = {"stride": stride, "padding": _local_padding(padding, sizes), "dilation": dilation, "groups": int(getattr(config, "groups_local", 1))}
            x_c = x if x.dtype == x_aug.dtype else torch.empty(0, dtype=x_aug.dtype, device=x.device).new_empty(x.shape)
            ctx.framed = _frame_decision(config, x_c, geom, weight.shape, kwargs) is not None
        if ctx.framed:
            ctx.save_for_backward(x_aug, weight, x)  # x_aug may be a frame only: keep the tile
        else:
            ctx.save_for_backward(x_aug, weight)
        ctx.spatial_groups, ctx.channel_group = spatial_groups, channel_group
        ctx.local_in_spatial = tuple(x.shape[-config.n_spatial :])
        ctx.stride, ctx.padding, ctx.dilation, ctx.config = stride, padding, dilation, config
        ctx.has_bias = bias is not None

    @staticmethod
    def backward(ctx, grad_output, grad_x_aug):  # noqa: D102
        config = ctx.config
        if ctx.framed:
            x_aug, weight, x_tile = ctx.saved_tensors
            x_tile = x_tile.to(x_aug.dtype)
            if weight.dtype != x_aug.dtype:
                # the forward ran in the autocast dtype, the backward runs in the weight's
                # (functional.py:126-129): the framed kernels do not cover that, so the tile
                # goes back into its frame and the padded tile takes the unframed route
                n = config.n_spatial
                ranks, sizes = _mesh_position(ctx.spatial_groups)
                geom = HaloGeometry.for_conv(ctx.local_in_spatial, weight.shape[-n:], ctx.stride, ctx.padding,
                                             ctx.dilation, ranks, sizes)
                x_aug = x_aug.clone()
                inner = tuple(slice(lo, lo + sz) for lo, sz in zip(geom.lo, geom.size))
                x_aug[(Ellipsis, *inner)] = x_tile
                x_tile = None
        else:
            (x_aug, weight), x_tile = ctx.saved_tensors, None
        x_aug = x_aug.to(weight.dtype)
        need_x, need_w, need_b = ctx.needs_input_grad[:3]
        need_b = need_b and ctx.has_bias
        if getattr(config, "fused_bias_grad", False):
            # the weight-gradient kernel adds up g on the way
            g_x, g_w, g_b = config.dist_conv_backward_fn(
                grad_output, x_aug, weight, ctx.stride, ctx.padding, ctx.dilation, ctx.local_in_spatial,
                ctx.spatial_groups, ctx.channel_group, config, need=(need_x, need_w, need_b),
                **({"x_tile": x_tile} if x_tile is not None else {}),
            )
        else:
            g_b = config.grad_bias(grad_output.contiguous()) if need_b else None
            g_x, g_w = config.dist_conv_backward_fn(
                grad_output, x_aug, weight, ctx.stride, ctx.padding, ctx.dilation, ctx.local_in_spatial,
                ctx.spatial_groups, ctx.channel_group, config, need=(need_x, need_w),
                **({"x_tile": x_tile} if x_tile is not None else {}),
            )
        return g_x, g_w, g_b, None, None, None, None, None, None


__all__ = [
    "HaloExchange",
    "HipConvNdConfig",
    "TileGroup",
    "layer_key",
    "_ConvNd",
    "conv_halo_nway",
    "conv_halo_nway_backward",
    "conv_nd",
    "conv_nd_input",
    "conv_nd_weight",
    "sum_grad_bias",
]
