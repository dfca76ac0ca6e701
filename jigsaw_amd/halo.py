"""Halo pack / assemble / fold of the halo-exchange convolution on the GPU.

Host-side mirror of jigsaw/modules/convolution/_conv/halo.py. The reference
pads one split axis at a time through an uneven all-to-all (``halo_gather``,
halo.py:66-156) and folds gradients back the same way (``halo_scatter_add``,
halo.py:159-251). Here the exchange is expressed once for all axes: a rank cuts
up to 8 (2-D) / 26 (3-D) strips for its neighbours (``halo_pack``), and builds
its padded tile from its own tile plus the strips it received in one pass
(``halo_assemble``); the backward direction cuts the halo blocks of the padded
gradient and folds the received ones in the reference's association order
(``halo_fold``). What travels between ranks is outside this module.
"""

from __future__ import annotations

import ctypes
import itertools
from dataclasses import dataclass
from typing import Mapping, Sequence

import torch

from . import _lib
from ._lib import AxisSegment, HaloGeom, VoidP27

Offset = tuple  # one entry in {-1, 0, 1} per spatial axis


def needed_input_span(
    rank: int,
    group_size: int,
    local_in_size: int,
    kernel: int,
    stride: int,
    padding: int,
    dilation: int,
) -> tuple[int, int, int, int]:
    """Return ``(lo, hi, need_size, out_local)`` of a rank's output block.

    Same contract as ``needed_input_span`` of
    jigsaw/modules/convolution/_conv/halo.py:9-63, including the
    ``NotImplementedError`` when the global output size does not divide by the
    group size.
    """
    extent = dilation * (kernel - 1) + 1
    global_out = (group_size * local_in_size + 2 * padding - extent) // stride + 1
    if global_out % group_size != 0:
        raise NotImplementedError(
            "Distributed convolution with a halo exchange needs the global "
            f"output size along the split axis ({global_out}) to be divisible by "
            f"the spatial group size ({group_size})."
        )
    out_local = global_out // group_size
    lo = rank * out_local * stride - padding
    need_size = (out_local - 1) * stride + extent
    return lo, lo + need_size, need_size, out_local


def halo_widths(
    rank: int, group_size: int, local_in_size: int, kernel: int, stride: int, padding: int, dilation: int
) -> tuple[int, int, int]:
    """``(lo_width, hi_width, out_local)`` of the need span around the owned rows.

    The widths may differ from rank to rank (a span that drifts against the tiles,
    ``out_local * stride != local size``, e.g. a convolution without padding). Accepted is
    what the fused kernels handle: the span covers the owned rows completely and starts
    at most one tile before / ends at most one tile after them, so that every strip
    comes from an adjacent rank. Anything else raises ``NotImplementedError``.
    """
    n = local_in_size
    lo, hi, _, out_local = needed_input_span(rank, group_size, n, kernel, stride, padding, dilation)
    lo_w = rank * n - lo
    hi_w = hi - (rank + 1) * n
    if lo_w < 0 or hi_w < 0:
        raise NotImplementedError(
            f"need span ({lo}, {hi}) of rank {rank} does not cover its owned rows [{rank * n}, {(rank + 1) * n})"
        )
    if lo_w > n or hi_w > n:
        raise NotImplementedError(
            f"halo ({lo_w}, {hi_w}) of rank {rank} wider than the tile ({n}): strips would come from non-adjacent ranks"
        )
    return lo_w, hi_w, out_local


def neighbour_widths(widths, rank: int, group_size: int) -> tuple[int, int, int, int]:
    """``(lo, hi, their_lo, their_hi)`` of a rank: its own halo widths, the lo width of
    the rank above and the hi width of the rank below (what those need of this rank's
    tile). ``widths(r)`` returns ``(lo, hi, ...)`` of rank ``r``; a side without a
    neighbour repeats the own width (nothing is sent there)."""
    lo, hi = widths(rank)[:2]
    their_lo = widths(rank + 1)[0] if rank + 1 < group_size else lo
    their_hi = widths(rank - 1)[1] if rank >= 1 else hi
    return lo, hi, their_lo, their_hi


def slot(offset: Sequence[int]) -> int:
    """Index of a neighbour offset in the 27-entry table of the C ABI."""
    o = (0,) * (3 - len(offset)) + tuple(int(v) for v in offset)
    if len(o) != 3 or any(v not in (-1, 0, 1) for v in o):
        raise ValueError(f"bad neighbour offset {tuple(offset)}")
    return (o[0] + 1) * 9 + (o[1] + 1) * 3 + (o[2] + 1)


@dataclass(frozen=True)
class HaloGeometry:
    """Tile size and halo widths of one rank (1 to 3 spatial axes).

    ``their_lo`` / ``their_hi`` are the halos the neighbours have of this rank's tile:
    the lo width of the rank above and the hi width of the rank below, per axis. They
    size what this rank sends forward and what it receives in the fold. ``None``: the
    same as ``lo`` / ``hi`` (every rank's span sits the same way around its tile)."""

    size: tuple  # interior extent per spatial axis
    lo: tuple  # halo in front of the interior
    hi: tuple  # halo behind the interior
    their_lo: tuple | None = None
    their_hi: tuple | None = None

    def __post_init__(self) -> None:
        ns = len(self.size)
        if not 1 <= ns <= 3 or len(self.lo) != ns or len(self.hi) != ns:
            raise ValueError("HaloGeometry needs 1 to 3 spatial axes with matching lo / hi")
        for name in ("their_lo", "their_hi"):
            v = getattr(self, name)
            if v is None:
                continue
            if len(v) != ns:
                raise ValueError(f"HaloGeometry: {name} needs one entry per spatial axis")
            if tuple(v) == tuple(self.lo if name == "their_lo" else self.hi):
                object.__setattr__(self, name, None)  # one spelling per geometry (cache keys, equality)
            else:
                object.__setattr__(self, name, tuple(int(x) for x in v))

    @property
    def n_spatial(self) -> int:
        return len(self.size)

    @property
    def padded(self) -> tuple:
        return tuple(l + n + h for l, n, h in zip(self.lo, self.size, self.hi))

    @property
    def same_on_every_rank(self) -> bool:
        return self.their_lo is None and self.their_hi is None

    def theirs(self) -> "HaloGeometry":
        """The geometry whose halos are the neighbours' halos of this tile."""
        if self.same_on_every_rank:
            return self
        return HaloGeometry(self.size, self.lo if self.their_lo is None else self.their_lo,
                            self.hi if self.their_hi is None else self.their_hi)

    def offsets(self) -> list:
        """All neighbour offsets except the rank itself."""
        return [o for o in itertools.product((-1, 0, 1), repeat=self.n_spatial) if any(o)]

    def strip_extent(self, offset: Sequence[int], verb: str) -> tuple:
        """Spatial extent of the strip of ``offset`` for ``verb``.

        ``assemble`` / ``pack_bwd``: (lo, size, hi) for offset (-1, 0, +1);
        ``fold`` / ``pack_fwd``: (their hi, size, their lo).
        """
        if verb in ("assemble", "pack_bwd"):
            pick = lambda a, o: (self.lo[a], self.size[a], self.hi[a])[o + 1]  # noqa: E731
        elif verb in ("fold", "pack_fwd"):
            t = self.theirs()
            pick = lambda a, o: (t.hi[a], t.size[a], t.lo[a])[o + 1]  # noqa: E731
        else:
            raise ValueError(f"unknown verb {verb!r}")
        return tuple(pick(a, o) for a, o in enumerate(offset))

    def c_geom(self, planes: int) -> HaloGeom:
        pad = 3 - self.n_spatial
        g = HaloGeom()
        g.planes = planes
        for a in range(3):
            if a < pad:
                g.size[a], g.lo[a], g.hi[a] = 1, 0, 0
            else:
                g.size[a], g.lo[a], g.hi[a] = self.size[a - pad], self.lo[a - pad], self.hi[a - pad]
        return g

    @classmethod
    def for_conv(
        cls,
        local_in_spatial: Sequence[int],
        kernel: Sequence[int],
        stride: Sequence[int],
        padding: Sequence[int],
        dilation: Sequence[int],
        ranks: Sequence[int],
        group_sizes: Sequence[int],
    ) -> "HaloGeometry":
        """Geometry of a rank's need span; axes with a group of one are not padded
        (the local conv pads them itself, spatial_split.py:75-82)."""
        lo, hi, tlo, thi = [], [], [], []
        for a, n in enumerate(local_in_spatial):
            if group_sizes[a] <= 1:
                for w in (lo, hi, tlo, thi):
                    w.append(0)
                continue
            args = (group_sizes[a], n, kernel[a], stride[a], padding[a], dilation[a])
            l, h, tl, th = neighbour_widths(lambda r: halo_widths(r, *args), ranks[a], group_sizes[a])  # noqa: B023
            lo.append(l)
            hi.append(h)
            tlo.append(tl)
            thi.append(th)
        return cls(tuple(int(n) for n in local_in_spatial), tuple(lo), tuple(hi), tuple(tlo), tuple(thi))


def _check_tile(x: torch.Tensor, spatial: tuple, what: str) -> int:
    ns = len(spatial)
    if x.dim() < ns + 1:
        raise ValueError(f"{what}: expected (..., C, {', '.join('S' * ns)}) but got shape {tuple(x.shape)}")
    if tuple(x.shape[-ns:]) != tuple(spatial):
        raise ValueError(f"{what}: spatial shape {tuple(x.shape[-ns:])} != expected {tuple(spatial)}")
    if not x.is_contiguous():
        raise ValueError(f"{what}: tensor must be contiguous")
    planes = 1
    for s in x.shape[:-ns]:
        planes *= int(s)
    return planes


def _table(
    strips: Mapping[Offset, torch.Tensor | None],
    geom: HaloGeometry,
    verb: str,
    lead: tuple,
    like: torch.Tensor,
    own: torch.Tensor | None,
) -> VoidP27:
    tab = VoidP27()
    for o in geom.offsets():
        t = strips.get(o)
        if t is None:
            continue
        want = lead + geom.strip_extent(o, verb)
        if tuple(t.shape) != want:
            raise ValueError(f"strip {o}: shape {tuple(t.shape)} != expected {want}")
        if t.dtype != like.dtype or t.device != like.device or not t.is_contiguous():
            raise ValueError(f"strip {o}: must be contiguous, {like.dtype}, on {like.device}")
        if t.numel():
            tab[slot(o)] = t.data_ptr()
    if own is not None:
        tab[13] = own.data_ptr()
    return tab


def halo_assemble(
    x: torch.Tensor,
    strips: Mapping[Offset, torch.Tensor | None],
    geom: HaloGeometry,
    out: torch.Tensor | None = None,
    bands: tuple | None = None,
) -> torch.Tensor:
    """Padded tile from the own tile and the strips received from the neighbours.

    A missing / ``None`` strip is a neighbour outside the domain and reads as
    zero (halo.py:77). Bit-exact copy, one pass over the destination.

    ``bands = (band_lo, band_hi)`` (one entry per spatial axis) writes only the
    frame of the padded tile: the cells within ``band_lo[a]`` of the start or
    ``band_hi[a]`` of the end of some axis. The rest of the result is left
    uninitialised; it is meant for the framed convolution functions, which read
    the own tile everywhere else (``conv.frame_bands``).
    """
    _lib.require_gpu(x)
    planes = _check_tile(x, geom.size, "halo_assemble")
    lead = tuple(x.shape[: -geom.n_spatial])
    if out is None:
        out = torch.empty(lead + geom.padded, dtype=x.dtype, device=x.device)
    elif tuple(out.shape) != lead + geom.padded or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("halo_assemble: `out` has the wrong shape / dtype / layout")
    tab = _table(strips, geom, "assemble", lead, x, x)
    cg = geom.c_geom(planes)
    if bands is None:
        rc = _lib.load().jg_halo_assemble_3d(_lib.ptr(out), tab, cg, x.element_size(), _lib.stream_ptr(x.device))
        _lib.check(rc, "jg_halo_assemble_3d")
        return out
    band_lo, band_hi = bands
    if len(band_lo) != geom.n_spatial or len(band_hi) != geom.n_spatial:
        raise ValueError("halo_assemble: `bands` needs one (lo, hi) entry per spatial axis")
    pad = 3 - geom.n_spatial
    c_lo = (ctypes.c_int32 * 3)(*([0] * pad + [int(v) for v in band_lo]))
    c_hi = (ctypes.c_int32 * 3)(*([0] * pad + [int(v) for v in band_hi]))
    rc = _lib.load().jg_halo_assemble_frame_3d(
        _lib.ptr(out), tab, cg, c_lo, c_hi, x.element_size(), _lib.stream_ptr(x.device)
    )
    _lib.check(rc, "jg_halo_assemble_frame_3d")
    return out


_LAYOUTS: dict = {}


def _strip_layout(geom: "HaloGeometry", verb: str, lead: tuple, offs: tuple, elem_size: int) -> tuple:
    """Where each strip of a pack sits in one flat buffer: ``(offset, shape, strides, start, count)`` per
    strip in elements, starts rounded up to 256 bytes, and the buffer's length. Cached per geometry."""
    key = (tuple(geom.size), tuple(geom.lo), tuple(geom.hi), geom.their_lo, geom.their_hi, verb, lead, offs, elem_size)
    hit = _LAYOUTS.get(key)
    if hit is not None:
        return hit
    per = 256 // elem_size
    rows, start = [], 0
    for o in offs:
        shape = lead + geom.strip_extent(o, verb)
        strides, count = [], 1
        for n in reversed(shape):
            strides.append(count)
            count *= n
        rows.append((o, shape, tuple(reversed(strides)), start, count))
        start += (count + per - 1) // per * per
    if len(_LAYOUTS) > 256:
        _LAYOUTS.clear()
    _LAYOUTS[key] = (tuple(rows), start)
    return _LAYOUTS[key]


def new_strips(geom: "HaloGeometry", verb: str, lead: tuple, offs: Sequence, dtype: torch.dtype, device) -> tuple:
    """Uninitialised strips for the offsets ``offs`` (``{offset: tensor}``) and the pointer table
    the C entry points take. One allocation holds them all, each strip a contiguous view that
    starts on a 256-byte boundary: 26 separate allocations cost more host time than the kernels
    that fill the strips take on the GPU."""
    elem = torch.empty((), dtype=dtype).element_size()
    layout, total = _strip_layout(geom, verb, tuple(lead), tuple(offs), elem)
    flat = torch.empty(total, dtype=dtype, device=device)
    base = flat.data_ptr()
    out: dict = {}
    tab = VoidP27()
    for o, shape, strides, start, count in layout:
        out[o] = flat.as_strided(shape, strides, start)
        if count:
            tab[slot(o)] = base + start * elem
    return out, tab


def strip_table(strips: Mapping[Offset, torch.Tensor], geom: "HaloGeometry", verb: str, lead: tuple, like: torch.Tensor) -> VoidP27:
    """The pointer table for strips that exist already (what :func:`new_strips` returned on an earlier
    call), each checked against the shape the geometry gives it."""
    tab = VoidP27()
    for o, t in strips.items():
        want = tuple(lead) + geom.strip_extent(o, verb)
        if tuple(t.shape) != want or t.dtype != like.dtype or t.device != like.device or not t.is_contiguous():
            raise ValueError(f"strip {o}: expected a contiguous {like.dtype} tensor of shape {want} on {like.device}")
        if t.numel():
            tab[slot(o)] = t.data_ptr()
    return tab


def halo_pack(
    src: torch.Tensor,
    geom: HaloGeometry,
    *,
    from_padded: bool,
    present: Sequence[Offset] | None = None,
    out: Mapping[Offset, torch.Tensor] | None = None,
) -> dict:
    """Cut the strips this rank sends, keyed by the neighbour's offset.

    ``from_padded=False``: ``src`` is the own tile, strips are the edge blocks the
    neighbours need for their halos (forward). ``from_padded=True``: ``src`` is a
    padded tensor (the dgrad of the padded tile) and strips are its halo blocks,
    owned by the neighbours (backward). ``present`` limits the offsets to the
    neighbours that exist. ``out``: the strips of an earlier call with the same
    arguments, filled again instead of new ones.
    """
    _lib.require_gpu(src)
    spatial = geom.padded if from_padded else geom.size
    planes = _check_tile(src, spatial, "halo_pack")
    lead = tuple(src.shape[: -geom.n_spatial])
    verb = "pack_bwd" if from_padded else "pack_fwd"
    offs = geom.offsets() if present is None else [tuple(o) for o in present]
    if out is None:
        out, tab = new_strips(geom, verb, lead, offs, src.dtype, src.device)
    else:
        if set(out) != set(tuple(o) for o in offs):
            raise ValueError("halo_pack: `out` holds strips for other offsets than `present`")
        tab = strip_table(out, geom, verb, lead, src)
    # forward: the blocks are sized by the neighbours' halos of this tile
    cg = (geom if from_padded else geom.theirs()).c_geom(planes)
    rc = _lib.load().jg_halo_pack_3d(
        tab, _lib.ptr(src), cg, int(from_padded), src.element_size(), _lib.stream_ptr(src.device)
    )
    _lib.check(rc, "jg_halo_pack_3d")
    return out


def halo_fold(
    gx_aug: torch.Tensor,
    strips: Mapping[Offset, torch.Tensor | None],
    geom: HaloGeometry,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Owned gradient from the padded gradient and the neighbours' halo blocks.

    Same result, bit for bit, as ``halo_scatter_add`` (halo.py:159-251) applied
    per split axis in reverse order (distributed.py:378-389).
    """
    _lib.require_gpu(gx_aug)
    planes = _check_tile(gx_aug, geom.padded, "halo_fold")
    lead = tuple(gx_aug.shape[: -geom.n_spatial])
    if out is None:
        out = torch.empty(lead + geom.size, dtype=gx_aug.dtype, device=gx_aug.device)
    elif tuple(out.shape) != lead + geom.size or out.dtype != gx_aug.dtype or not out.is_contiguous():
        raise ValueError("halo_fold: `out` has the wrong shape / dtype / layout")
    tab = _table(strips, geom, "fold", lead, gx_aug, None)
    cg = geom.c_geom(planes)
    if not geom.same_on_every_rank:
        # The neighbours' blocks are not as wide as the own halos: the own part first
        # (0 + own in every cell, the fold without neighbours), then the neighbours' blocks
        # by their widths. Same additions in the same order as the one-pass fold.
        rc = _lib.load().jg_halo_fold_3d(
            _lib.ptr(out), _lib.ptr(gx_aug), VoidP27(), cg, _lib.dtype_code(gx_aug.dtype), _lib.stream_ptr(gx_aug.device)
        )
        _lib.check(rc, "jg_halo_fold_3d")
        rc = _lib.load().jg_halo_fold_border_3d(
            _lib.ptr(out), tab, geom.theirs().c_geom(planes), _lib.dtype_code(out.dtype), _lib.stream_ptr(out.device)
        )
        _lib.check(rc, "jg_halo_fold_border_3d")
        return out
    rc = _lib.load().jg_halo_fold_3d(
        _lib.ptr(out), _lib.ptr(gx_aug), tab, cg, _lib.dtype_code(gx_aug.dtype), _lib.stream_ptr(gx_aug.device)
    )
    _lib.check(rc, "jg_halo_fold_3d")
    return out


def halo_fold_border_(
    gx: torch.Tensor,
    strips: Mapping[Offset, torch.Tensor | None],
    geom: HaloGeometry,
) -> torch.Tensor:
    """Second half of a fold whose own contributions are already in ``gx``.

    ``gx`` holds ``0 + own`` in every cell (what ``conv.conv_nd_input_fold``
    writes); the cells a neighbour reaches get the neighbours' halo blocks added in
    place, in the order of ``halo_scatter_add`` (halo.py:207-249,
    distributed.py:378-389), so the result has the bits of ``halo_fold``.
    """
    _lib.require_gpu(gx)
    planes = _check_tile(gx, geom.size, "halo_fold_border_")
    lead = tuple(gx.shape[: -geom.n_spatial])
    tab = _table(strips, geom, "fold", lead, gx, None)
    cg = geom.theirs().c_geom(planes)
    rc = _lib.load().jg_halo_fold_border_3d(
        _lib.ptr(gx), tab, cg, _lib.dtype_code(gx.dtype), _lib.stream_ptr(gx.device)
    )
    _lib.check(rc, "jg_halo_fold_border_3d")
    return gx


# --------------------------------------------------------------------------- #
# Need spans of any shape, one split axis at a time: the reference's own scheme
# (halo_gather / halo_scatter_add, _conv/halo.py:66-251, with exchange_along_axis,
# _common/halo.py:7-63). The fused strip functions above serve spans that hold the
# rank's own rows and reach at most one tile to either side; a span that leaves out
# owned rows (stride 2 without padding on an odd tile) or reaches further (a kernel
# wider than the tile) takes these.
# --------------------------------------------------------------------------- #
MAX_AXIS_SEGMENTS = 16


def spans_fit_the_strips(local_in_spatial, kernel, stride, padding, dilation, group_sizes) -> bool:
    """Whether EVERY rank's need span on every split axis holds its own rows and reaches one tile to
    either side at most: what the one-pass strip functions need. Decided for the whole group, so
    that all of its ranks exchange the same way. ``NotImplementedError`` for an output size the
    group does not divide (``needed_input_span``) passes through."""
    for a, n in enumerate(local_in_spatial):
        G = group_sizes[a]
        if G <= 1:
            continue
        for r in range(G):
            lo, hi, _, _ = needed_input_span(r, G, n, kernel[a], stride[a], padding[a], dilation[a])
            lo_w, hi_w = r * n - lo, hi - (r + 1) * n
            if lo_w < 0 or hi_w < 0 or lo_w > n or hi_w > n:
                return False
    return True


def span_overlap(lo: int, hi: int, peer: int, n: int, group_size: int) -> tuple[int, int]:
    """``(first row, count)`` of the rows of ``[lo, hi)`` that rank ``peer`` owns, in global rows
    (_conv/halo.py:134-138, 217-221: ``max(lo, peer * n, 0)`` to ``min(hi, (peer + 1) * n, G * n)``)."""
    r0 = max(lo, peer * n, 0)
    return r0, max(min(hi, (peer + 1) * n, group_size * n) - r0, 0)


def _axis_view(t: torch.Tensor, axis: int) -> tuple[int, int, int]:
    axis %= t.dim()
    outer = 1
    for v in t.shape[:axis]:
        outer *= int(v)
    inner = 1
    for v in t.shape[axis + 1:]:
        inner *= int(v)
    return outer, int(t.shape[axis]), inner


def _segments(parts, axis: int, like: torch.Tensor, dst_rows: int, what: str):
    """``(array, count, kept)`` for parts ``(tensor, src_start, dst_start, count)``; the tensors checked against
    ``like`` everywhere but along ``axis``."""
    axis %= like.dim()
    live = [p for p in parts if p[3] > 0]
    if len(live) > MAX_AXIS_SEGMENTS:
        raise NotImplementedError(f"{what}: {len(live)} parts, the kernels take {MAX_AXIS_SEGMENTS} a call")
    arr = (AxisSegment * max(len(live), 1))()
    kept = []
    for i, (t, src_start, dst_start, count) in enumerate(live):
        want = list(like.shape)
        want[axis] = t.shape[axis]
        if list(t.shape) != want or t.dtype != like.dtype or t.device != like.device:
            raise ValueError(f"{what}: part {i} has shape {tuple(t.shape)} / {t.dtype}, expected {tuple(want)} / {like.dtype} on {like.device}")
        t = t.contiguous()
        kept.append(t)
        if src_start < 0 or src_start + count > t.shape[axis] or dst_start < 0 or dst_start + count > dst_rows:
            raise ValueError(f"{what}: part {i} does not fit ({src_start}, {dst_start}, {count})")
        arr[i].src, arr[i].src_rows = t.data_ptr(), int(t.shape[axis])
        arr[i].src_start, arr[i].dst_start, arr[i].count = int(src_start), int(dst_start), int(count)
    return arr, len(live), kept


def axis_gather(dst_rows: int, axis: int, parts: Sequence, like: torch.Tensor) -> torch.Tensor:
    """A tensor like ``like`` with ``dst_rows`` rows along ``axis``: zero, then every part
    ``(tensor, src_start, dst_start, count)`` copied in (bit-exact; ``jg_halo_axis_gather``)."""
    _lib.require_gpu(like)
    axis %= like.dim()
    shape = list(like.shape)
    shape[axis] = int(dst_rows)
    out = torch.empty(shape, dtype=like.dtype, device=like.device)
    arr, n, kept = _segments(parts, axis, like, int(dst_rows), "axis_gather")
    outer, _, inner = _axis_view(out, axis)
    rc = _lib.load().jg_halo_axis_gather(_lib.ptr(out), outer, int(dst_rows), inner, arr, n, like.element_size(),
                                         _lib.stream_ptr(like.device))
    _lib.check(rc, "jg_halo_axis_gather")
    del kept
    return out


def axis_scatter_add(dst_rows: int, axis: int, parts: Sequence, like: torch.Tensor) -> torch.Tensor:
    """``zeros`` with ``dst_rows`` rows along ``axis``, then ``out[dst_start : +count] += part`` for the parts in the
    order given, every sum rounded to the dtype (``jg_halo_axis_scatter_add``)."""
    _lib.require_gpu(like)
    axis %= like.dim()
    shape = list(like.shape)
    shape[axis] = int(dst_rows)
    out = torch.empty(shape, dtype=like.dtype, device=like.device)
    arr, n, kept = _segments(parts, axis, like, int(dst_rows), "axis_scatter_add")
    outer, _, inner = _axis_view(out, axis)
    rc = _lib.load().jg_halo_axis_scatter_add(_lib.ptr(out), outer, int(dst_rows), inner, arr, n, _lib.dtype_code(like.dtype),
                                              _lib.stream_ptr(like.device))
    _lib.check(rc, "jg_halo_axis_scatter_add")
    del kept
    return out


def halo_gather_axis(x, axis, rank, group_size, kernel, stride, padding, dilation, all_to_all):
    """The need span of ``rank`` along ``axis`` from its tile and its peers' (``halo_gather``,
    _conv/halo.py:66-156). ``all_to_all(send)`` is the exchange of that axis' group
    (``exchange_along_axis``, _common/halo.py:7-63): ``send[p]`` is the contiguous part cut for
    peer ``p`` (``None`` where there is none, and for the rank itself, whose part never travels); it
    returns the parts the peers cut for this rank, by peer."""
    G, n = int(group_size), int(x.shape[axis])
    spans = [needed_input_span(r, G, n, kernel, stride, padding, dilation) for r in range(G)]
    lo, hi, need, _ = spans[rank]
    send: list = [None] * G
    for peer in range(G):
        if peer == rank:
            continue
        r0, cnt = span_overlap(spans[peer][0], spans[peer][1], rank, n, G)  # rows of mine that peer needs
        if cnt > 0:
            send[peer] = axis_gather(cnt, axis, [(x, r0 - rank * n, 0, cnt)], x)
    recv = all_to_all(send)
    parts = []
    for peer in range(G):
        r0, cnt = span_overlap(lo, hi, peer, n, G)
        if cnt <= 0:
            continue
        if peer == rank:
            parts.append((x, r0 - rank * n, r0 - lo, cnt))
        else:
            if recv[peer] is None or recv[peer].shape[axis] != cnt:
                raise ValueError(f"halo_gather_axis: expected {cnt} rows from peer {peer}")
            parts.append((recv[peer], 0, r0 - lo, cnt))
    return axis_gather(need, axis, parts, x)


def halo_scatter_add_axis(g_need, axis, rank, group_size, kernel, stride, padding, dilation, local_in_size, all_to_all):
    """The gradient of the rows ``rank`` owns from its own span's gradient and its peers'
    (``halo_scatter_add``, _conv/halo.py:159-251): the parts are added in peer order 0 .. G-1, the
    own one in its place, each sum rounded to the dtype — the bits of the reference's loop."""
    G, n = int(group_size), int(local_in_size)
    spans = [needed_input_span(r, G, n, kernel, stride, padding, dilation) for r in range(G)]
    lo, hi, need, _ = spans[rank]
    if g_need.shape[axis] != need:
        raise ValueError(f"halo_scatter_add_axis: the span has {need} rows, the gradient {g_need.shape[axis]}")
    send: list = [None] * G
    for peer in range(G):
        if peer == rank:
            continue
        r0, cnt = span_overlap(lo, hi, peer, n, G)  # rows of my span that peer owns
        if cnt > 0:
            send[peer] = axis_gather(cnt, axis, [(g_need, r0 - lo, 0, cnt)], g_need)
    recv = all_to_all(send)
    parts = []
    for peer in range(G):
        r0, cnt = span_overlap(spans[peer][0], spans[peer][1], rank, n, G)  # rows of peer's span that I own
        if cnt <= 0:
            continue
        if peer == rank:
            parts.append((g_need, r0 - lo, r0 - rank * n, cnt))
        else:
            if recv[peer] is None or recv[peer].shape[axis] != cnt:
                raise ValueError(f"halo_scatter_add_axis: expected {cnt} rows from peer {peer}")
            parts.append((recv[peer], 0, r0 - rank * n, cnt))
    return axis_scatter_add(n, axis, parts, g_need)


__all__ = [
    "HaloGeometry",
    "axis_gather",
    "axis_scatter_add",
    "halo_assemble",
    "halo_fold",
    "halo_fold_border_",
    "halo_gather_axis",
    "halo_pack",
    "halo_scatter_add_axis",
    "halo_widths",
    "neighbour_widths",
    "new_strips",
    "needed_input_span",
    "slot",
    "span_overlap",
    "spans_fit_the_strips",
    "strip_table",
]
