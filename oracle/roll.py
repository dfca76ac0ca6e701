"""Oracle for DistributedRoll. All ranks of the ring are simulated in one
process. Test infrastructure only."""

from __future__ import annotations

import itertools

import torch


def exchange_axis(tiles, dim, window):
    """One ``exchange_halo_1d`` over a ring of ranks.

    ``tiles[r]`` is rank r's (already locally rolled) tensor; modified in place.
    Follows jigsaw/modules/roll/_distributed_roll.py:41-60: the leading
    ``window`` entries (``window > 0``) or trailing ``|window|`` entries are sent
    with ``offset = +1 / -1``; the peer rule ``send_to = rank + direction``,
    ``recv_from = rank - direction`` modulo the ring size is
    jigsaw/_core/comm.py:207-208.
    """
    if window == 0:
        return tiles
    G = len(tiles)
    sl = [slice(None)] * tiles[0].ndim
    sl[dim] = slice(0, window) if window > 0 else slice(window, None)
    sl = tuple(sl)
    direction = 1 if window > 0 else -1
    sent = [t[sl].contiguous().clone() for t in tiles]
    for r in range(G):
        tiles[r][sl] = sent[(r - direction) % G]
    return tiles


def distributed_roll_mesh(tiles, mesh_shape, shifts, dims, distributed_dims):
    """Rolled tile of every rank of a mesh.

    ``tiles`` maps mesh coordinates (one entry per distributed dim, in the order
    of ``distributed_dims``) to local tensors. Follows ``distributed_roll``,
    jigsaw/modules/roll/_distributed_roll.py:99-112: local ``torch.roll`` first,
    then one exchange per distributed dim, in order.
    """
    cur = {c: torch.roll(t, shifts=shifts, dims=dims) for c, t in tiles.items()}
    ndim = next(iter(cur.values())).ndim
    dim_to_shift = {d % ndim: s for d, s in zip(dims, shifts)}
    for k, d in enumerate(distributed_dims):
        if d % ndim not in dim_to_shift:
            raise ValueError(f"distributed dim {d} not in dims {dims}")
        others = [range(s) if i != k else [None] for i, s in enumerate(mesh_shape)]
        for idx in itertools.product(*others):
            line = [tuple(r if j is None else j for j in idx) for r in range(mesh_shape[k])]
            exchange_axis([cur[c] for c in line], d % ndim, dim_to_shift[d % ndim])
    return cur
