"""Shared helpers of the parity tests (seeded meshes of tiles, bit comparisons)."""

from __future__ import annotations

import itertools

import torch

from jigsaw_amd.halo import HaloGeometry


def bits(t: torch.Tensor) -> torch.Tensor:
    """Reinterpret a float tensor as integers so that equality is bit equality."""
    t = t.detach().contiguous().cpu()
    return t.view({2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def assert_bit_equal(got: torch.Tensor, want: torch.Tensor, what: str = "") -> None:
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert got.dtype == want.dtype, f"{what}: dtype {got.dtype} != {want.dtype}"
    g, w = bits(got), bits(want)
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} elements differ bitwise; first at {bad[0].tolist()}")


def rel_l2(got: torch.Tensor, want: torch.Tensor) -> float:
    g = got.detach().double().cpu()
    w = want.detach().double().cpu()
    den = w.norm().item()
    return (g - w).norm().item() / (den if den > 0 else 1.0)


def mesh_coords(mesh_shape):
    return list(itertools.product(*[range(s) for s in mesh_shape]))


def neighbour(coord, offset, mesh_shape):
    """Mesh coordinate of the neighbour at ``offset`` or None outside the mesh.

    Axes with a group of one have no neighbours (offset must be 0 there).
    """
    out = []
    for c, o, s in zip(coord, offset, mesh_shape):
        if s <= 1 and o != 0:
            return None
        v = c + o
        if v < 0 or v >= s:
            return None
        out.append(v)
    return tuple(out)


def conv_geometry(local_spatial, mesh_shape, coord, kernel, stride, padding, dilation) -> HaloGeometry:
    return HaloGeometry.for_conv(local_spatial, kernel, stride, padding, dilation, coord, mesh_shape)


def special_values_(t: torch.Tensor) -> torch.Tensor:
    """Sprinkle -0.0, +0.0 and a denormal into a tensor (bit-exactness probes)."""
    flat = t.view(-1)
    n = flat.numel()
    if n >= 16:
        flat[::7] = -0.0
        flat[3::11] = 0.0
        flat[5::13] = 1e-39 if t.dtype == torch.float32 else 1e-39
    return t


def kaiming_uniform_bound(c_in, kernel, a=5 ** 0.5):
    """Half-width of the uniform weight distribution jigsaw's layers initialise with.

    Follows jigsaw/init.py:115-158 as called from convolution/_conv/base.py:236-238 (a = sqrt(5)):
    gain = sqrt(2 / (1 + a^2)), bound = sqrt(3) * gain / sqrt(fan_in), fan_in = c_in * prod(kernel).
    """
    fan_in = c_in
    for k in kernel:
        fan_in *= k
    gain = (2.0 / (1.0 + a * a)) ** 0.5
    return (3.0 ** 0.5) * gain / fan_in ** 0.5


class LockstepMesh:
    """Every rank of a spatial mesh in this process, one thread each, for the exchanges that need all ranks
    at once (``HaloExchange.along_axis``: every rank cuts parts for its peers, then every rank picks up
    what was cut for it). ``run(fn)`` calls ``fn(coord, exchange)`` per rank and returns ``{coord: result}``;
    an exception in one rank releases the others and is raised again. All ranks launch on the default
    stream, so a part is read behind the kernel that cut it."""

    def __init__(self, mesh_shape):
        import threading

        self.mesh = tuple(mesh_shape)
        self.coords = list(mesh_coords(self.mesh))
        self._barrier = threading.Barrier(len(self.coords))
        self._box: dict = {}
        self.calls: list = []  # (coord, axis, backward, rows sent per peer) in call order per rank

    def exchange_for(self, coord):
        mesh = self

        class _Rank:
            def forward(self, send):
                raise AssertionError("the strip exchange is not what general spans use")

            backward = forward

            def along_axis(self, axis, send, backward):
                if len(send) != mesh.mesh[axis] or send[coord[axis]] is not None:
                    raise AssertionError("one part per peer of the axis, none for the rank itself")
                mesh.calls.append((coord, axis, backward, [None if t is None else int(t.shape[axis - len(mesh.mesh)]) for t in send]))
                mesh._box[(coord, axis, backward)] = send
                mesh._barrier.wait(timeout=60)
                recv = []
                for p in range(mesh.mesh[axis]):
                    peer = tuple(p if a == axis else v for a, v in enumerate(coord))
                    recv.append(None if peer == coord else mesh._box[(peer, axis, backward)][coord[axis]])
                mesh._barrier.wait(timeout=60)
                return recv

        return _Rank()

    def run(self, fn):
        import threading

        results, errors = {}, []

        def body(c):
            try:
                results[c] = fn(c, self.exchange_for(c))
            except BaseException as exc:  # noqa: BLE001
                errors.append(exc)
                self._barrier.abort()

        threads = [threading.Thread(target=body, args=(c,)) for c in self.coords]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        self._barrier.reset()
        if errors:
            first = [e for e in errors if not isinstance(e, threading.BrokenBarrierError)]
            raise (first or errors)[0]
        return results
