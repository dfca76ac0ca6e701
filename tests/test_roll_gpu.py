"""HIP roll and slab pack / unpack against torch.roll and the oracle: exact (GPU)."""

import pytest
import torch

from helpers import assert_bit_equal, mesh_coords
from jigsaw_amd import roll as jr
from oracle import roll as orl

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "shape,shifts,dims",
    [
        ((2, 16, 16, 8), (4, 4), (1, 2)),
        ((2, 16, 16, 8), (-4, -3), (1, 2)),
        ((3, 7, 5), (2,), (2,)),
        ((3, 7, 5), (1, -2, 3), (0, 1, 2)),
        ((4, 6, 10, 3), (13, -25), (1, 2)),
        ((1, 256, 256, 128), (-4, -4), (1, 2)),
        ((5,), (2,), (0,)),
        ((2, 3, 4, 5, 6, 7), (1, 2), (1, 4)),
    ],
)
def test_roll_equals_torch_roll(shape, shifts, dims, dtype, dev):
    torch.manual_seed(0)
    x = torch.randn(*shape).to(dtype)
    want = torch.roll(x, shifts, dims)
    got = jr.roll(x.to(dev), shifts, dims)
    assert_bit_equal(got, want)


@pytest.mark.parametrize("window", [4, -4, 1, -3])
@pytest.mark.parametrize("dim", [1, 2, -1])
def test_slab_pack_unpack(window, dim, dev):
    torch.manual_seed(1)
    x = torch.randn(2, 12, 10, 8).bfloat16()
    sl = [slice(None)] * 4
    sl[dim] = slice(0, window) if window > 0 else slice(window, None)
    want = x[tuple(sl)].contiguous()
    xg = x.to(dev)
    got = jr.slab_pack(xg, dim, window)
    assert_bit_equal(got, want)
    repl = torch.randn_like(want)
    x2 = x.clone()
    x2[tuple(sl)] = repl
    jr.slab_unpack_(xg, repl.to(dev), dim, window)
    assert_bit_equal(xg, x2)


class RingComm:
    """Stand-in for RollConfig.comm_halo_1d_fn on one GPU: the slab every rank would
    send is precomputed by the oracle side of the test and handed over on request."""

    def __init__(self):
        self.sent = []
        self.answers = []

    def __call__(self, data, buffer, direction, *, group, async_op):
        self.sent.append((data.clone(), direction, group))
        buffer.copy_(self.answers.pop(0))
        return buffer, None


@pytest.mark.parametrize("shift", [4, -4, -1])
@pytest.mark.parametrize("mesh", [(2, 2), (3, 2), (1, 2)])
def test_distributed_roll_matches_oracle_and_global_roll(mesh, shift, dev):
    torch.manual_seed(2)
    n = (8, 8)
    b, c = 2, 16
    glob = torch.randn(b, n[0] * mesh[0], n[1] * mesh[1], c).bfloat16()
    tiles = {
        co: glob[:, co[0] * n[0] : (co[0] + 1) * n[0], co[1] * n[1] : (co[1] + 1) * n[1]].contiguous()
        for co in mesh_coords(mesh)
    }
    shifts, dims = (shift, shift), (1, 2)
    want = orl.distributed_roll_mesh({k: v.clone() for k, v in tiles.items()}, mesh, shifts, dims, [1, 2])
    # the oracle's result is the tile of the globally rolled tensor
    groll = torch.roll(glob, shifts, dims)
    for co, t in want.items():
        assert torch.equal(t, groll[:, co[0] * n[0] : (co[0] + 1) * n[0], co[1] * n[1] : (co[1] + 1) * n[1]])

    # GPU, rank by rank. Slabs received: axis H first (from the H-neighbour's locally
    # rolled tile), then axis W (from the W-neighbour's tile after *its* H exchange).
    direction = 1 if shift > 0 else -1
    sl_h = slice(0, shift) if shift > 0 else slice(shift, None)
    after_local = {co: torch.roll(t, shifts, dims) for co, t in tiles.items()}
    after_h = orl.distributed_roll_mesh({k: v.clone() for k, v in tiles.items()}, mesh, shifts, dims, [1])
    for co in mesh_coords(mesh):
        comm = RingComm()
        src_h = ((co[0] - direction) % mesh[0], co[1])
        src_w = (co[0], (co[1] - direction) % mesh[1])
        comm.answers.append(after_local[src_h][:, sl_h].contiguous().to(dev))
        comm.answers.append(after_h[src_w][:, :, sl_h].contiguous().to(dev))
        got = jr.distributed_roll(tiles[co].to(dev), shifts, dims, [1, 2], ["gh", "gw"], comm)
        assert_bit_equal(got, want[co], f"rank {co}")
        assert [s[1] for s in comm.sent] == [direction, direction]
        assert [s[2] for s in comm.sent] == ["gh", "gw"]
        assert_bit_equal(comm.sent[0][0], after_local[co][:, sl_h].contiguous())


def test_roll_errors(dev):
    x = torch.zeros(2, 4, 4, 3, device=dev)
    with pytest.raises(ValueError):
        jr.distributed_roll(x, (1,), (1,), [2], [None], lambda *a, **k: None)
    with pytest.raises(ValueError):
        jr.slab_pack(x, 1, 5)


def test_roll_autograd_is_inverse_roll(dev):
    x = torch.randn(1, 8, 8, 4, device=dev, requires_grad=True)
    y = jr._Roll.apply(x, (2, -3), (1, 2), (), (), None)
    g = torch.randn_like(y)
    y.backward(g)
    assert torch.equal(x.grad, torch.roll(g, (-2, 3), (1, 2)))


class ScriptedComm:
    """Answers every exchange with a tensor made from the call number, and records what was sent."""

    def __init__(self, seed):
        self.gen = torch.Generator().manual_seed(seed)
        self.sent = []

    def __call__(self, data, buffer, direction, *, group, async_op):
        assert buffer.shape == data.shape and float(buffer.abs().sum()) == 0.0  # the receive buffer arrives cleared
        self.sent.append((data.clone(), direction, group))
        buffer.copy_(torch.randn(buffer.shape, generator=self.gen).to(buffer.dtype))
        return buffer, None


@pytest.mark.parametrize("shape,dtype,shifts,dims,dist", [
    ((2, 8, 8, 16), torch.bfloat16, (4, 4), (1, 2), [1, 2]),     # one pass per exchange
    ((2, 8, 8, 16), torch.bfloat16, (-3, 2), (1, 2), [2, 1]),    # the W exchange first, different windows
    ((1, 16, 8, 4), torch.float32, (5, -1), (1, 2), [1, 2]),     # 4-byte elements, 16-byte rows
    ((1, 8, 8, 8), torch.bfloat16, (2, 0), (1, 2), [1, 2]),      # a zero shift drops its exchange
    ((3, 8, 12, 8), torch.bfloat16, (-8, 3), (1, 2), [1]),       # one distributed axis, a slab as long as the axis
    ((2, 8, 8, 4), torch.bfloat16, (1, 1), (1, 2), [1, 2]),      # 8-byte rows: the step-by-step route
    ((4, 6, 16), torch.float32, (2, 4), (0, 1), [0, 1]),         # rolled leading axis, 3-D tensor
])
def test_distributed_roll_one_pass_equals_step_by_step(shape, dtype, shifts, dims, dist, dev):
    """distributed_roll (which runs one launch per exchange where the layout allows) against the
    reference's sequence written out with the separate kernels: roll, then per distributed axis
    cut, exchange, write back (_distributed_roll.py:44-59, 99-113). Same result bits, same slabs
    sent in the same order with the same directions."""
    torch.manual_seed(9)
    x = torch.randn(*shape).to(dtype).to(dev)
    groups = [f"g{d}" for d in dist]
    a = ScriptedComm(4)
    got = jr.distributed_roll(x.clone(), shifts, dims, list(dist), groups, a)
    b = ScriptedComm(4)
    want = jr.roll(x.clone(), shifts, dims)
    shift_of = {d % x.dim(): s for d, s in zip(dims, shifts)}
    for d, g in zip(dist, groups):
        want = jr.exchange_halo_1d(want, dim=d, window_size=shift_of[d % x.dim()], group=g, comm_halo_1d_fn=b)
    torch.cuda.synchronize()
    assert_bit_equal(got, want)
    assert len(a.sent) == len(b.sent)
    for (sa, da, ga), (sb, db, gb) in zip(a.sent, b.sent):
        assert da == db and ga == gb
        assert_bit_equal(sa, sb)
