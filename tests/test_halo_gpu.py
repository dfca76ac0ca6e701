"""HIP halo assemble / pack / fold against the oracle: bit-exact (GPU)."""

import itertools

import pytest
import torch

from helpers import assert_bit_equal, conv_geometry, mesh_coords, neighbour, special_values_
from jigsaw_amd.halo import HaloGeometry, halo_assemble, halo_fold, halo_pack
from oracle import halo as oh

pytestmark = pytest.mark.gpu

CASES = [
    # mesh, local spatial, kernel, stride, padding, dilation
    ((2, 2), (16, 24), (3, 3), (1, 1), (1, 1), (1, 1)),
    ((3, 3), (8, 9), (3, 3), (1, 1), (1, 1), (1, 1)),
    ((3, 3), (7, 5), (5, 5), (1, 1), (2, 2), (1, 1)),
    ((2, 3), (9, 8), (3, 5), (1, 1), (1, 2), (1, 1)),
    ((3, 2), (8, 8), (3, 3), (1, 1), (2, 2), (2, 2)),
    ((2, 1), (8, 10), (3, 3), (1, 1), (1, 1), (1, 1)),
    ((1, 3), (8, 10), (3, 3), (1, 1), (1, 1), (1, 1)),
    ((3, 3), (4, 6), (3, 5), (2, 2), (1, 2), (1, 1)),  # strided: halo (lo 1, hi 0) and (lo 2, hi 1)
    ((3, 3), (2, 2), (5, 5), (1, 1), (2, 2), (1, 1)),  # halo as wide as the tile
    ((2, 2, 2), (6, 5, 8), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((3, 3, 3), (4, 5, 6), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((3, 1, 3), (4, 5, 6), (5, 3, 3), (1, 1, 1), (2, 1, 1), (1, 1, 1)),
    # rows long enough for a whole wavefront each (the W strips' elements then come through the scalar cache)
    ((1, 3), (4, 1040), (3, 3), (1, 1), (1, 1), (1, 1)),
    ((2, 2), (6, 528), (3, 3), (1, 1), (1, 1), (1, 1)),
    ((2, 3), (5, 600), (3, 5), (1, 1), (1, 2), (1, 1)),  # two columns wide: the per-column path on long rows
    # spans that drift against the tiles: the halo widths change from rank to rank
    ((2, 2), (8, 10), (3, 3), (1, 1), (0, 0), (1, 1)),  # no padding: (lo 0, hi 1) on rank 0, (lo 1, hi 0) on rank 1
    ((4, 2), (6, 8), (5, 3), (1, 1), (0, 0), (1, 1)),   # four ranks: (lo r, hi 3 - r)
    ((2, 2), (8, 8), (6, 6), (2, 2), (0, 0), (1, 1)),   # strided and drifting
    ((2, 1, 2), (4, 5, 6), (3, 3, 5), (1, 1, 1), (0, 1, 1), (1, 1, 1)),
]


def _case_id(c):
    return "mesh{}_n{}_k{}_s{}_p{}_d{}".format(*["x".join(map(str, v)) for v in c])


def gpu_strips(tiles_gpu, geoms, coord, mesh, from_padded):
    """Strips rank `coord` receives: each neighbour packs, the slot facing us is kept."""
    ns = len(mesh)
    out = {}
    for o in itertools.product((-1, 0, 1), repeat=ns):
        if not any(o):
            continue
        nb = neighbour(coord, o, mesh)
        if nb is None:
            continue
        back = tuple(-v for v in o)
        out[o] = halo_pack(tiles_gpu[nb], geoms[nb], from_padded=from_padded, present=[back])[back]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CASES, ids=_case_id)
def test_assemble_matches_oracle_bitwise(case, dtype, dev):
    mesh, n, k, s, p, d = case
    torch.manual_seed(0)
    gshape = tuple(a * b for a, b in zip(n, mesh))
    x = special_values_(torch.randn(2, 3, *gshape)).to(dtype)
    tiles = oh.split_global(x, mesh)
    want = oh.gather_mesh(tiles, mesh, k, s, p, d)
    tiles_gpu = {c: t.to(dev) for c, t in tiles.items()}
    geoms = {c: conv_geometry(n, mesh, c, k, s, p, d) for c in tiles}
    for c in mesh_coords(mesh):
        strips = gpu_strips(tiles_gpu, geoms, c, mesh, from_padded=False)
        got = halo_assemble(tiles_gpu[c], strips, geoms[c])
        assert_bit_equal(got, want[c], f"rank {c}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CASES, ids=_case_id)
def test_fold_matches_oracle_bitwise(case, dtype, dev):
    mesh, n, k, s, p, d = case
    torch.manual_seed(1)
    geoms = {c: conv_geometry(n, mesh, c, k, s, p, d) for c in mesh_coords(mesh)}
    # magnitudes spread over many binades so that the association order matters
    grads = {}
    for c, g in geoms.items():
        t = torch.randn(2, 3, *g.padded) * torch.exp2(torch.randint(-12, 12, (2, 3, *g.padded)).float())
        grads[c] = special_values_(t).to(dtype)
    want = oh.scatter_add_mesh(grads, mesh, k, s, p, d, n)
    grads_gpu = {c: t.to(dev) for c, t in grads.items()}
    for c in mesh_coords(mesh):
        strips = gpu_strips(grads_gpu, geoms, c, mesh, from_padded=True)
        got = halo_fold(grads_gpu[c], strips, geoms[c])
        assert_bit_equal(got, want[c], f"rank {c}")


def test_assemble_rejects_wrong_shapes(dev):
    g = HaloGeometry((8, 8), (1, 1), (1, 1))
    x = torch.zeros(1, 2, 8, 8, device=dev)
    with pytest.raises(ValueError):
        halo_assemble(x, {(0, 1): torch.zeros(1, 2, 8, 2, device=dev)}, g)
    with pytest.raises(ValueError):
        halo_assemble(torch.zeros(1, 2, 8, 7, device=dev), {}, g)
    with pytest.raises(RuntimeError):
        halo_assemble(torch.zeros(1, 2, 8, 8), {}, g)


def test_geometry_of_drifting_spans():
    # kernel 3, stride 2, padding 1 on 8 rows per rank: every rank's span sits the same way
    g = HaloGeometry.for_conv((8,), (3,), (2,), (1,), (1,), (1,), (2,))
    assert g.same_on_every_rank and (g.lo, g.hi) == ((1,), (0,))
    # no padding: 16 of 18 rows come out, 8 per rank; rank 0 needs a row of rank 1 and the other way round
    g0 = HaloGeometry.for_conv((9,), (3,), (1,), (0,), (1,), (0,), (2,))
    g1 = HaloGeometry.for_conv((9,), (3,), (1,), (0,), (1,), (1,), (2,))
    assert (g0.lo, g0.hi, g1.lo, g1.hi) == ((0,), (1,), (1,), (0,))
    assert g0.strip_extent((1,), "pack_fwd") == (1,) and g0.strip_extent((1,), "assemble") == (1,)
    assert g1.strip_extent((-1,), "pack_fwd") == (1,) and g1.strip_extent((-1,), "fold") == (1,)
    assert g0.theirs().lo == (1,) and g1.theirs().hi == (1,)
    # four ranks, kernel 5: (lo r, hi 3 - r); rank 1 sends 1 row down (rank 0's hi is 3 ... of which rank 1 owns 3)
    gs = [HaloGeometry.for_conv((6,), (5,), (1,), (0,), (1,), (r,), (4,)) for r in range(4)]
    assert [(g.lo[0], g.hi[0]) for g in gs] == [(0, 3), (1, 2), (2, 1), (3, 0)]
    assert gs[1].strip_extent((-1,), "pack_fwd") == (3,) and gs[1].strip_extent((1,), "pack_fwd") == (2,)
    # a span that leaves out owned rows (stride 2 without padding on 9 rows per rank) is not covered
    with pytest.raises(NotImplementedError):
        HaloGeometry.for_conv((9,), (3,), (2,), (0,), (1,), (1,), (2,))
    # nor is a halo wider than the tile
    with pytest.raises(NotImplementedError):
        HaloGeometry.for_conv((2,), (7,), (1,), (3,), (1,), (1,), (3,))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_assemble_fold_full_size_properties(dtype, dev):
    """Config-2-like tile (reduced batch): window identity and adjoint identity on device."""
    torch.manual_seed(3)
    n, mesh, c = (1024, 1024), (3, 3), (1, 1)
    geom = HaloGeometry(n, (1, 1), (1, 1))
    lead = (2, 64)
    x = torch.randn(*lead, *n, device=dev).to(dtype)
    strips = {o: torch.randn(*lead, *geom.strip_extent(o, "assemble"), device=dev).to(dtype) for o in geom.offsets()}
    aug = halo_assemble(x, strips, geom)
    assert torch.equal(aug[..., 1:-1, 1:-1], x)
    assert torch.equal(aug[..., 0:1, 1:-1], strips[(-1, 0)])
    assert torch.equal(aug[..., 1:-1, -1:], strips[(0, 1)])
    assert torch.equal(aug[..., -1:, 0:1], strips[(1, -1)])
    # a rank with no neighbours: the halo is zero and fold(assemble(x)) == x + 0
    alone = halo_assemble(x, {}, geom)
    assert alone[..., 0, :].abs().max().item() == 0 and alone[..., :, -1].abs().max().item() == 0
    back = halo_fold(alone, {}, geom)
    assert torch.equal(back, x + 0.0)
    # pack_bwd of the padded tensor returns exactly the strips that went in
    cut = halo_pack(aug, geom, from_padded=True)
    for o, t in strips.items():
        assert torch.equal(cut[o], t), o


def _slices(geom, offset, from_padded):
    """The block of the source a pack takes for neighbour ``offset``, per spatial axis."""
    out = []
    for o, n, lo, hi in zip(offset, geom.size, geom.lo, geom.hi):
        if not from_padded:  # forward: the part of my tile that lies in that neighbour's halo
            out.append(slice(0, hi) if o < 0 else slice(0, n) if o == 0 else slice(n - lo, n))
        else:                # backward: the part of my padded gradient that neighbour owns
            out.append(slice(0, lo) if o < 0 else slice(lo, lo + n) if o == 0 else slice(lo + n, lo + n + hi))
    return tuple(out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("from_padded", [False, True], ids=["own-tile", "padded"])
@pytest.mark.parametrize("size,lo,hi", [
    ((1024, 80), (1, 2), (1, 2)),      # 65536 rows of more than a cache line: the two W faces leave in one pass
    ((1024, 80), (1, 2), (0, 1)),      # faces of different thickness
    ((1024, 80), (0, 0), (1, 2)),      # one of the two faces is empty: the general kernel takes the other
    ((8, 96, 96), (1, 1, 1), (1, 1, 1)),
], ids=["w2", "w2-1", "one-face", "3d"])
def test_pack_takes_the_blocks_the_neighbours_need(size, lo, hi, from_padded, dtype, dev):
    """Every strip of ``halo_pack`` equals the slice of the source it stands for (bit for bit), whichever kernel
    cut it; the strips of one call do not overlap in memory."""
    torch.manual_seed(11)
    geom = HaloGeometry(size, lo, hi)
    lead = (64, 1) if len(size) == 2 else (9, 2)
    spatial = geom.padded if from_padded else geom.size
    src = torch.randn(*lead, *spatial, device=dev).to(dtype)
    strips = halo_pack(src, geom, from_padded=from_padded)
    spans = []
    for o, t in strips.items():
        want = src[(..., *_slices(geom, o, from_padded))]
        assert t.shape == want.shape and t.is_contiguous(), o
        assert torch.equal(t, want), o
        if t.numel():
            spans.append((t.data_ptr(), t.data_ptr() + t.numel() * t.element_size()))
    spans.sort()
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))


# need spans the strip functions do not cover: one split axis at a time through the per-peer overlap
# loop (halo.py:134-154, 217-249). (mesh, local spatial, kernel, stride, padding, dilation)
GENERAL_SPANS = [
    ((2,), (9,), (3,), (2,), (0,), (1,)),            # stride 2 without padding on an odd tile: rank 1 leaves out its last row
    ((3,), (2,), (7,), (1,), (3,), (1,)),            # kernel wider than the tile: rows from ranks two away
    ((4,), (3,), (9,), (1,), (4,), (1,)),            # four ranks, every rank reaches every other
    ((2, 2), (9, 9), (3, 3), (2, 2), (0, 0), (1, 1)),
    ((3, 2), (2, 9), (7, 3), (1, 2), (3, 0), (1, 1)),
    ((2, 3, 1), (4, 2, 5), (5, 7, 3), (1, 1, 1), (2, 3, 1), (1, 1, 1)),
    ((3, 2), (2, 6), (3, 3), (1, 1), (3, 1), (3, 1)),  # dilated: three taps with an extent of 7 over tiles of 2
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", GENERAL_SPANS, ids=lambda c: "mesh" + "x".join(map(str, c[0])) + "_n" + "x".join(map(str, c[1])) + "_k" + "x".join(map(str, c[2])))
def test_general_spans_axis_by_axis_bit_exact(case, dtype, dev):
    """Gather and scatter-add of every rank, axis by axis, against the oracle's restatement of the
    reference's loops: the gather bit for bit (copies, -0.0 kept), the scatter-add bit for bit (the
    peers' parts added in rank order, each sum rounded to the dtype)."""
    from helpers import LockstepMesh
    from jigsaw_amd.halo import halo_gather_axis, halo_scatter_add_axis, spans_fit_the_strips

    mesh, n, k, s, p, d = case
    ns = len(mesh)
    assert not spans_fit_the_strips(n, k, s, p, d, mesh)
    torch.manual_seed(7)
    lead = (2, 3)
    tiles = {c: special_values_(torch.randn(*lead, *n)).to(dtype) for c in mesh_coords(mesh)}
    want = oh.gather_mesh(tiles, mesh, k, s, p, d)
    grads = {c: (torch.randn(want[c].shape) * torch.exp2(torch.randint(-12, 12, want[c].shape).float())).to(dtype) for c in tiles}
    want_back = oh.scatter_add_mesh(grads, mesh, k, s, p, d, n)
    lock = LockstepMesh(mesh)

    def rank(c, exchange):
        cur = tiles[c].to(dev)
        for a in range(ns):
            if mesh[a] > 1:
                cur = halo_gather_axis(cur, a - ns, c[a], mesh[a], k[a], s[a], p[a], d[a],
                                       lambda send, a=a: exchange.along_axis(a, send, False))
        g = grads[c].to(dev)
        for a in reversed(range(ns)):
            if mesh[a] > 1:
                g = halo_scatter_add_axis(g, a - ns, c[a], mesh[a], k[a], s[a], p[a], d[a], n[a],
                                          lambda send, a=a: exchange.along_axis(a, send, True))
        return cur.cpu(), g.cpu()

    got = lock.run(rank)
    for c in tiles:
        assert_bit_equal(got[c][0], want[c], f"gather of rank {c}")
        assert_bit_equal(got[c][1], want_back[c], f"scatter-add of rank {c}")


def test_axis_segment_kernels_check_their_arguments(dev):
    from jigsaw_amd.halo import axis_gather, axis_scatter_add

    x = torch.arange(24, dtype=torch.float32, device=dev).reshape(2, 4, 3)
    out = axis_gather(6, 1, [(x, 1, 0, 2), (x, 0, 3, 1)], x)  # rows 1, 2 to the front, row 0 to row 3, rows 2, 4, 5 zero
    want = torch.zeros(2, 6, 3)
    want[:, 0:2] = x.cpu()[:, 1:3]
    want[:, 3] = x.cpu()[:, 0]
    assert torch.equal(out.cpu(), want)
    acc = axis_scatter_add(2, 1, [(x, 0, 0, 2), (x, 2, 0, 2), (x, 1, 1, 1)], x)
    ref = torch.zeros(2, 2, 3)
    ref += x.cpu()[:, 0:2]
    ref += x.cpu()[:, 2:4]
    ref[:, 1:2] += x.cpu()[:, 1:2]
    assert torch.equal(acc.cpu(), ref)
    with pytest.raises(ValueError):
        axis_gather(2, 1, [(x, 3, 0, 2)], x)  # reads past the source
    with pytest.raises(ValueError):
        axis_gather(2, 1, [(x[:, :, :2], 0, 0, 1)], x)  # another inner shape
    with pytest.raises(NotImplementedError):
        axis_gather(40, 1, [(x, 0, i, 1) for i in range(17)], x)
