"""Distributed transposed convolution on the GPU against the global operator.

The reference's parity method (tests/test_conv_transpose*.py compare every rank's output
and gradients with the serial op on the gathered tensor): all ranks of a mesh run one
after the other here; strips move through tables filled from the other ranks' tensors.
Tolerances: rel-L2 <= 1e-5 in fp32, 2e-2 in bf16.
"""

import pytest
import torch
import torch.nn.functional as F

from helpers import mesh_coords, neighbour, rel_l2
from jigsaw_amd import conv as jc
from jigsaw_amd import conv_transpose as jct
from jigsaw_amd.halo import halo_pack
from oracle import conv_transpose as oct_
from oracle import halo as oh

CONVT = {1: F.conv_transpose1d, 2: F.conv_transpose2d, 3: F.conv_transpose3d}
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


class TableExchange:
    def __init__(self, fwd, bwd):
        self.fwd, self.bwd = fwd, bwd

    def forward(self, send):
        return self.fwd

    def backward(self, send):
        return self.bwd


def _recv_tables(tensors, geoms, mesh, from_padded):
    """For every rank: offset -> the strip its neighbour at that offset packs for it."""
    out = {}
    for c in tensors:
        tab = {}
        for o in geoms[c].offsets():
            nb = neighbour(c, o, mesh)
            if nb is None:
                continue
            back = tuple(-v for v in o)
            strips = halo_pack(tensors[nb], geoms[nb], from_padded=from_padded, present=[back])
            if back in strips:
                tab[o] = strips[back]
        out[c] = tab
    return out


def test_transpose_geometry_and_spans():
    g = jct.transpose_geometry((8, 8), (4, 4), (2, 2), (1, 1), (1, 1), (1, 0), (2, 2))
    assert g.size == (16, 16) and g.lo == (1, 1) and g.hi == (1, 1)
    g = jct.transpose_geometry((8, 5), (2, 3), (2, 1), (0, 1), (1, 1), (0, 0), (2, 1))
    assert g.size == (16, 5) and g.lo == (0, 0) and g.hi == (0, 0)
    # k5 s1 p1 on a split axis: 14 columns come out of 12, 7 per rank, the raw spans (10 wide) drift
    g0 = jct.transpose_geometry((6,), (5,), (1,), (1,), (1,), (0,), (2,))
    g1 = jct.transpose_geometry((6,), (5,), (1,), (1,), (1,), (1,), (2,))
    assert (g0.size, g0.lo, g0.hi) == ((7,), (1,), (2,)) and (g1.size, g1.lo, g1.hi) == ((7,), (2,), (1,))
    assert g0.strip_extent((1,), "fold") == (2,) and g1.strip_extent((-1,), "fold") == (2,)
    with pytest.raises(NotImplementedError):  # a raw span that starts behind the block its rank keeps
        jct.transpose_geometry((4,), (2,), (2,), (2,), (1,), (2,), (4,))
    for args in [(1, 3, 4, 4, 2, 1, 1), (0, 2, 5, 3, 1, 1, 2)]:
        assert jct.produced_output_span(*args) == oct_.produced_output_span(*args)
    with pytest.raises(NotImplementedError):
        jct.produced_output_span(0, 2, 4, 3, 2, 1, 1)


CASES = [
    # mesh, local input, N, Cin, Cout, kernel, stride, padding, dilation, dtype
    ((2, 2), (6, 8), 2, 3, 5, (4, 4), (2, 2), (1, 1), (1, 1), torch.float32),
    ((3, 2), (4, 6), 1, 4, 2, (3, 3), (1, 1), (1, 1), (1, 1), torch.float32),
    ((2, 2), (5, 4), 2, 2, 3, (2, 2), (2, 2), (0, 0), (1, 1), torch.float32),      # no overlap: nothing to exchange
    ((2, 1), (6, 7), 1, 3, 3, (4, 3), (2, 1), (1, 1), (1, 1), torch.float32),      # W not split: the op pads it itself
    ((2, 2), (8, 6), 1, 2, 2, (3, 5), (1, 1), (2, 2), (2, 1), torch.float32),      # dilated, 2-wide halos
    ((2, 2), (16, 32), 1, 32, 32, (3, 3), (1, 1), (1, 1), (1, 1), torch.bfloat16),  # MFMA path, fused fold
    ((2, 2), (16, 32), 1, 64, 64, (3, 3), (1, 1), (1, 1), (1, 1), torch.bfloat16),
    ((2, 2, 2), (3, 4, 4), 1, 2, 3, (4, 3, 4), (2, 1, 2), (1, 1, 1), (1, 1, 1), torch.float32),
    # raw spans that drift against the kept blocks (extent != stride + 2 * padding)
    ((2, 2), (6, 6), 2, 2, 2, (5, 3), (1, 3), (1, 0), (1, 1), torch.float32),
    ((2, 2), (5, 7), 1, 3, 2, (4, 4), (2, 2), (0, 0), (1, 1), torch.float32),      # k4 s2 p0: one column more per rank
    ((4, 1), (4, 5), 1, 2, 3, (5, 3), (1, 1), (0, 1), (1, 1), torch.float32),      # four ranks: (lo r, hi 3 - r)
    ((2, 2), (16, 32), 1, 32, 32, (3, 3), (1, 1), (0, 0), (1, 1), torch.bfloat16),  # MFMA path, drifting
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"mesh{'x'.join(map(str, c[0]))}_{c[3]}to{c[4]}_k{''.join(map(str, c[5]))}_s{''.join(map(str, c[6]))}_{str(c[9]).split('.')[-1]}")
def test_distributed_transposed_conv_matches_global(case, dev):
    mesh, n, N, cin, cout, k, s, p, d, dtype = case
    ns = len(mesh)
    torch.manual_seed(1)
    gshape = tuple(a * b for a, b in zip(n, mesh))
    X = torch.randn(N, cin, *gshape).to(dtype)
    fan = cout * int(torch.tensor(k).prod())
    W = ((torch.rand(cin, cout, *k) * 2 - 1) / fan**0.5).to(dtype)
    B = (torch.randn(cout) * 0.1).to(dtype)
    Xd, Wd, Bd = (t.double().requires_grad_() for t in (X, W, B))
    Y = CONVT[ns](Xd, Wd, Bd, stride=s, padding=p, dilation=d)
    G = torch.randn_like(Y).to(dtype)
    Y.backward(G.double())

    tiles = {c: t.to(dev) for c, t in oh.split_global(X, mesh).items()}
    gtiles = {c: t.to(dev).contiguous() for c, t in oh.split_global(G, mesh).items()}
    geoms = {c: jct.transpose_geometry(n, k, s, p, d, c, mesh) for c in tiles}
    lp = oh.local_padding(p, mesh)
    Wg, Bg = W.to(dev), B.to(dev)
    # what the ranks exchange: forward the overlap of the raw outputs, backward the edges of g
    raws = {c: jc.conv_nd_input((N, cout, *geoms[c].padded), Wg, tiles[c], stride=s, padding=lp, dilation=d) for c in tiles}
    fwd_tabs = _recv_tables(raws, geoms, mesh, from_padded=True)
    bwd_tabs = _recv_tables(gtiles, geoms, mesh, from_padded=False)

    tol = TOL[dtype]
    gw_sum = torch.zeros_like(W, dtype=torch.float64)
    gb_sum = torch.zeros_like(B, dtype=torch.float64)
    no = tuple(Y.shape[2 + a] // mesh[a] for a in range(ns))
    for c in mesh_coords(mesh):
        cfg = jct.HipConvTransposeNdConfig.for_rank(ns, Bg, TableExchange(fwd_tabs[c], bwd_tabs[c]))
        groups = tuple(jc.TileGroup(mesh[a], c[a]) for a in range(ns))
        xl = tiles[c].clone().requires_grad_()
        wl, bl = Wg.clone().requires_grad_(), Bg.clone().requires_grad_()
        y, x_aug = jct._ConvTransposeNd.apply(xl, wl, bl, s, p, d, groups, None, cfg)
        assert not x_aug.requires_grad and tuple(y.shape[2:]) == no
        so = (slice(None), slice(None)) + tuple(slice(c[a] * no[a], (c[a] + 1) * no[a]) for a in range(ns))
        si = (slice(None), slice(None)) + tuple(slice(c[a] * n[a], (c[a] + 1) * n[a]) for a in range(ns))
        assert rel_l2(y, Y.detach()[so]) < tol, f"y of rank {c}: {rel_l2(y, Y.detach()[so]):.3e}"
        y.backward(gtiles[c])
        assert rel_l2(xl.grad, Xd.grad[si]) < tol, f"dx of rank {c}: {rel_l2(xl.grad, Xd.grad[si]):.3e}"
        gw_sum += wl.grad.double().cpu()
        gb_sum += bl.grad.double().cpu()
    assert rel_l2(gw_sum, Wd.grad) < tol, f"dw: {rel_l2(gw_sum, Wd.grad):.3e}"
    assert rel_l2(gb_sum, Bd.grad) < tol, f"db: {rel_l2(gb_sum, Bd.grad):.3e}"


@pytest.mark.gpu
def test_transposed_conv_primitive_equals_torch(dev):
    torch.manual_seed(3)
    for shape, wshape, s, p, d in [((2, 3, 7, 9), (3, 4, 3, 3), (2, 1), (1, 0), (1, 2)), ((1, 2, 4, 5, 3), (2, 2, 2, 3, 1), (2, 2, 1), (0, 1, 0), (1, 1, 1))]:
        x, w, b = torch.randn(*shape), torch.randn(*wshape) * 0.3, torch.randn(wshape[1])
        want = CONVT[len(shape) - 2](x.double(), w.double(), b.double(), stride=s, padding=p, dilation=d)
        got = jct.conv_transpose_nd(x.to(dev), w.to(dev), b.to(dev), stride=s, padding=p, dilation=d)
        assert rel_l2(got, want) < 1e-5


@pytest.mark.gpu
def test_grouped_transposed_conv_primitive_equals_torch(dev):
    """``groups`` of ``F.conv_transpose2d``: the weight is (C_in, C_out / groups, *k) and the output has
    ``groups`` times its second extent in channels."""
    torch.manual_seed(4)
    for groups, cin, cout_g in [(2, 6, 3), (4, 4, 1)]:
        x, w, b = torch.randn(2, cin, 7, 9), torch.randn(cin, cout_g, 3, 4) * 0.3, torch.randn(cout_g * groups)
        want = CONVT[2](x.double(), w.double(), b.double(), stride=(2, 1), padding=(1, 0), dilation=(1, 2), groups=groups)
        got = jct.conv_transpose_nd(x.to(dev), w.to(dev), b.to(dev), stride=(2, 1), padding=(1, 0), dilation=(1, 2), groups=groups)
        assert got.shape == want.shape and rel_l2(got, want) < 1e-5
