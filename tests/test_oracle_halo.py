"""Pins the halo oracle without the reference: brute force and closed forms (CPU)."""

import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import halo as oh


def brute_span(rank, G, n, k, s, p, d):
    """Input positions touched by output block `rank`, by enumeration."""
    extent = d * (k - 1) + 1
    gout = (G * n + 2 * p - extent) // s + 1
    ol = gout // G
    touched = [o * s - p + t * d for o in range(rank * ol, (rank + 1) * ol) for t in range(k)]
    return min(touched), max(touched) + 1, ol


@pytest.mark.parametrize("G", [1, 2, 3, 4])
def test_needed_input_span_brute_force(G):
    checked = 0
    for n, k, s, p, d in itertools.product([4, 6, 8, 9], [1, 2, 3, 5], [1, 2, 3], [0, 1, 2], [1, 2]):
        extent = d * (k - 1) + 1
        if G * n + 2 * p < extent:
            continue
        gout = (G * n + 2 * p - extent) // s + 1
        if gout % G:
            with pytest.raises(NotImplementedError):
                oh.needed_input_span(0, G, n, k, s, p, d)
            continue
        for r in range(G):
            lo, hi, need, ol = oh.needed_input_span(r, G, n, k, s, p, d)
            blo, bhi, bol = brute_span(r, G, n, k, s, p, d)
            assert (lo, hi, ol) == (blo, bhi, bol)
            assert need == hi - lo
            checked += 1
    assert checked > 50


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "mesh,k,s,p,d",
    [
        ((2, 2), (3, 3), (1, 1), (1, 1), (1, 1)),
        ((2, 1), (3, 3), (1, 1), (1, 1), (1, 1)),
        ((3, 2), (5, 3), (1, 1), (2, 1), (1, 1)),
        ((2, 2), (3, 3), (1, 1), (2, 2), (2, 2)),
        ((2, 2), (3, 3), (2, 2), (1, 1), (1, 1)),
        ((4, 1), (2, 1), (1, 1), (0, 0), (1, 1)),
    ],
)
def test_gather_equals_zero_padded_window(mesh, k, s, p, d, dtype):
    """x_aug(rank) is exactly the rank's window of the zero-padded global tensor."""
    torch.manual_seed(0)
    n = (12, 12)
    x = torch.randn(2, 3, n[0] * mesh[0], n[1] * mesh[1]).to(dtype)
    try:
        spans = [[oh.needed_input_span(r, mesh[a], n[a], k[a], s[a], p[a], d[a]) for r in range(mesh[a])] for a in range(2)]
    except NotImplementedError:
        pytest.skip("not divisible")
    tiles = oh.split_global(x, mesh)
    aug = oh.gather_mesh(tiles, mesh, k, s, p, d)
    big = 64
    xp = F.pad(x, (big, big, big, big))
    for c, t in aug.items():
        win = xp
        for a in range(2):
            if mesh[a] > 1:
                lo, hi = spans[a][c[a]][0], spans[a][c[a]][1]
            else:
                lo, hi = 0, n[a]
            win = win.narrow(a - 2, big + lo, hi - lo)
        assert torch.equal(t, win), f"rank {c}"


@pytest.mark.parametrize("mesh", [(2, 2), (3, 1), (1, 2), (2, 3)])
def test_conv_on_gathered_tile_equals_global_conv(mesh):
    """F.conv2d(x_aug, pad 0 on split axes) == F.conv2d(global, pad p)[tile]."""
    torch.manual_seed(1)
    k, s, p, d = (3, 3), (1, 1), (1, 1), (1, 1)
    x = torch.randn(2, 3, 8 * mesh[0], 8 * mesh[1], dtype=torch.float64)
    w = torch.randn(4, 3, 3, 3, dtype=torch.float64)
    want = F.conv2d(x, w, padding=p)
    aug = oh.gather_mesh(oh.split_global(x, mesh), mesh, k, s, p, d)
    lp = oh.local_padding(p, mesh)
    for c, t in aug.items():
        y = F.conv2d(t, w, padding=lp)
        ref = want[:, :, c[0] * 8 : (c[0] + 1) * 8, c[1] * 8 : (c[1] + 1) * 8]
        torch.testing.assert_close(y, ref, atol=1e-12, rtol=0)


@pytest.mark.parametrize("mesh,k,s,p,d", [((2, 2), (3, 3), (1, 1), (1, 1), (1, 1)), ((3, 2), (5, 3), (1, 1), (2, 1), (1, 1)), ((2, 2), (3, 3), (2, 2), (1, 1), (1, 1))])
def test_scatter_add_is_the_adjoint_of_gather(mesh, k, s, p, d):
    """<A x, g> == <x, A^T g> over the whole mesh (fp64, exact up to rounding)."""
    torch.manual_seed(2)
    n = (6, 6)
    tiles = {c: torch.randn(1, 2, *n, dtype=torch.float64) for c in itertools.product(range(mesh[0]), range(mesh[1]))}
    aug = oh.gather_mesh(tiles, mesh, k, s, p, d)
    grads = {c: torch.randn_like(t) for c, t in aug.items()}
    folded = oh.scatter_add_mesh(grads, mesh, k, s, p, d, n)
    lhs = sum((aug[c] * grads[c]).sum() for c in tiles)
    rhs = sum((tiles[c] * folded[c]).sum() for c in tiles)
    assert abs(lhs - rhs) < 1e-9 * max(1.0, abs(lhs))


def test_scatter_add_association_on_a_corner():
    """Corner cell of an interior rank: (left-diag + top) + (left + own), W fold first."""
    mesh, k, s, p, d, n = (3, 3), (3, 3), (1, 1), (1, 1), (1, 1), (4, 4)
    vals = {}
    base = 1.0
    grads = {}
    for i, c in enumerate(itertools.product(range(3), range(3))):
        g = torch.zeros(1, 1, 6, 6, dtype=torch.float32)
        grads[c] = g
    # cell (0, 0) of rank (1, 1): own padded (1,1); left nb (1,0) padded (1,5);
    # top nb (0,1) padded (5,1); diagonal (0,0) padded (5,5)
    own, left, top, diag = 1.0, 2.0**-24, 2.0**-24, 2.0**-24
    grads[(1, 1)][0, 0, 1, 1] = own
    grads[(1, 0)][0, 0, 1, 5] = left
    grads[(0, 1)][0, 0, 5, 1] = top
    grads[(0, 0)][0, 0, 5, 5] = diag
    folded = oh.scatter_add_mesh(grads, mesh, k, s, p, d, n)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32)  # noqa: E731
    want = (f32(diag) + f32(top)) + (f32(left) + f32(own))  # = 1 + 2^-23 (tie rounds via pair sum)
    other = ((f32(own) + f32(left)) + f32(top)) + f32(diag)  # = 1.0 (each add is a tie to even)
    assert want.item() != other.item()
    assert folded[(1, 1)][0, 0, 0, 0].item() == want.item()


def test_scatter_add_clears_negative_zero():
    mesh, k, s, p, d, n = (2, 1), (3, 3), (1, 1), (1, 1), (1, 1), (4, 4)
    grads = {(0, 0): torch.full((1, 1, 6, 4), -0.0), (1, 0): torch.full((1, 1, 6, 4), -0.0)}
    folded = oh.scatter_add_mesh(grads, mesh, k, s, p, d, n)
    assert not torch.signbit(folded[(0, 0)]).any()


def test_gather_preserves_negative_zero():
    """The forward halo is a pure copy: a -0.0 in a neighbour's rows arrives as -0.0 (bit pattern kept)."""
    mesh, k, s, p, d = (2, 2), (3, 3), (1, 1), (1, 1), (1, 1)
    x = torch.full((1, 1, 8, 8), -0.0)
    tiles = oh.split_global(x, mesh)
    aug = oh.gather_mesh(tiles, mesh, k, s, p, d)
    t = aug[(0, 0)]
    assert t.shape[-2:] == (6, 6)
    bits = t.view(torch.int32)
    sign = torch.tensor(-0.0).view(torch.int32)
    assert (bits[..., 1:, 1:] == sign).all()       # own tile and the live neighbours' rows
    assert (bits[..., 0, :] == 0).all() and (bits[..., :, 0] == 0).all()  # out-of-domain border is +0.0
