"""Pins of the transposed-convolution oracle (CPU only): span arithmetic by brute force,
reduce / expand against the global operator and against each other (adjoint)."""

import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import conv_transpose as oct_
from oracle import halo as oh

CONVT = {1: F.conv_transpose1d, 2: F.conv_transpose2d, 3: F.conv_transpose3d}


def test_produced_output_span_brute_force():
    """Which global output columns do a rank's inputs touch? Input i and tap j write column
    i * s - p + d * j (the definition of the transposed convolution)."""
    seen = 0
    for G, n, k, s, p, d in itertools.product((1, 2, 3), (2, 5), (1, 2, 3, 4), (1, 2, 3), (0, 1, 2), (1, 2)):
        extent = d * (k - 1) + 1
        cols_all = [i * s - p + d * j for i in range(G * n) for j in range(k)]
        global_out = max(cols_all) + 1 - p  # columns 0 .. global_out - 1 survive the crop of p on either side
        if global_out <= 0:
            continue
        if global_out % G != 0:
            with pytest.raises(NotImplementedError):
                oct_.produced_output_span(0, G, n, k, s, p, d)
            continue
        for r in range(G):
            base, wloc, out_local, go = oct_.produced_output_span(r, G, n, k, s, p, d)
            cols = [i * s - p + d * j for i in range(r * n, (r + 1) * n) for j in range(k)]
            assert base == min(cols) and base + wloc == max(cols) + 1
            assert go == global_out and out_local * G == go and wloc == (n - 1) * s + extent
            seen += 1
    assert seen > 100


CASES = [
    # mesh, local input, Cin, Cout, kernel, stride, padding, dilation
    ((2, 2), (4, 5), 3, 2, (4, 4), (2, 2), (1, 1), (1, 1)),
    ((3, 1), (4, 6), 2, 3, (3, 3), (1, 1), (1, 1), (1, 1)),
    ((2, 2), (3, 3), 2, 2, (2, 2), (2, 2), (0, 0), (1, 1)),
    ((2, 3), (4, 4), 2, 2, (3, 5), (1, 1), (2, 2), (2, 1)),
    ((2, 2, 2), (3, 2, 4), 2, 3, (4, 3, 4), (2, 1, 2), (1, 1, 1), (1, 1, 1)),
    ((2, 2), (6, 6), 2, 2, (5, 3), (1, 3), (1, 0), (1, 1)),       # drifting span on H (k5 s1 p1 -> out = n + 2/G... )
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"mesh{'x'.join(map(str, c[0]))}_k{''.join(map(str, c[4]))}_s{''.join(map(str, c[5]))}_p{''.join(map(str, c[6]))}")
def test_reduce_and_expand_against_the_global_operator(case):
    mesh, n, cin, cout, k, s, p, d = case
    ns = len(mesh)
    torch.manual_seed(2)
    gshape = tuple(a * b for a, b in zip(n, mesh))
    try:
        for a in range(ns):
            oct_.produced_output_span(0, mesh[a], n[a], k[a], s[a], p[a], d[a])
    except NotImplementedError:
        pytest.skip("global output not divisible by the group size")
    X = torch.randn(2, cin, *gshape, dtype=torch.float64, requires_grad=True)
    W = torch.randn(cin, cout, *k, dtype=torch.float64, requires_grad=True)
    B = torch.randn(cout, dtype=torch.float64)
    Y = CONVT[ns](X, W, B, stride=s, padding=p, dilation=d)
    G = torch.randn_like(Y)
    Y.backward(G)
    lp = oh.local_padding(p, mesh)
    tiles = oh.split_global(X.detach(), mesh)
    raws = {c: oct_.local_forward(t, W.detach(), s, lp, d) for c, t in tiles.items()}
    ys = oct_.reduce_mesh(raws, mesh, n, k, s, p, d)
    ytiles = oh.split_global(Y.detach(), mesh)
    for c in tiles:
        assert torch.allclose(ys[c] + B.view((1, -1) + (1,) * ns), ytiles[c], rtol=1e-10, atol=1e-10), c
    # backward: expand, then the local operator's own gradients
    gtiles = oh.split_global(G, mesh)
    graws = oct_.expand_mesh(gtiles, mesh, n, k, s, p, d)
    xg = oh.split_global(X.grad, mesh)
    gw = torch.zeros_like(W)
    for c in tiles:
        assert graws[c].shape == raws[c].shape
        xl = tiles[c].clone().requires_grad_()
        wl = W.detach().clone().requires_grad_()
        oct_.local_forward(xl, wl, s, lp, d).backward(graws[c])
        assert torch.allclose(xl.grad, xg[c], rtol=1e-10, atol=1e-10), c
        gw += wl.grad
    assert torch.allclose(gw, W.grad, rtol=1e-9, atol=1e-9)
    # adjoint identity <reduce(a), b> == <a, expand(b)>
    a = {c: torch.randn_like(t) for c, t in raws.items()}
    b = {c: torch.randn_like(t) for c, t in ys.items()}
    ra = oct_.reduce_mesh(a, mesh, n, k, s, p, d)
    eb = oct_.expand_mesh(b, mesh, n, k, s, p, d)
    lhs = sum((ra[c] * b[c]).sum() for c in a)
    rhs = sum((a[c] * eb[c]).sum() for c in a)
    assert torch.allclose(lhs, rhs, rtol=1e-10)
