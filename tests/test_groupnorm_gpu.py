"""Spatially sharded GroupNorm: HIP kernels (through the C ABI) against the oracle.

The shards of a spatial split run one after the other in this process; the all-reduces
of a shard see the other shards' contributions through a stand-in group that holds them
(computed in fp64 from the same inputs), in the order the operator asks for them:
(count, sum), centred squares, and in the backward the two per-group sums.
Tolerances: rel-L2 <= 1e-5 in fp32, 2e-2 in bf16.
"""

import pytest
import torch

from helpers import rel_l2
from jigsaw_amd import groupnorm as jgn
from oracle import groupnorm as ogn

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 4e-3}


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


class Others:
    """Stand-in process group: adds what the other ranks would contribute to each sum."""

    def __init__(self, contributions):
        self.contributions, self.calls = list(contributions), 0

    def size(self):
        return 2

    def all_reduce(self, t, op):
        assert op == "sum"
        t += self.contributions[self.calls].to(device=t.device, dtype=t.dtype)
        self.calls += 1


CASES = [
    # global shape, groups, dtype, weight, bias, shards along the first spatial axis
    ((2, 8, 6, 10), 4, torch.float32, True, True, 2),
    ((1, 6, 6, 7, 3), 3, torch.float32, True, False, 3),       # odd extents: element-wise path
    ((2, 64, 64, 64), 8, torch.bfloat16, True, True, 2),
    ((1, 4, 256, 300), 2, torch.float32, True, True, 2),       # long spans: several chunks per group and row
    ((3, 16, 8, 8), 16, torch.float32, False, False, 2),       # one channel per group, no affine
    ((2, 32, 32, 48), 4, torch.bfloat16, False, True, 4),
    ((2, 12, 10, 16), 3, torch.float16, True, True, 2),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{'x'.join(map(str, c[0]))}_g{c[1]}_{str(c[2]).split('.')[-1]}_p{c[5]}")
def test_sharded_groupnorm_matches_oracle(case, dev):
    shape, G, dtype, has_w, has_b, P = case
    torch.manual_seed(5)
    X = (torch.randn(*shape) * 1.5 + 0.3).to(dtype)
    W = (1 + 0.2 * torch.randn(shape[1])).to(dtype) if has_w else None
    B = (0.2 * torch.randn(shape[1])).to(dtype) if has_b else None
    GR = torch.randn(*shape).to(dtype)
    eps = 1e-5
    xs, gs = list(X.chunk(P, dim=2)), list(GR.chunk(P, dim=2))
    xd, gd = [t.double() for t in xs], [t.double() for t in gs]
    wd, bd = (None if W is None else W.double()), (None if B is None else B.double())
    outs, rstd, n = ogn.forward(xd, G, wd, bd, eps)
    back = ogn.backward(gd, [o[1] for o in outs], rstd, n, G, wd)

    # what every shard contributes to the three sums (fp64)
    N = shape[0]
    seg = [t.reshape(N, G, -1) for t in xd]
    mean = (sum(t.sum(-1) for t in seg) / n.squeeze(-1)).unsqueeze(-1)
    c1 = [torch.stack([torch.full((N, G), float(t.shape[-1]), dtype=torch.float64), t.sum(-1)], -1) for t in seg]
    c2 = [((t - mean) ** 2).sum(-1) for t in seg]
    gg = [(g if wd is None else g * wd.reshape((1, -1) + (1,) * (g.dim() - 2))).reshape(N, G, -1) for g in gd]
    xn = [o[1].reshape(N, G, -1) for o in outs]
    c3 = [torch.stack([a.sum(-1), (a * b).sum(-1)], -1) for a, b in zip(gg, xn)]

    tol = TOL[dtype]
    for i in range(P):
        others = Others([sum(c[j] for j in range(P) if j != i) for c in (c1, c2, c3)])
        x = xs[i].to(dev).requires_grad_()
        w = None if W is None else W.to(dev).requires_grad_()
        b = None if B is None else B.to(dev).requires_grad_()
        y, x_norm, rstd_g, n_g = jgn._GroupNorm.apply(x, G, w, b, (others,), eps)
        assert y.dtype == dtype and not x_norm.requires_grad
        assert rel_l2(y, outs[i][0]) < tol and rel_l2(x_norm, outs[i][1]) < tol
        assert rel_l2(rstd_g, rstd) < tol and torch.equal(n_g.double().cpu(), n)
        y.backward(gs[i].to(dev))
        assert others.calls == 3
        gx, gw, gb = back[i]
        assert rel_l2(x.grad, gx) < tol
        if has_w:
            assert rel_l2(w.grad, gw) < tol
        if has_b:
            assert rel_l2(b.grad, gb) < tol


def test_unsharded_groupnorm_equals_torch(dev):
    """No spatial groups: the operator is F.group_norm, forward and backward; under bf16
    autocast it computes in fp32 (promote_to_fp32_under_autocast)."""
    torch.manual_seed(6)
    x = torch.randn(2, 12, 9, 11)
    w, b = 1 + 0.1 * torch.randn(12), 0.1 * torch.randn(12)
    g = torch.randn_like(x)
    xd, wd, bd = (t.double().requires_grad_() for t in (x, w, b))
    want = torch.nn.functional.group_norm(xd, 3, wd, bd, 1e-5)
    want.backward(g.double())
    xg, wg, bg = (t.to(dev).requires_grad_() for t in (x, w, b))
    y = jgn.group_norm(xg, 3, wg, bg, (), 1e-5)
    y.backward(g.to(dev))
    assert rel_l2(y, want) < 1e-5 and rel_l2(xg.grad, xd.grad) < 1e-5
    assert rel_l2(wg.grad, wd.grad) < 1e-5 and rel_l2(bg.grad, bd.grad) < 1e-5
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y16 = jgn.group_norm(xg.detach().bfloat16(), 3, wg.detach(), bg.detach(), (), 1e-5)
    assert y16.dtype == torch.float32
    want16 = torch.nn.functional.group_norm(x.bfloat16().double(), 3, w.double(), b.double(), 1e-5)
    assert rel_l2(y16, want16) < 1e-5


def test_groupnorm_argument_errors(dev):
    x = torch.zeros(1, 6, 4, 4, device=dev)
    with pytest.raises(ValueError):
        jgn.group_norm(x, 4)
