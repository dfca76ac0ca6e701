"""Pins the attention, LayerNorm, conv and roll oracles against textbook forms (CPU)."""

import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oa
from oracle import conv as oc
from oracle import layernorm as ol
from oracle import roll as orl


def _chunks(P=4, b=2, h=3, n=16, d=8, dtype=torch.float64, seed=0):
    torch.manual_seed(seed)
    q = torch.randn(b, h, n, d, dtype=dtype) / d**0.5
    ks = [torch.randn(b, h, n, d, dtype=dtype) for _ in range(P)]
    vs = [torch.randn(b, h, n, d, dtype=dtype) for _ in range(P)]
    return q, ks, vs


@pytest.mark.parametrize("rank", [0, 1, 3])
def test_ring_forward_equals_full_softmax_attention(rank):
    q, ks, vs = _chunks()
    scale = 8**-0.5
    out, lse = oa.ring_forward(q, ks, vs, scale, rank=rank)
    K, V = torch.cat(ks, 2), torch.cat(vs, 2)
    s = (q @ K.mT) * scale
    want = torch.softmax(s, -1) @ V
    torch.testing.assert_close(out, want, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(lse, torch.logsumexp(s, -1), atol=1e-12, rtol=1e-10)
    # torch's own SDPA as an independent routine
    torch.testing.assert_close(out, F.scaled_dot_product_attention(q, K, V, scale=scale), atol=1e-10, rtol=1e-8)


def test_ring_backward_equals_autograd_of_full_attention():
    q, ks, vs = _chunks(seed=1)
    scale = 8**-0.5
    K = torch.cat(ks, 2).requires_grad_()
    V = torch.cat(vs, 2).requires_grad_()
    qr = q.clone().requires_grad_()
    out = torch.softmax((qr @ K.mT) * scale, -1) @ V
    dout = torch.randn_like(out)
    out.backward(dout)
    o, lse = oa.ring_forward(q, ks, vs, scale)
    dq, dks, dvs = oa.ring_backward(dout, q, o, lse, ks, vs, scale)
    torch.testing.assert_close(dq, qr.grad, atol=1e-11, rtol=1e-9)
    torch.testing.assert_close(torch.cat(dks, 2), K.grad, atol=1e-11, rtol=1e-9)
    torch.testing.assert_close(torch.cat(dvs, 2), V.grad, atol=1e-11, rtol=1e-9)


@pytest.mark.parametrize("scope", ["global", "local"])
def test_ring_all_ranks_equals_autograd_of_full_attention(scope):
    """All P ranks of the ring with the owners' dK/dV sums == autograd through full
    softmax attention of the concatenated queries over the concatenated K/V."""
    torch.manual_seed(11)
    P, b, h, n, d = 3, 2, 2, 8, 4
    scale = d**-0.5
    qs = [torch.randn(b, h, n, d, dtype=torch.float64) for _ in range(P)]
    ks = [torch.randn(b, h, n, d, dtype=torch.float64) for _ in range(P)]
    vs = [torch.randn(b, h, n, d, dtype=torch.float64) for _ in range(P)]
    douts = [torch.randn(b, h, n, d, dtype=torch.float64) for _ in range(P)]
    Q, K, V = (torch.cat(t, 2).requires_grad_() for t in (qs, ks, vs))
    full = torch.softmax((Q @ K.mT) * scale, -1) @ V
    full.backward(torch.cat(douts, 2))
    outs, lses, dqs, dks, dvs = oa.ring_all_ranks(qs, ks, vs, douts, scale, save_scope=scope)
    torch.testing.assert_close(torch.cat(outs, 2), full.detach(), atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(torch.cat(lses, 2), torch.logsumexp((Q @ K.mT).detach() * scale, -1), atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(torch.cat(dqs, 2), Q.grad, atol=1e-11, rtol=1e-9)
    torch.testing.assert_close(torch.cat(dks, 2), K.grad, atol=1e-11, rtol=1e-9)
    torch.testing.assert_close(torch.cat(dvs, 2), V.grad, atol=1e-11, rtol=1e-9)


@pytest.mark.parametrize("form", ["eager", "fused"])
def test_merge_special_cases(form):
    torch.manual_seed(2)
    o2 = torch.randn(1, 2, 4, 8)
    l2 = torch.randn(1, 2, 4)
    # seed state: l1 = -inf, o1 = 0  ->  (o2, l2)
    o1, l1 = torch.zeros_like(o2), torch.full_like(l2, float("-inf"))
    o, l = oa.merge_(o1, l1, o2, l2, form=form)
    assert torch.equal(o, o2) and torch.equal(l, l2)
    # equal weights -> mean, lse + log 2
    a, b = torch.randn_like(o2), torch.randn_like(o2)
    o, l = oa.merge_(a.clone(), l2.clone(), b, l2.clone(), form=form)
    torch.testing.assert_close(o, (a + b) / 2, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(l, l2 + torch.log(torch.tensor(2.0)), atol=1e-6, rtol=1e-6)
    # both forms agree
    la, lb = torch.randn_like(l2), torch.randn_like(l2)
    oe, le = oa.merge_(a.clone(), la, b, lb, form="eager")
    of, lf = oa.merge_(a.clone(), la, b, lb, form="fused")
    torch.testing.assert_close(oe, of, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(le, lf, atol=1e-6, rtol=1e-6)


def test_merge_is_order_independent_and_bshd_matches_bhsd():
    q, ks, vs = _chunks(P=3, seed=3)
    scale = 8**-0.5
    outs = []
    for perm in itertools.permutations(range(3)):
        o, l = oa.ring_forward(q, [ks[i] for i in perm], [vs[i] for i in perm], scale)
        outs.append((o, l))
    for o, l in outs[1:]:
        torch.testing.assert_close(o, outs[0][0], atol=1e-12, rtol=1e-10)
        torch.testing.assert_close(l, outs[0][1], atol=1e-12, rtol=1e-10)
    a, b = torch.randn(2, 3, 5, 4), torch.randn(2, 3, 5, 4)
    la, lb = torch.randn(2, 3, 5), torch.randn(2, 3, 5)
    o1, l1 = oa.merge_(a.clone(), la, b, lb, layout="bhsd")
    o2, l2 = oa.merge_(a.transpose(1, 2).contiguous(), la, b.transpose(1, 2).contiguous(), lb, layout="bshd")
    assert torch.equal(o1, o2.transpose(1, 2)) and torch.equal(l1, l2)


@pytest.mark.parametrize("G", [1, 2, 4])
def test_layernorm_oracle_equals_full_layer_norm(G):
    torch.manual_seed(4)
    C, eps = 32, 1e-5
    x = torch.randn(3, 7, C, dtype=torch.float64, requires_grad=True)
    w = (1 + 0.2 * torch.randn(C, dtype=torch.float64)).requires_grad_()
    b = (0.2 * torch.randn(C, dtype=torch.float64)).requires_grad_()
    want = F.layer_norm(x, (C,), w, b, eps)
    g = torch.randn_like(want)
    want.backward(g)
    xs, ws, bs, gs = (list(t.detach().chunk(G, -1)) for t in (x, w, b, g))
    ys, xns, std = ol.forward(xs, ws, bs, eps)
    torch.testing.assert_close(torch.cat(ys, -1), want.detach(), atol=1e-12, rtol=1e-10)
    gxs, gws, gbs = ol.backward(gs, xns, ws, std)
    torch.testing.assert_close(torch.cat(gxs, -1), x.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(torch.cat(gws, -1), w.grad, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(torch.cat(gbs, -1), b.grad, atol=1e-12, rtol=1e-10)
    # law of total variance: combined variance is the variance of the full row
    m, v = zip(*[ol.partial_stats(t) for t in xs])
    mean = torch.stack(m).mean(0)
    var = torch.stack([vi + (mi - mean) ** 2 for vi, mi in zip(v, m)]).mean(0)
    torch.testing.assert_close(var, x.detach().var(-1, keepdim=True, unbiased=False), atol=1e-12, rtol=1e-10)


def test_conv_oracle_against_brute_force_and_autograd():
    torch.manual_seed(5)
    x = torch.randn(2, 3, 6, 7, dtype=torch.float64)
    w = torch.randn(4, 3, 3, 2, dtype=torch.float64)
    b = torch.randn(4, dtype=torch.float64)
    for stride, pad, dil in [((1, 1), (0, 0), (1, 1)), ((2, 1), (1, 0), (1, 2)), ((1, 1), (1, 1), (1, 1))]:
        y = oc.forward(x, w, b, stride, pad, dil)
        torch.testing.assert_close(y, oc.brute_forward(x, w, b, stride, pad, dil), atol=1e-12, rtol=1e-10)
        xr, wr, br = x.clone().requires_grad_(), w.clone().requires_grad_(), b.clone().requires_grad_()
        yr = F.conv2d(xr, wr, br, stride, pad, dil)
        g = torch.randn_like(yr)
        yr.backward(g)
        torch.testing.assert_close(oc.dgrad(x.shape, w, g, stride, pad, dil), xr.grad, atol=1e-12, rtol=1e-10)
        torch.testing.assert_close(oc.wgrad(x, w.shape, g, stride, pad, dil), wr.grad, atol=1e-12, rtol=1e-10)
        torch.testing.assert_close(oc.grad_bias(g, 2), br.grad, atol=1e-12, rtol=1e-10)


def test_conv3d_oracle_against_autograd():
    torch.manual_seed(6)
    x = torch.randn(1, 2, 5, 6, 7, dtype=torch.float64, requires_grad=True)
    w = torch.randn(3, 2, 3, 3, 3, dtype=torch.float64, requires_grad=True)
    y = F.conv3d(x, w)
    g = torch.randn_like(y)
    y.backward(g)
    torch.testing.assert_close(oc.forward(x.detach(), w.detach(), None, (1, 1, 1), (0, 0, 0), (1, 1, 1)), y.detach())
    torch.testing.assert_close(oc.dgrad(x.shape, w.detach(), g, (1, 1, 1), (0, 0, 0), (1, 1, 1)), x.grad)
    torch.testing.assert_close(oc.wgrad(x.detach(), w.shape, g, (1, 1, 1), (0, 0, 0), (1, 1, 1)), w.grad)


@pytest.mark.parametrize("mesh,shift", [((2, 2), 3), ((3, 2), -2), ((1, 4), 1)])
def test_roll_oracle_equals_global_roll(mesh, shift):
    torch.manual_seed(7)
    n = (6, 5)
    glob = torch.randn(2, n[0] * mesh[0], n[1] * mesh[1], 3)
    tiles = {
        (i, j): glob[:, i * n[0] : (i + 1) * n[0], j * n[1] : (j + 1) * n[1]].clone()
        for i in range(mesh[0])
        for j in range(mesh[1])
    }
    got = orl.distributed_roll_mesh(tiles, mesh, (shift, shift), (1, 2), [1, 2])
    want = torch.roll(glob, (shift, shift), (1, 2))
    for (i, j), t in got.items():
        assert torch.equal(t, want[:, i * n[0] : (i + 1) * n[0], j * n[1] : (j + 1) * n[1]])


def test_window_attention_oracle_equals_sdpa():
    torch.manual_seed(8)
    q, k, v = (torch.randn(2, 5, 4, 16, 8, dtype=torch.float64) for _ in range(3))
    bias = torch.randn(5, 4, 16, 16, dtype=torch.float64)
    bias[0, :, :, 3] = float("-inf")
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=bias)
    torch.testing.assert_close(oa.window_attention(q, k, v, bias), want, atol=1e-12, rtol=1e-10)


def test_kaiming_bound_closed_form():
    """With a = sqrt(5) the bound collapses to 1/sqrt(fan_in); torch's own initialiser stays inside it."""
    from helpers import kaiming_uniform_bound

    assert abs(kaiming_uniform_bound(64, (3, 3)) - 1.0 / 24.0) < 1e-12
    assert abs(kaiming_uniform_bound(32, (3, 3, 3)) - 864 ** -0.5) < 1e-12
    torch.manual_seed(0)
    w = torch.empty(64, 64, 3, 3)
    torch.nn.init.kaiming_uniform_(w, a=5 ** 0.5)
    bound = kaiming_uniform_bound(64, (3, 3))
    assert w.abs().max() <= bound and w.abs().max() > 0.99 * bound


def test_groupnorm_oracle_equals_torch_on_the_undivided_tensor():
    """The sharded restatement (sums over the shards in place of the all-reduces) against
    F.group_norm and autograd on the gathered tensor; weight / bias gradients of the
    shards add up to the global ones."""
    from oracle import groupnorm as ogn

    torch.manual_seed(12)
    for shape, G, P, dim in [((2, 8, 6, 10), 4, 2, 2), ((1, 6, 4, 9, 5), 3, 3, 3), ((3, 4, 8), 1, 4, 2)]:
        X = (torch.randn(*shape, dtype=torch.float64) * 2 + 0.5).requires_grad_()
        W = (1 + 0.3 * torch.randn(shape[1], dtype=torch.float64)).requires_grad_()
        B = (0.3 * torch.randn(shape[1], dtype=torch.float64)).requires_grad_()
        GR = torch.randn(*shape, dtype=torch.float64)
        Y = torch.nn.functional.group_norm(X, G, W, B, 1e-5)
        Y.backward(GR)
        xs, gs = list(X.detach().chunk(P, dim=dim)), list(GR.chunk(P, dim=dim))
        outs, rstd, n = ogn.forward(xs, G, W.detach(), B.detach(), 1e-5)
        assert torch.allclose(torch.cat([o[0] for o in outs], dim=dim), Y.detach(), rtol=1e-10, atol=1e-12)
        assert float(n.flatten()[0]) == X[0].numel() / G
        back = ogn.backward(gs, [o[1] for o in outs], rstd, n, G, W.detach())
        assert torch.allclose(torch.cat([b[0] for b in back], dim=dim), X.grad, rtol=1e-9, atol=1e-11)
        assert torch.allclose(sum(b[1] for b in back), W.grad, rtol=1e-9, atol=1e-11)
        assert torch.allclose(sum(b[2] for b in back), B.grad, rtol=1e-9, atol=1e-11)


def test_projection_oracle_equals_linear_and_rearrange():
    """The restated projections against F.linear + einops' rearrange with the reference's
    patterns (_attention.py:885-890, 909-916) and autograd through them."""
    from einops import rearrange

    from oracle import projection as op

    torch.manual_seed(13)
    for lead, s, c, heads, d in [((2,), 5, 6, 2, 3), ((2, 3), 4, 8, 3, 2), ((), 7, 4, 1, 4)]:
        x = torch.randn(*lead, s, c, dtype=torch.float64, requires_grad=True)
        w = torch.randn(3 * heads * d, c, dtype=torch.float64, requires_grad=True)
        b = torch.randn(3 * heads * d, dtype=torch.float64, requires_grad=True)
        want = rearrange(torch.nn.functional.linear(x, w, b), "... s (three h d) -> three ... h s d", three=3, h=heads)
        got = op.qkv_forward(x.detach(), w.detach(), b.detach(), heads)
        assert got.shape == want.shape and torch.allclose(got, want.detach(), rtol=1e-12, atol=1e-12)
        g = torch.randn_like(want)
        want.backward(g)
        gx, gw, gb = op.qkv_backward(g, x.detach(), w.detach(), heads)
        assert torch.allclose(gx, x.grad, rtol=1e-11, atol=1e-11)
        assert torch.allclose(gw, w.grad, rtol=1e-11, atol=1e-11)
        assert torch.allclose(gb, b.grad, rtol=1e-11, atol=1e-11)

        o = torch.randn(*lead, heads, s, d, dtype=torch.float64, requires_grad=True)
        wo = torch.randn(5, heads * d, dtype=torch.float64, requires_grad=True)
        bo = torch.randn(5, dtype=torch.float64, requires_grad=True)
        want = torch.nn.functional.linear(rearrange(o, "... h s d -> ... s (h d)").contiguous(), wo, bo)
        got = op.heads_forward(o.detach(), wo.detach(), bo.detach())
        assert got.shape == want.shape and torch.allclose(got, want.detach(), rtol=1e-12, atol=1e-12)
        g = torch.randn_like(want)
        want.backward(g)
        go, gw, gb = op.heads_backward(g, o.detach(), wo.detach())
        assert torch.allclose(go, o.grad, rtol=1e-11, atol=1e-11)
        assert torch.allclose(gw, wo.grad, rtol=1e-11, atol=1e-11)
        assert torch.allclose(gb, bo.grad, rtol=1e-11, atol=1e-11)
