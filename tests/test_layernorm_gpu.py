"""HIP sharded LayerNorm against the oracle and nn.LayerNorm (GPU).

Tolerances: fp32 path atol 1e-5 / rtol 1e-5 (the reference's own test uses 1e-3,
tests/modules/normalization/test_normalization.py); bf16 path rel-L2 2e-2.
"""

import pytest
import torch
import torch.nn.functional as F

from helpers import rel_l2
from jigsaw_amd import layernorm as jl
from oracle import layernorm as ol

pytestmark = pytest.mark.gpu


class ShardGroup:
    """Channel group stand-in on one GPU: holds the other shards' statistics, in the
    order the forward / backward ask for them."""

    def __init__(self, size, others):
        self._size = size
        self.others = list(others)  # per all_reduce call: list of peer tensors
        self.calls = []

    def size(self):
        return self._size

    def all_reduce(self, t, op):
        peers = self.others.pop(0)
        self.calls.append(op)
        total = t.clone()
        for p in peers:
            total += p.to(t.device, t.dtype)
        t.copy_(total / self._size if op == "avg" else total)


@pytest.mark.parametrize("rows,cols", [((4, 33), 256), ((2, 5, 7), 96), ((1, 4096), 256), ((3,), 1000), ((9,), 130)])
def test_partial_stats(rows, cols, dev):
    torch.manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = (torch.randn(*rows, cols) * 3 + 1.5).to(dtype)
        m, v = jl.partial_stats(x.to(dev))
        wm, wv = ol.partial_stats(x.double())
        torch.testing.assert_close(m.cpu().double(), wm, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(v.cpu().double(), wv, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("G", [1, 2, 4])
@pytest.mark.parametrize("bias", [True, False])
def test_layernorm_forward_backward_fp32(G, bias, dev):
    torch.manual_seed(1)
    C, eps = 64 * G, 1e-5
    x = torch.randn(2, 37, C)
    w = 1 + 0.2 * torch.randn(C)
    b = 0.2 * torch.randn(C) if bias else None
    g = torch.randn(2, 37, C)
    xs, ws, gs = (list(t.chunk(G, -1)) for t in (x, w, g))
    bs = list(b.chunk(G, -1)) if bias else [None] * G
    ys, xns, std = ol.forward([t.double() for t in xs], [t.double() for t in ws], [None if t is None else t.double() for t in bs], eps)
    gxs, gws, gbs = ol.backward([t.double() for t in gs], xns, [t.double() for t in ws], std, has_bias=bias)
    # full-width torch layer norm agrees with the oracle
    torch.testing.assert_close(torch.cat(ys, -1), F.layer_norm(x.double(), (C,), w.double(), None if b is None else b.double(), eps), atol=1e-10, rtol=1e-8)

    for r in range(G):
        peers = [i for i in range(G) if i != r]
        lm = [ol.partial_stats(xs[i]) for i in range(G)]
        mean = torch.stack([m for m, _ in lm]).mean(0)
        others = []
        if G > 1:
            others.append([lm[i][0] for i in peers])
            others.append([lm[i][1] + (lm[i][0] - mean) ** 2 for i in peers])
            gxn = [gs[i] * ws[i] for i in range(G)]
            others.append([gxn[i].mean(-1, keepdim=True) for i in peers])
            others.append([(gxn[i] * xns[i].float()).sum(-1, keepdim=True) for i in peers])
        grp = ShardGroup(G, others)
        xr = xs[r].to(dev).requires_grad_()
        wr = ws[r].to(dev).requires_grad_()
        br = bs[r].to(dev).requires_grad_() if bias else None
        y, x_norm, w_out, var_eps = jl._LayerNorm.apply(xr, wr, br, grp, eps)
        assert y.dtype == torch.float32 and not x_norm.requires_grad
        torch.testing.assert_close(y.cpu().double(), ys[r], atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(x_norm.cpu().double(), xns[r], atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(var_eps.cpu().double(), std**2, atol=1e-6, rtol=1e-5)
        y.backward(gs[r].to(dev))
        torch.testing.assert_close(xr.grad.cpu().double(), gxs[r], atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(wr.grad.cpu().double(), gws[r], atol=1e-4, rtol=1e-5)
        if bias:
            torch.testing.assert_close(br.grad.cpu().double(), gbs[r], atol=1e-4, rtol=1e-5)
        if G > 1:
            assert grp.calls == ["avg", "avg", "avg", "sum"]


WIDTH_CASES = [
    # local width, leading shape, dtype: widths that are a multiple of 8 up to 2048 run on the kernels that
    # hold rows in registers (1 to 4 chunks a lane, several rows a wavefront when narrow), the rest on
    # the kernels that walk a row
    (8, (3, 5), torch.float32), (24, (67,), torch.float32), (24, (67,), torch.bfloat16), (128, (1,), torch.float32),
    (136, (2, 77), torch.float16), (512, (130,), torch.bfloat16), (1000, (41,), torch.float32),
    (1536, (9,), torch.bfloat16), (2048, (2, 3), torch.float32), (2048, (35,), torch.bfloat16),
    (130, (19,), torch.float32), (1996, (5,), torch.bfloat16), (4, (33,), torch.float32),
]


@pytest.mark.parametrize("cols,lead,dtype", WIDTH_CASES, ids=lambda v: str(v).replace("torch.", ""))
def test_layernorm_two_shards_over_widths(cols, lead, dtype, dev):
    """Forward and backward of one of two channel shards, over the local widths that pick the
    different row kernels, against the oracle in fp64."""
    torch.manual_seed(cols)
    G, eps = 2, 1e-5
    C = cols * G
    x = (torch.randn(*lead, C) * 2 + 0.5).to(dtype)
    w = (1 + 0.2 * torch.randn(C)).to(dtype)
    b = (0.2 * torch.randn(C)).to(dtype)
    g = torch.randn(*lead, C).to(dtype)
    xs, ws, bs, gs = (list(t.chunk(G, -1)) for t in (x, w, b, g))
    ys, xns, std = ol.forward([t.double() for t in xs], [t.double() for t in ws], [t.double() for t in bs], eps)
    gxs, gws, gbs = ol.backward([t.double() for t in gs], xns, [t.double() for t in ws], std, has_bias=True)
    lm = [ol.partial_stats(t.double()) for t in xs]
    mean = torch.stack([m for m, _ in lm]).mean(0)
    gxn = [gs[i].double() * ws[i].double() for i in range(G)]
    r, o = 1, 0
    grp = ShardGroup(G, [[lm[o][0]], [lm[o][1] + (lm[o][0] - mean) ** 2],
                         [gxn[o].mean(-1, keepdim=True)], [(gxn[o] * xns[o]).sum(-1, keepdim=True)]])
    xr, wr, br = (t.to(dev).requires_grad_() for t in (xs[r], ws[r], bs[r]))
    y, x_norm, _, var_eps = jl._LayerNorm.apply(xr, wr, br, grp, eps)
    y.backward(gs[r].to(dev))
    assert grp.calls == ["avg", "avg", "avg", "sum"]
    # the statistics travel in the tensor dtype
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    torch.testing.assert_close(var_eps.cpu().double(), std**2, atol=tol, rtol=tol)
    if dtype == torch.float32:
        for got, want, tol in ((y, ys[r], 1e-5), (x_norm, xns[r], 1e-5), (xr.grad, gxs[r], 2e-5)):
            torch.testing.assert_close(got.cpu().double(), want, atol=tol, rtol=1e-5)
        torch.testing.assert_close(wr.grad.cpu().double(), gws[r], atol=2e-4, rtol=1e-4)
        torch.testing.assert_close(br.grad.cpu().double(), gbs[r], atol=2e-4, rtol=1e-4)
    else:
        for got, want in ((y, ys[r]), (x_norm, xns[r]), (xr.grad, gxs[r]), (wr.grad, gws[r]), (br.grad, gbs[r])):
            assert got.dtype == dtype and rel_l2(got, want) < 2e-2


def test_layernorm_under_autocast_returns_fp32_and_leaf_dtype_grad(dev):
    """LayerNorm under autocast computes in fp32 (reference: tests/test_autocast.py:265-292)."""
    torch.manual_seed(2)
    C = 256
    x = torch.randn(4, 128, C).bfloat16()
    w, b = 1 + 0.2 * torch.randn(C), 0.2 * torch.randn(C)
    want = F.layer_norm(x.float(), (C,), w, b, 1e-5)
    xr = x.to(dev).requires_grad_()
    wr, br = w.to(dev).requires_grad_(), b.to(dev).requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = jl.layer_norm(xr, wr, br, None, 1e-5)
    assert y.dtype == torch.float32
    torch.testing.assert_close(y.cpu(), want, atol=1e-4, rtol=1e-4)
    y.backward(torch.randn_like(y))
    assert xr.grad.dtype == torch.bfloat16 and wr.grad.dtype == torch.float32


def test_layernorm_bf16_config4_shape(dev):
    """Sharded-channel LayerNorm of config 4: dim 512, 256 local, 4096 tokens."""
    torch.manual_seed(3)
    C, G, eps = 512, 2, 1e-5
    x = torch.randn(1, 4096, C)
    w, b = 1 + 0.2 * torch.randn(C), 0.2 * torch.randn(C)
    want = F.layer_norm(x, (C,), w, b, eps)
    xs, ws, bs = (list(t.chunk(G, -1)) for t in (x, w, b))
    lm = [ol.partial_stats(t) for t in xs]
    mean = torch.stack([m for m, _ in lm]).mean(0)
    for r in range(G):
        o = 1 - r
        grp = ShardGroup(G, [[lm[o][0]], [lm[o][1] + (lm[o][0] - mean) ** 2]])
        y = jl.layer_norm(xs[r].bfloat16().to(dev), ws[r].bfloat16().to(dev), bs[r].bfloat16().to(dev), grp, eps)
        assert y.dtype == torch.bfloat16
        assert rel_l2(y, want.chunk(G, -1)[r]) < 2e-2


# --------------------------------------------------------------------------- #
# nn.LayerNorm over rows one rank holds whole (fused kernels): the oracle with a single shard
# --------------------------------------------------------------------------- #
PLAIN_CASES = [
    # shape, x dtype, out dtype, grad dtype, bias
    ((1, 256, 256, 128), torch.bfloat16, torch.bfloat16, torch.bfloat16, True),   # Swin block tile, autocast
    ((3, 70, 128), torch.bfloat16, torch.float32, torch.float32, True),           # torch's autocast dtypes
    ((5, 33, 8), torch.float32, torch.float32, torch.float32, True),              # one lane per row
    ((2, 9, 200), torch.float32, torch.float32, torch.float32, False),            # 32 lanes, the last ones idle
    ((7, 1000), torch.float32, torch.bfloat16, torch.bfloat16, True),             # two chunks per lane
    ((3, 2048), torch.float16, torch.float16, torch.float16, True),               # widest row the kernels hold
    ((4, 16, 64), torch.float32, torch.float32, torch.bfloat16, True),            # low-precision gradient
]


@pytest.mark.parametrize("case", PLAIN_CASES, ids=lambda c: f"{'x'.join(map(str, c[0]))}_{str(c[1])[6:]}_{str(c[2])[6:]}")
def test_plain_layer_norm_matches_oracle(case, dev):
    shape, xdt, odt, gdt, has_b = case
    torch.manual_seed(11)
    C, eps = shape[-1], 1e-5
    x = (2.0 * torch.randn(*shape) + 0.5).to(xdt)
    w, b = 1 + 0.2 * torch.randn(C), (0.2 * torch.randn(C) if has_b else None)
    g = torch.randn(*shape).to(gdt)
    print(f"plain_layer_norm {case}", flush=True)
    xr = x.to(dev).requires_grad_()
    wr = w.to(dev).requires_grad_()
    br = b.to(dev).requires_grad_() if has_b else None
    y = jl.plain_layer_norm(xr, wr, br, eps, out_dtype=odt)
    assert y.dtype == odt and y.shape == x.shape
    y.backward(g.to(dev))
    ys, xns, std = ol.forward([x.double()], [w.double()], [b.double() if has_b else None], eps)
    gxs, gws, gbs = ol.backward([g.double()], xns, [w.double()], std, has_bias=has_b)
    lo = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 4e-3}
    assert rel_l2(y.detach().cpu(), ys[0]) < lo[odt]
    tol_g = max(lo[gdt], lo[xdt])
    assert xr.grad.dtype == xdt and rel_l2(xr.grad.cpu(), gxs[0]) < tol_g
    assert wr.grad.dtype == torch.float32 and rel_l2(wr.grad.cpu(), gws[0]) < max(lo[gdt], 1e-5)
    if has_b:
        assert rel_l2(br.grad.cpu(), gbs[0]) < max(lo[gdt], 1e-5)


def test_plain_layer_norm_defaults_and_fallback(dev):
    """Default output dtype is torch's (fp32 under autocast); a width the fused kernels do not take
    (not a multiple of 8) goes through the partial-statistics kernels; no rows is fine."""
    torch.manual_seed(12)
    x = torch.randn(4, 50, 128).bfloat16().to(dev)
    w, b = torch.ones(128, device=dev), torch.zeros(128, device=dev)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert jl.plain_layer_norm(x, w, b).dtype == torch.float32
    assert jl.plain_layer_norm(x, w, b).dtype == torch.bfloat16
    x2 = torch.randn(6, 130, device=dev)
    w2, b2 = torch.randn(130, device=dev), torch.randn(130, device=dev)
    torch.testing.assert_close(jl.plain_layer_norm(x2, w2, b2).cpu(), F.layer_norm(x2.cpu(), (130,), w2.cpu(), b2.cpu()),
                               atol=1e-5, rtol=1e-5)
    assert jl.plain_layer_norm(x[:0], w, b).shape == (0, 50, 128)


def test_plain_layer_norm_entry_point_refuses_what_it_cannot_do(dev):
    """Through the C ABI: widths that are not a multiple of 8 or beyond 2048 columns are 'unsupported'
    (status -2, NotImplementedError), a bf16 input with an fp16 output is a bad argument (status -1)."""
    from jigsaw_amd import _lib

    lib = _lib.load()
    assert lib.jg_ln_plain_supported(128) == 1 and lib.jg_ln_plain_supported(2048) == 1
    assert lib.jg_ln_plain_supported(12) == 0 and lib.jg_ln_plain_supported(2056) == 0 and lib.jg_ln_plain_supported(4) == 0
    x = torch.randn(4, 16, device=dev)
    y, mean, rstd, w = torch.empty_like(x), torch.empty(4, device=dev), torch.empty(4, device=dev), torch.ones(16, device=dev)

    def call(cols, x_dt, y_dt):
        return lib.jg_ln_plain_fwd(_lib.ptr(y), _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(x), _lib.ptr(w), None, 4, cols, 1e-5,
                                   x_dt, y_dt, _lib.stream_ptr(dev))

    f32, bf16, f16 = (_lib.dtype_code(t) for t in (torch.float32, torch.bfloat16, torch.float16))
    assert call(16, f32, f32) == 0
    assert call(12, f32, f32) == -2
    assert call(16, bf16, f16) == -1
    with pytest.raises(NotImplementedError):
        _lib.check(call(12, f32, f32), "jg_ln_plain_fwd")
    torch.cuda.synchronize()


def test_plain_layer_norm_takes_non_contiguous_input(dev):
    torch.manual_seed(13)
    x = torch.randn(6, 64, 10, device=dev).transpose(1, 2)  # (6, 10, 64) view with strides
    w, b = torch.randn(64, device=dev), torch.randn(64, device=dev)
    got = jl.plain_layer_norm(x, w, b)
    want = F.layer_norm(x.cpu().double(), (64,), w.cpu().double(), b.cpu().double())
    assert rel_l2(got.cpu(), want) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plain_layer_norm_fork_adds_the_residual_gradient_in_the_kernel(dtype, dev):
    """x + f(norm(x)) through plain_layer_norm_fork against the same expression with the plain call
    and autograd's own sum of the two gradients of x: same numbers (the kernel adds the gradient
    that comes over the residual connection to the rounded LayerNorm gradient, as the separate sum
    does)."""
    from jigsaw_amd import layernorm as jl

    torch.manual_seed(5)
    x = torch.randn(3, 37, 128, device=dev).to(dtype)
    w, b = torch.randn(128, device=dev), torch.randn(128, device=dev)
    g = torch.randn(3, 37, 128, device=dev).to(dtype)

    def run(fork):
        xs = x.clone().requires_grad_()
        ws, bs = w.clone().requires_grad_(), b.clone().requires_grad_()
        if fork:
            y, keep = jl.plain_layer_norm_fork(xs, ws, bs, 1e-5, out_dtype=dtype)
        else:
            y, keep = jl.plain_layer_norm(xs, ws, bs, 1e-5, out_dtype=dtype), xs
        out = keep + torch.tanh(y)
        out.backward(g)
        return out, xs.grad, ws.grad, bs.grad

    a, b_ = run(True), run(False)
    torch.cuda.synchronize()
    for got, want in zip(a, b_):
        assert torch.equal(got, want)
    # only the branch, and only the connection
    xs = x.clone().requires_grad_()
    y, keep = jl.plain_layer_norm_fork(xs, w, b, 1e-5, out_dtype=dtype)
    keep.backward(g)
    assert torch.equal(xs.grad, g)
