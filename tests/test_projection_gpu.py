"""Projections around the attention core (head split / merge fused into the GEMM):
HIP kernels through the C ABI against the oracle (fp64 on the same rounded inputs).

Tolerances: rel-L2 <= 1e-5 in fp32, 2e-2 in bf16, 4e-3 in fp16. The layout itself is
checked exactly: with a one-hot weight the projection is a pure copy.
"""

import pytest
import torch

from helpers import rel_l2
from jigsaw_amd import projection as jp
from oracle import projection as op

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 4e-3}


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


CASES = [
    # lead, seq, channels, heads, head_dim, out features of the second projection, dtype, bias
    ((1,), 4096, 512, 8, 64, 512, torch.bfloat16, True),     # the ring-attention configuration
    ((4, 16), 64, 128, 4, 32, 128, torch.bfloat16, True),    # Swin windows: two leading axes
    ((2,), 200, 96, 3, 32, 80, torch.bfloat16, False),       # ragged tiles: 400 tokens, 288 / 96 / 80 features
    ((3,), 50, 72, 3, 24, 40, torch.bfloat16, True),         # head_dim 24, contraction not a multiple of 64
    ((1,), 130, 64, 2, 20, 24, torch.bfloat16, True),        # head_dim 20: not a multiple of 8, FMA path
    ((2,), 33, 24, 2, 8, 10, torch.float32, True),
    ((2, 2), 17, 16, 1, 16, 16, torch.float16, True),
    ((0,), 16, 32, 2, 16, 32, torch.bfloat16, True),         # empty batch
]


def _id(c):
    return f"{'x'.join(map(str, c[0]))}_{c[1]}x{c[2]}_h{c[3]}d{c[4]}_{c[5]}_{str(c[6]).split('.')[-1]}"


@pytest.mark.parametrize("case", CASES, ids=_id)
def test_projections_match_oracle(case, dev):
    lead, s, c, heads, d, n2, dtype, has_b = case
    tol = TOL[dtype]
    torch.manual_seed(21)
    x = torch.randn(*lead, s, c).to(dtype)
    w = (torch.randn(3 * heads * d, c) / c ** 0.5).to(dtype)
    b = (0.1 * torch.randn(3 * heads * d)).to(dtype) if has_b else None
    g = torch.randn(3, *lead, heads, s, d).to(dtype)
    print(f"qkv_projection {case}", flush=True)
    xd, wd = x.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    bd = b.to(dev).requires_grad_() if has_b else None
    y = jp.qkv_projection(xd, wd, bd, heads)
    assert y.shape == (3, *lead, heads, s, d) and y.dtype == dtype and y.is_contiguous()
    y.backward(g.to(dev))
    want = op.qkv_forward(x.double(), w.double(), b.double() if has_b else None, heads)
    gx, gw, gb = op.qkv_backward(g.double(), x.double(), w.double(), heads)
    if x.numel():
        assert rel_l2(y.detach().cpu(), want) <= tol
        assert rel_l2(xd.grad.cpu(), gx) <= tol
        assert rel_l2(wd.grad.cpu(), gw) <= tol
        if has_b:
            assert rel_l2(bd.grad.cpu(), gb) <= tol
    else:
        assert float(wd.grad.abs().sum()) == 0.0 and xd.grad.shape == x.shape

    o = torch.randn(*lead, heads, s, d).to(dtype)
    wo = (torch.randn(n2, heads * d) / (heads * d) ** 0.5).to(dtype)
    bo = (0.1 * torch.randn(n2)).to(dtype) if has_b else None
    g2 = torch.randn(*lead, s, n2).to(dtype)
    print(f"heads_projection {case}", flush=True)
    od, wod = o.to(dev).requires_grad_(), wo.to(dev).requires_grad_()
    bod = bo.to(dev).requires_grad_() if has_b else None
    z = jp.heads_projection(od, wod, bod)
    assert z.shape == (*lead, s, n2) and z.dtype == dtype
    z.backward(g2.to(dev))
    want = op.heads_forward(o.double(), wo.double(), bo.double() if has_b else None)
    go, gw, gb = op.heads_backward(g2.double(), o.double(), wo.double())
    if o.numel():
        assert rel_l2(z.detach().cpu(), want) <= tol
        assert rel_l2(od.grad.cpu(), go) <= tol
        assert rel_l2(wod.grad.cpu(), gw) <= tol
        if has_b:
            assert rel_l2(bod.grad.cpu(), gb) <= tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_identity_weight_is_the_rearrange_exactly(dtype, dev):
    """With the identity as weight and no bias the projection only moves data: the
    result must equal torch's reshape / permute of the input bit for bit."""
    torch.manual_seed(22)
    lead, s, heads, d = (2, 3), 40, 3, 16
    c = 3 * heads * d
    x = torch.randn(*lead, s, c, device=dev).to(dtype)
    eye = torch.eye(c, device=dev, dtype=dtype)
    y = jp.qkv_projection(x, eye, None, heads)
    want = x.reshape(*lead, s, 3, heads, d).permute(3, 0, 1, 4, 2, 5).contiguous()
    assert torch.equal(y, want)
    o = torch.randn(*lead, heads, s, d, device=dev).to(dtype)
    eye = torch.eye(heads * d, device=dev, dtype=dtype)
    z = jp.heads_projection(o, eye, None)
    want = o.permute(0, 1, 3, 2, 4).reshape(*lead, s, heads * d)
    assert torch.equal(z, want)


def test_full_size_against_torch_gemm(dev):
    """Eight sequences of the ring-attention configuration: the fused projections against
    torch's own bf16 GEMM + rearrange on the GPU (both accumulate in fp32 and round once,
    so they agree to a few bf16 roundings), and forward -> backward runs at full size."""
    torch.manual_seed(23)
    bsz, s, c, heads, d = 8, 4096, 512, 8, 64
    x = torch.randn(bsz, s, c, device=dev).bfloat16().requires_grad_()
    w = (torch.randn(3 * c, c, device=dev) / c ** 0.5).bfloat16().requires_grad_()
    b = (0.1 * torch.randn(3 * c, device=dev)).bfloat16().requires_grad_()
    y = jp.qkv_projection(x, w, b, heads)
    want = torch.nn.functional.linear(x.detach(), w.detach(), b.detach())
    want = want.reshape(bsz, s, 3, heads, d).permute(2, 0, 3, 1, 4)
    assert rel_l2(y.detach().float(), want.float()) <= 4e-3
    g = torch.randn_like(y)
    y.backward(g)
    gflat = g.permute(1, 3, 0, 2, 4).reshape(bsz * s, 3 * c)
    assert rel_l2(x.grad.float(), (gflat.float() @ w.detach().float()).reshape(bsz, s, c)) <= 4e-3
    assert rel_l2(w.grad.float(), gflat.float().t() @ x.detach().reshape(-1, c).float()) <= 4e-3
    assert rel_l2(b.grad.float(), gflat.float().sum(0)) <= 4e-3


@pytest.mark.parametrize("shape,n_out,dtype,has_b", [
    ((1, 256, 256, 128), 512, torch.bfloat16, True),   # the MLP of a Swin block on a 256 x 256 token tile
    ((3, 50, 72), 40, torch.bfloat16, True),
    ((130, 64), 24, torch.bfloat16, False),
    ((2, 33, 24), 10, torch.float32, True),
    ((0, 32), 16, torch.bfloat16, True),
], ids=lambda v: str(v).replace(" ", ""))
def test_linear_matches_oracle(shape, n_out, dtype, has_b, dev):
    """``projection.linear`` is the output projection with one head: the oracle's heads_forward /
    heads_backward on ``x`` viewed as ``(..., 1, tokens, features)``."""
    tol = TOL[dtype]
    torch.manual_seed(5)
    k = shape[-1]
    x = torch.randn(*shape).to(dtype)
    w = (torch.randn(n_out, k) / k ** 0.5).to(dtype)
    b = (0.1 * torch.randn(n_out)).to(dtype) if has_b else None
    g = torch.randn(*shape[:-1], n_out).to(dtype)
    print(f"linear {shape} -> {n_out} {dtype}", flush=True)
    xd, wd = x.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    bd = b.to(dev).requires_grad_() if has_b else None
    y = jp.linear(xd, wd, bd)
    assert y.shape == g.shape and y.dtype == dtype
    y.backward(g.to(dev))
    if x.numel():
        x3 = x.reshape(1, 1, -1, k).double()
        want = op.heads_forward(x3, w.double(), b.double() if has_b else None).reshape(g.shape)
        gx, gw, gb = op.heads_backward(g.reshape(1, -1, n_out).double(), x3, w.double())
        assert rel_l2(y.detach().cpu(), want) <= tol
        assert rel_l2(xd.grad.cpu(), gx.reshape(shape)) <= tol
        assert rel_l2(wd.grad.cpu(), gw) <= tol
        if has_b:
            assert rel_l2(bd.grad.cpu(), gb) <= tol
    else:
        assert float(wd.grad.abs().sum()) == 0.0 and xd.grad.shape == x.shape


@pytest.mark.parametrize("shape,n_out", [((4, 64, 128), 256), ((3, 50, 20), 12)], ids=["mfma", "fma"])
def test_fp32_parameters_get_unrounded_fp32_gradients(shape, n_out, dev):
    """fp32 parameters with bf16 activations (autocast): the weight and bias gradients come back in
    fp32 straight from the fp32 sums, closer to the oracle than one bf16 rounding allows."""
    torch.manual_seed(6)
    k = shape[-1]
    x = torch.randn(*shape).bfloat16()
    w, b = torch.randn(n_out, k) / k ** 0.5, 0.1 * torch.randn(n_out)
    g = torch.randn(*shape[:-1], n_out).bfloat16()
    xd = x.to(dev).requires_grad_()
    wd, bd = w.to(dev).requires_grad_(), b.to(dev).requires_grad_()
    jp.linear(xd, wd, bd).backward(g.to(dev))
    assert wd.grad.dtype == torch.float32 and bd.grad.dtype == torch.float32
    x3 = x.reshape(1, 1, -1, k).double()
    _, gw, gb = op.heads_backward(g.reshape(1, -1, n_out).double(), x3, w.bfloat16().double())
    assert rel_l2(wd.grad.cpu(), gw) < 1e-5 and rel_l2(bd.grad.cpu(), gb) < 1e-5


@pytest.mark.parametrize("rows,dim,hid,with_res", [((3, 50), 64, 256, True), ((200,), 128, 512, True), ((2, 33), 40, 96, False)])
def test_gelu_mlp_fused_epilogues(rows, dim, hid, with_res, dev):
    """residual + Linear(GELU(Linear(x))) on the fused epilogues (GELU beside the pre-activation, the
    GELU derivative and the residual sum on the way out of a GEMM) against fp64 autograd of the same
    expression with torch's erf GELU (examples/swin.py:190-209). rel-L2 2e-2: bf16 operands, the bar
    of the other bf16 projection tests; fp32 parameters get fp32 gradients."""
    torch.manual_seed(11)
    x = torch.randn(*rows, dim).bfloat16()
    res = torch.randn(*rows, dim).bfloat16() if with_res else None
    w1, b1 = torch.randn(hid, dim) * dim**-0.5, torch.randn(hid) * 0.1
    w2, b2 = torch.randn(dim, hid) * hid**-0.5, torch.randn(dim) * 0.1
    g = torch.randn(*rows, dim).bfloat16()

    leaves = [t.double().requires_grad_() for t in (x, w1.bfloat16(), b1.bfloat16(), w2.bfloat16(), b2.bfloat16())]
    xd, w1d, b1d, w2d, b2d = leaves
    want = torch.nn.functional.linear(torch.nn.functional.gelu(torch.nn.functional.linear(xd, w1d, b1d)), w2d, b2d)
    if with_res:
        rd = res.double().requires_grad_()
        want = rd + want
    want.backward(g.double())

    gx = x.to(dev).requires_grad_()
    params = [t.to(dev).requires_grad_() for t in (w1, b1, w2, b2)]  # fp32 parameters, as under autocast
    gres = res.to(dev).requires_grad_() if with_res else None
    assert jp.mlp_fusable(gx, params[0], params[2], gres)
    out = jp.gelu_mlp(gx, *params, residual=gres)
    out.backward(g.to(dev))
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and rel_l2(out, want) < 2e-2
    assert rel_l2(gx.grad, xd.grad) < 2e-2
    for name, got, w in zip(("w1", "b1", "w2", "b2"), params, (w1d, b1d, w2d, b2d)):
        assert got.grad.dtype == torch.float32
        assert rel_l2(got.grad, w.grad) < 2e-2, f"{name}: {rel_l2(got.grad, w.grad):.3e}"
    if with_res:
        assert torch.equal(gres.grad, g.to(dev))
    # the separate-steps form of the same function (what runs when the fused form does not apply)
    y2 = jp.linear(torch.nn.functional.gelu(jp.linear(gx.detach(), *[p.detach() for p in params[:2]])), *[p.detach() for p in params[2:]])
    if with_res:
        y2 = gres.detach() + y2
    assert rel_l2(out, y2) < 1e-2


def test_fused_projection_entry_refuses_what_it_has_no_kernel_for(dev):
    """jg_proj_nt_fused: an unknown epilogue code and a missing aux tensor are bad arguments
    (ValueError), operands other than bf16 are not supported (NotImplementedError); the host
    function gelu_mlp then takes the separate-steps route by itself."""
    from jigsaw_amd import _lib

    x = torch.randn(16, 64, device=dev).bfloat16()
    w = torch.randn(32, 64, device=dev).bfloat16()
    out, aux = torch.empty(16, 32, device=dev).bfloat16(), torch.empty(16, 32, device=dev).bfloat16()
    lib = _lib.load()

    def call(epi, a=x, wt=w, o=out, au=aux):
        return lib.jg_proj_nt_fused(_lib.ptr(o), _lib.ptr(au), epi, _lib.ptr(a), _lib.ptr(wt), None,
                                    _lib.dtype_code(a.dtype), 16, 32, 64, _lib.stream_ptr(dev))

    with pytest.raises(ValueError):
        _lib.check(call(9), "jg_proj_nt_fused")
    with pytest.raises(ValueError):
        _lib.check(call(jp.EPI_ADD, au=None), "jg_proj_nt_fused")
    with pytest.raises(NotImplementedError):
        _lib.check(call(jp.EPI_GELU, a=x.float(), wt=w.float(), o=out.float(), au=aux.float()), "jg_proj_nt_fused")
    assert _lib.check(call(jp.EPI_GELU), "jg_proj_nt_fused") is None
    torch.cuda.synchronize()
    want = torch.nn.functional.gelu((x.float() @ w.float().T).bfloat16().float())
    assert rel_l2(aux, want) < 1e-2
    # fp32 tokens: not fusable, same function through separate steps
    xf = torch.randn(4, 64, device=dev)
    w2 = torch.randn(64, 32, device=dev)
    assert not jp.mlp_fusable(xf, w.float(), w2, None)
    y = jp.gelu_mlp(xf, w.float(), None, w2, None)
    ref = torch.nn.functional.linear(torch.nn.functional.gelu(torch.nn.functional.linear(xf, w.float())), w2)
    assert rel_l2(y, ref) < 1e-5
