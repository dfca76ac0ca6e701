"""HIP attention core, fused ring step and ring loops against the oracle (GPU).

Tolerances: rel-L2 1e-5 for fp32 tensors, 2e-2 for bf16 / fp16 (north-star bar); the
reference's own ring tests use atol 1e-3 fp32 / 1e-2 bf16
(tests/modules/attention/test_ring_attention.py:159-368).
"""

import pytest
import torch

from helpers import rel_l2
from jigsaw_amd import attention as ja
from oracle import attention as oa

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _qkv(b, h, sq, sk, d, dtype, seed=0):
    torch.manual_seed(seed)
    q = (torch.randn(b, h, sq, d) / d**0.5).to(dtype)
    k = torch.randn(b, h, sk, d).to(dtype)
    v = torch.randn(b, h, sk, d).to(dtype)
    return q, k, v


CORE_SHAPES = [
    (3, 6, 64, 64, 16),   # the reference's ring test shape per chunk (b=3, h=6, n=16*4, d=16)
    (2, 2, 50, 70, 32),   # ragged
    (1, 3, 130, 33, 64),
    (1, 2, 128, 128, 64),  # MFMA path for bf16
    (2, 2, 256, 384, 64),  # MFMA path for bf16
    (1, 1, 40, 40, 128),
    (1, 2, 17, 9, 8),
    (1, 3, 256, 128, 32),  # head size below 64: bf16 runs the head-size-64 MFMA kernels on zero-padded q, k, v
    (2, 2, 128, 256, 16),
    (1, 2, 200, 300, 32),  # ragged queries and keys below head size 64: padded, spare-column key mask
    (1, 2, 130, 260, 64),  # ragged at head size 64: MFMA on 256 keys + FMA kernel on 4, merged
    (2, 1, 128, 130, 16),
    (1, 1, 70, 1000, 64),
    (1, 2, 128, 256, 128),  # head sizes 96 and 128: their own MFMA kernels for bf16
    (2, 2, 256, 128, 96),
    (1, 1, 384, 640, 128),
    (1, 2, 200, 300, 80),   # padded to head size 96, spare-column key mask
    (1, 1, 130, 260, 128),  # ragged at head size 128: MFMA on 256 keys + FMA kernel on 4, merged
    (1, 1, 70, 200, 96),
    (1, 2, 256, 128, 72),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", CORE_SHAPES, ids=lambda s: "b{}h{}q{}k{}d{}".format(*s))
def test_core_forward_backward_match_oracle(shape, dtype, dev):
    b, h, sq, sk, d = shape
    q, k, v = _qkv(b, h, sq, sk, d, dtype)
    scale = d**-0.5
    want_o, want_l = oa.core_forward(q.double(), k.double(), v.double(), scale)
    out, lse, rng = ja.forward(q.to(dev), k.to(dev), v.to(dev), scale, 0.0, layout="bhsd")
    assert rng is None and out.dtype == dtype and lse.dtype == torch.float32
    assert rel_l2(out, want_o) < TOL[dtype], f"out {rel_l2(out, want_o):.3e}"
    assert rel_l2(lse, want_l) < max(TOL[dtype] * 0.1, 1e-5), f"lse {rel_l2(lse, want_l):.3e}"

    dout = torch.randn(b, h, sq, d).to(dtype)
    # backward from the oracle's own (global) out / lse, rounded as the ring would hold them
    o_in, l_in = want_o.to(dtype), want_l.float()
    wdq, wdk, wdv = oa.core_backward(dout.double(), q.double(), k.double(), v.double(), o_in.double(), l_in.double(), scale)
    dq, dk, dv = ja.backward(dout.to(dev), q.to(dev), k.to(dev), v.to(dev), o_in.to(dev), l_in.to(dev), scale, sq, sk)
    assert dq.dtype == dtype
    for name, got, want in (("dq", dq, wdq), ("dk", dk, wdk), ("dv", dv, wdv)):
        assert rel_l2(got, want) < TOL[dtype], f"{name} {rel_l2(got, want):.3e}"


@pytest.mark.parametrize(
    "b,h,n,d,P,dtype",
    [
        (3, 6, 16, 16, 4, torch.float32),
        (3, 6, 16, 16, 4, torch.bfloat16),
        (1, 2, 256, 64, 4, torch.bfloat16),
        (1, 2, 128, 64, 3, torch.float32),
        (1, 2, 128, 128, 3, torch.bfloat16),  # head sizes 128 and 96: their own kernels, merge fused as well
        (1, 1, 256, 96, 2, torch.bfloat16),
        (1, 2, 128, 128, 2, torch.float16),   # fp16 on the matrix cores, merge fused
        (1, 2, 256, 64, 2, torch.float16),    # fp16, head size 64: padded to the 96-wide kernels per step
    ],
)
@pytest.mark.parametrize("rank", [0, 2])
def test_ring_forward_backward_match_full_attention(b, h, n, d, P, dtype, rank, dev):
    """Ring over P local chunks == full softmax attention over the concatenated K/V
    (the reference's method, test_ring_attention.py:267-275), forward and backward."""
    torch.manual_seed(1)
    scale = d**-0.5
    q = (torch.randn(b, h, n, d) / d**0.5).to(dtype)
    ks = [torch.randn(b, h, n, d).to(dtype) for _ in range(P)]
    vs = [torch.randn(b, h, n, d).to(dtype) for _ in range(P)]
    K = torch.cat(ks, 2).double().requires_grad_()
    V = torch.cat(vs, 2).double().requires_grad_()
    Q = q.double().requires_grad_()
    s = (Q @ K.mT) * scale
    full = torch.softmax(s, -1) @ V
    dout = torch.randn(b, h, n, d).to(dtype)
    full.backward(dout.double())

    out, lse = ja.ring_forward(q.to(dev), [t.to(dev) for t in ks], [t.to(dev) for t in vs], scale, rank=rank % P)
    assert out.dtype == dtype and lse.dtype == torch.float32
    assert rel_l2(out, full.detach()) < TOL[dtype], f"out {rel_l2(out, full.detach()):.3e}"
    lse_tol = 1e-5 if dtype == torch.float32 else 1e-3
    lse_err = rel_l2(lse, torch.logsumexp(s.detach(), -1))
    assert lse_err < lse_tol, f"lse {lse_err:.3e}"
    # the oracle's ring loop (its chunk order, merge form and roundings) agrees too
    o_or, l_or = oa.ring_forward(q.float(), [t.float() for t in ks], [t.float() for t in vs], scale, rank=rank % P)
    assert rel_l2(out, o_or) < TOL[dtype]

    dq, dks, dvs = ja.ring_backward(dout.to(dev), q.to(dev), out, lse, [t.to(dev) for t in ks], [t.to(dev) for t in vs], scale)
    assert rel_l2(dq, Q.grad) < TOL[dtype], f"dq {rel_l2(dq, Q.grad):.3e}"
    assert rel_l2(torch.cat(dks, 2), K.grad) < TOL[dtype], f"dk {rel_l2(torch.cat(dks, 2), K.grad):.3e}"
    assert rel_l2(torch.cat(dvs, 2), V.grad) < TOL[dtype], f"dv {rel_l2(torch.cat(dvs, 2), V.grad):.3e}"


@pytest.mark.parametrize("d", [64, 96, 128])
def test_fused_step_equals_core_plus_merge(d, dev):
    """The fused epilogue merge and the separate merge kernel give the same accumulator."""
    q, k, v = _qkv(1, 4, 256, 512, d, torch.bfloat16, seed=2)
    q, k, v = q.to(dev), k.to(dev), v.to(dev)
    scale = d**-0.5
    acc1 = torch.randn(1, 4, 256, d, device=dev)
    l1 = torch.randn(1, 4, 256, device=dev)
    acc2, l2 = acc1.clone(), l1.clone()
    ja.core_forward(q, k, v, scale, out_acc=acc1, lse_acc=l1, want_out=False)
    out_j, l_j = ja.core_forward(q, k, v, scale)
    acc2, l2 = ja.fused_online_softmax_merge_(acc2, l2, out_j, l_j, "bhsd")
    torch.testing.assert_close(acc1, acc2, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(l1, l2, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("d,sq,sk", [(32, 200, 300), (64, 130, 33), (128, 257, 96), (64, 128, 4096)])
def test_fp32_matrix_core_step_with_merge(d, sq, sk, dev):
    """fp32 on the matrix cores, ragged lengths: the step against the oracle in fp64, the fused merge
    against the separate merge kernel and against the merge done in fp64, and a second merge on top."""
    q, k, v = _qkv(2, 3, sq, sk, d, torch.float32, seed=3)
    scale = d**-0.5
    want_o, want_l = oa.core_forward(q.double(), k.double(), v.double(), scale)
    q, k, v = q.to(dev), k.to(dev), v.to(dev)
    out_j, l_j = ja.core_forward(q, k, v, scale)
    assert rel_l2(out_j, want_o) < 1e-5 and rel_l2(l_j, want_l) < 1e-5
    acc1 = torch.randn(2, 3, sq, d, device=dev)
    l1 = torch.randn(2, 3, sq, device=dev)
    acc0, l0 = acc1.double().cpu(), l1.double().cpu()
    acc2, l2 = acc1.clone(), l1.clone()
    assert ja.core_forward(q, k, v, scale, out_acc=acc1, lse_acc=l1, want_out=False) == (None, None)
    acc2, l2 = ja.fused_online_softmax_merge_(acc2, l2, out_j, l_j, "bhsd")
    torch.testing.assert_close(acc1, acc2, atol=2e-6, rtol=2e-6)
    torch.testing.assert_close(l1, l2, atol=2e-6, rtol=2e-6)
    l_new = torch.logaddexp(l0, want_l)
    acc_new = acc0 * (l0 - l_new).exp().unsqueeze(-1) + want_o * (want_l - l_new).exp().unsqueeze(-1)
    assert rel_l2(acc1, acc_new) < 1e-5 and rel_l2(l1, l_new) < 1e-5
    # a fresh accumulator (lse -inf) takes the step as it is, and hands it out on request
    acc3 = torch.zeros_like(acc1)
    l3 = torch.full_like(l1, float("-inf"))
    out3, lse3 = ja.core_forward(q, k, v, scale, out_acc=acc3, lse_acc=l3)
    assert torch.equal(out3, out_j) and torch.equal(lse3, l_j)
    torch.testing.assert_close(acc3, out_j, atol=1e-7, rtol=1e-6)
    torch.testing.assert_close(l3, l_j, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("d", [8, 16, 96])
def test_fp32_head_sizes_between_the_matrix_core_sizes(d, dev):
    q, k, v = _qkv(1, 2, 70, 45, d, torch.float32, seed=4)
    scale = d**-0.5
    want_o, want_l = oa.core_forward(q.double(), k.double(), v.double(), scale)
    dout = torch.randn(1, 2, 70, d)
    wdq, wdk, wdv = oa.core_backward(dout.double(), q.double(), k.double(), v.double(), want_o, want_l, scale)
    out, lse = ja.core_forward(q.to(dev), k.to(dev), v.to(dev), scale)
    assert out.shape == q.shape and rel_l2(out, want_o) < 1e-5 and rel_l2(lse, want_l) < 1e-5
    dq, dk, dv = ja.core_backward(dout.to(dev), q.to(dev), k.to(dev), v.to(dev), want_o.float().to(dev), want_l.float().to(dev), scale)
    for got, want in ((dq, wdq), (dk, wdk), (dv, wdv)):
        assert got.shape == want.shape and rel_l2(got, want) < 1e-5


@pytest.mark.parametrize("pattern", ["late_spike", "rising", "first_tile_low", "huge_logits", "one_hot_rows"])
def test_mfma_forward_when_the_running_max_moves(pattern, dev):
    """The head-size-64 kernel keeps a per-query reference exponent that follows the running
    max lazily (it moves only when a tile exceeds it by 2^8) and folds it into the score
    product. Score patterns that move the max late, often, by hundreds of powers of two, or
    start far below zero must give the fp64 softmax all the same (bf16 bar), and so must
    the merge into a ring accumulator that already holds a chunk."""
    torch.manual_seed(11)
    b, h, sq, sk, d = 1, 2, 256, 1024, 64
    q = torch.randn(b, h, sq, d)
    k = torch.randn(b, h, sk, d)
    v = torch.randn(b, h, sk, d)
    if pattern == "late_spike":        # a few keys near the end dominate everything before them
        k[:, :, 900:905] *= 12.0
    elif pattern == "rising":          # the max moves in almost every tile
        k *= torch.linspace(0.2, 6.0, sk)[None, None, :, None]
    elif pattern == "first_tile_low":  # the first tiles hold only very negative scores
        k[:, :, :128] = -3.0 * q[:, :, :1].mean(2, keepdim=True).expand(b, h, 128, d) - 4.0
        q = q.abs()
    elif pattern == "huge_logits":     # logits in the thousands: softmax is one-hot, nothing may overflow
        q, k = q * 30.0, k * 30.0
    elif pattern == "one_hot_rows":    # every query has exactly one matching key, somewhere in the chunk
        k = torch.nn.functional.normalize(k, dim=-1) * 40.0
        q = k[:, :, torch.randperm(sk)[:sq]].clone()
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    scale = d**-0.5
    want_o, want_l = oa.core_forward(q.double(), k.double(), v.double(), scale)
    out, lse = ja.core_forward(q.to(dev), k.to(dev), v.to(dev), scale)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    assert rel_l2(out, want_o) < 2e-2, f"out {rel_l2(out, want_o):.3e}"
    assert rel_l2(lse, want_l) < 2e-3, f"lse {rel_l2(lse, want_l):.3e}"  # the core test's bar for bf16
    # the same chunk as the second step of a ring whose first chunk is ordinary
    k0, v0 = torch.randn(b, h, 256, d).bfloat16(), torch.randn(b, h, 256, d).bfloat16()
    ring_o, ring_l = ja.ring_forward(q.to(dev), [k0.to(dev), k.to(dev)], [v0.to(dev), v.to(dev)], scale)
    full_o, full_l = oa.core_forward(q.double(), torch.cat([k0, k], 2).double(), torch.cat([v0, v], 2).double(), scale)
    assert rel_l2(ring_o, full_o) < 2e-2 and rel_l2(ring_l, full_l) < 2e-3


def test_config4_shape_properties(dev):
    """Config 4 at full size: 8 heads, 4096 queries, 4 chunks of 4096 keys, d = 64, bf16.
    Size-independent checks: ring over 4 chunks == one core call over the concatenated
    K/V; permuting the chunks changes nothing beyond rounding; 128 sampled query rows
    match the fp64 oracle over all 16384 keys."""
    torch.manual_seed(3)
    b, h, n, d, P = 1, 8, 4096, 64, 4
    scale = d**-0.5
    q = (torch.randn(b, h, n, d, device=dev) / 8).bfloat16()
    ks = [torch.randn(b, h, n, d, device=dev).bfloat16() for _ in range(P)]
    vs = [torch.randn(b, h, n, d, device=dev).bfloat16() for _ in range(P)]
    out, lse = ja.ring_forward(q, ks, vs, scale, rank=1)
    full_o, full_l = ja.core_forward(q, torch.cat(ks, 2), torch.cat(vs, 2), scale)
    assert rel_l2(out, full_o) < 1e-2
    assert rel_l2(lse, full_l) < 1e-5
    out2, lse2 = ja.ring_forward(q, ks[::-1], vs[::-1], scale, rank=0)
    assert rel_l2(out2, out) < 1e-2 and rel_l2(lse2, lse) < 1e-5
    rows = torch.arange(0, n, 32)
    qs = q[:, :, rows].double().cpu()
    K, V = torch.cat(ks, 2).double().cpu(), torch.cat(vs, 2).double().cpu()
    s = (qs @ K.mT) * scale
    want = torch.softmax(s, -1) @ V
    assert rel_l2(out[:, :, rows], want) < 2e-2
    assert rel_l2(lse[:, :, rows], torch.logsumexp(s, -1)) < 1e-4


def test_config4_shape_in_fp32_on_the_matrix_cores(dev):
    """Config 4's ring at full size with fp32 inputs (8 heads, 4096 queries, 4 chunks of 4096 keys, d = 64):
    ring of fused steps == one core call over the concatenated K/V, forward and backward; sampled
    rows against fp64; and the bf16 kernels' result within bf16's tolerance of it."""
    torch.manual_seed(6)
    b, h, n, d, P = 1, 8, 4096, 64, 4
    scale = d**-0.5
    q = torch.randn(b, h, n, d, device=dev) / 8
    ks = [torch.randn(b, h, n, d, device=dev) for _ in range(P)]
    vs = [torch.randn(b, h, n, d, device=dev) for _ in range(P)]
    dout = torch.randn(b, h, n, d, device=dev)
    Kc, Vc = torch.cat(ks, 2), torch.cat(vs, 2)
    out, lse = ja.ring_forward(q, ks, vs, scale, rank=1)
    full_o, full_l = ja.core_forward(q, Kc, Vc, scale)
    assert out.dtype == torch.float32 and rel_l2(out, full_o) < 1e-5 and rel_l2(lse, full_l) < 1e-6
    rows = torch.arange(5, n, 64)
    qs = q[:, :, rows].double().cpu()
    s = (qs @ Kc.double().cpu().mT) * scale
    assert rel_l2(out[:, :, rows], torch.softmax(s, -1) @ Vc.double().cpu()) < 1e-5
    assert rel_l2(lse[:, :, rows], torch.logsumexp(s, -1)) < 1e-6
    o16, l16 = ja.ring_forward(q.bfloat16(), [t.bfloat16() for t in ks], [t.bfloat16() for t in vs], scale, rank=1)
    assert rel_l2(o16, out) < 2e-2 and rel_l2(l16, lse) < 1e-3

    dq, dks, dvs = ja.ring_backward(dout, q, out, lse, ks, vs, scale)
    fdq, fdk, fdv = ja.core_backward(dout, q, Kc, Vc, out, lse, scale)
    assert rel_l2(dq, fdq) < 1e-5 and rel_l2(torch.cat(dks, 2), fdk) < 1e-5 and rel_l2(torch.cat(dvs, 2), fdv) < 1e-5
    # sampled keys of one chunk against fp64 (every query takes part)
    keys = torch.arange(3, n, 128)
    Q, O, dO, L = q.double().cpu(), out.double().cpu(), dout.double().cpu(), lse.double().cpu()
    Kj, Vj = ks[2][:, :, keys].double().cpu(), vs[2][:, :, keys].double().cpu()
    p = torch.exp((Q @ Kj.mT) * scale - L.unsqueeze(-1))
    delta = (dO * O).sum(-1, keepdim=True)
    ds = p * (dO @ Vj.mT - delta) * scale
    assert rel_l2(dvs[2][:, :, keys], p.mT @ dO) < 1e-5
    assert rel_l2(dks[2][:, :, keys], ds.mT @ Q) < 1e-5


def test_config4_backward_shape_properties(dev):
    """Config 4 backward at full size (8 heads, 4096 queries, 4 chunks of 4096 keys, d = 64,
    bf16), from the GLOBAL out / lse as the ring holds them (backward.py:176-270).
    Size-independent checks against fp64 on samples: the rows of ``sum_j dq_j`` for 128
    sampled queries (each needs all 16384 keys), and the rows of ``dk_j`` / ``dv_j`` for 128
    sampled keys of every chunk (each needs all 4096 queries); plus ``sum_j dq_j`` == dq of
    one core call over the concatenated K/V."""
    torch.manual_seed(5)
    b, h, n, d, P = 1, 8, 4096, 64, 4
    scale = d**-0.5
    q = (torch.randn(b, h, n, d, device=dev) / 8).bfloat16()
    ks = [torch.randn(b, h, n, d, device=dev).bfloat16() for _ in range(P)]
    vs = [torch.randn(b, h, n, d, device=dev).bfloat16() for _ in range(P)]
    dout = torch.randn(b, h, n, d, device=dev).bfloat16()
    out, lse = ja.ring_forward(q, ks, vs, scale, rank=0)
    dq, dks, dvs = ja.ring_backward(dout, q, out, lse, ks, vs, scale)
    assert dq.dtype == torch.bfloat16 and len(dks) == P and len(dvs) == P

    Kc, Vc = torch.cat(ks, 2), torch.cat(vs, 2)
    dq_full, dk_full, dv_full = ja.backward(dout, q, Kc, Vc, out, lse, scale, n, P * n)
    assert rel_l2(dq, dq_full) < 1e-2
    assert rel_l2(torch.cat(dks, 2), dk_full) < 1e-2 and rel_l2(torch.cat(dvs, 2), dv_full) < 1e-2

    # fp64 on the host from the same bf16 inputs and the same (rounded) global out / lse
    Q, K, V = q.double().cpu(), Kc.double().cpu(), Vc.double().cpu()
    dO, O, L = dout.double().cpu(), out.double().cpu(), lse.double().cpu()
    D = (dO * O).sum(-1)  # (b, h, n)
    rows = torch.arange(5, n, 32)
    s = (Q[:, :, rows] @ K.mT) * scale
    p = torch.exp(s - L[:, :, rows, None])
    dp = dO[:, :, rows] @ V.mT
    ds = p * (dp - D[:, :, rows, None]) * scale
    assert rel_l2(dq[:, :, rows], ds @ K) < 2e-2, f"dq rows {rel_l2(dq[:, :, rows], ds @ K):.3e}"
    keys = torch.arange(3, n, 32)
    for j in range(P):
        kj, vj = K[:, :, j * n + keys], V[:, :, j * n + keys]
        s = (Q @ kj.mT) * scale  # (b, h, n, 128)
        p = torch.exp(s - L[..., None])
        want_dv = p.mT @ dO
        ds = p * (dO @ vj.mT - D[..., None]) * scale
        want_dk = ds.mT @ Q
        assert rel_l2(dvs[j][:, :, keys], want_dv) < 2e-2, f"dv chunk {j}: {rel_l2(dvs[j][:, :, keys], want_dv):.3e}"
        assert rel_l2(dks[j][:, :, keys], want_dk) < 2e-2, f"dk chunk {j}: {rel_l2(dks[j][:, :, keys], want_dk):.3e}"


@pytest.mark.parametrize("b,h,n,nk,P", [(1, 2, 256, 128, 3), (2, 3, 128, 384, 1), (1, 8, 512, 256, 5), (1, 1, 128, 128, 16)])
def test_backward_over_resident_chunks_in_one_pass(b, h, n, nk, P, dev):
    """``backward_chunks`` (one dQ launch over all chunks, the chunk as a grid dimension of the dK/dV
    kernel): dK / dV of every chunk have the bits of the per-chunk ``core_backward`` (same kernel, same
    arithmetic per chunk), dQ is the fp32 sum of the chunks rounded once, checked against fp64
    (backward.py:176-277 visits chunk s at step s and adds the steps' dq)."""
    torch.manual_seed(11)
    d = 64
    scale = d**-0.5
    q = (torch.randn(b, h, n, d, device=dev) / 4).bfloat16()
    ks = [torch.randn(b, h, nk, d, device=dev).bfloat16() for _ in range(P)]
    vs = [torch.randn(b, h, nk, d, device=dev).bfloat16() for _ in range(P)]
    dout = torch.randn(b, h, n, d, device=dev).bfloat16()
    out, lse = ja.ring_forward(q, ks, vs, scale, rank=0)
    res = ja.backward_chunks(dout, q, out, lse, ks, vs, scale)
    assert res is not None, "bf16 at head size 64 with lengths in multiples of 128 is what the one-pass kernels cover"
    dq, dks, dvs = res
    want_dq = torch.zeros(q.shape, dtype=torch.float64)
    for j in range(P):
        dq_j, dk_j, dv_j = ja.core_backward(dout, q, ks[j], vs[j], out, lse, scale)
        assert torch.equal(dks[j], dk_j) and torch.equal(dvs[j], dv_j), f"chunk {j}"
        ref = oa.core_backward(dout.double().cpu(), q.double().cpu(), ks[j].double().cpu(), vs[j].double().cpu(),
                                        out.double().cpu(), lse.double().cpu(), scale)
        want_dq += ref[0]
        assert rel_l2(dk_j, ref[1]) < 2e-2 and rel_l2(dv_j, ref[2]) < 2e-2
    assert rel_l2(dq, want_dq) < 2e-2, f"dq {rel_l2(dq, want_dq):.3e}"
    # and through ring_backward, which takes this route by itself
    dq2, dks2, dvs2 = ja.ring_backward(dout, q, out, lse, ks, vs, scale)
    assert torch.equal(dq2, dq) and all(torch.equal(a, c) for a, c in zip(dks2, dks))


def test_backward_over_chunks_declines_what_it_does_not_cover(dev):
    q = torch.randn(1, 1, 128, 64, device=dev)
    k = [torch.randn(1, 1, 128, 64, device=dev)]
    assert ja.backward_chunks(q, q, q, q[..., 0], k, k, 0.125) is None  # fp32
    qb = q.bfloat16()
    kb = [torch.randn(1, 1, 96, 64, device=dev).bfloat16()]
    assert ja.backward_chunks(qb, qb, qb, q[..., 0], kb, kb, 0.125) is None  # 96 keys
    many = [torch.randn(1, 1, 128, 64, device=dev).bfloat16() for _ in range(17)]
    assert ja.backward_chunks(qb, qb, qb, q[..., 0], many, many, 0.125) is None  # more chunks than a call takes


@pytest.mark.parametrize("d,n,nk", [(64, 192, 160), (32, 100, 70), (128, 64, 96)])
def test_fp32_ring_step_takes_the_fused_merge(d, n, nk, dev):
    """``attend_step_`` on fp32 tensors at the head sizes of the fp32 matrix-core kernel: one launch that merges in
    its epilogue, against the core followed by the separate merge (forward.py:64-96) and the fp64 oracle."""
    torch.manual_seed(3)
    scale = d**-0.5
    q = torch.randn(1, 2, n, d, device=dev)
    ks = [torch.randn(1, 2, nk, d, device=dev) for _ in range(3)]
    vs = [torch.randn(1, 2, nk, d, device=dev) for _ in range(3)]
    assert ja._fused_ok(q, ks[0])
    out = torch.zeros_like(q)
    lse = torch.full(q.shape[:-1], float("-inf"), device=dev)
    out2, lse2 = out.clone(), lse.clone()
    for kj, vj in zip(ks, vs):
        out, lse = ja.attend_step_(q, kj, vj, scale, out, lse)
        o_j, l_j = ja.core_forward(q, kj, vj, scale)
        out2, lse2 = ja.fused_online_softmax_merge_(out2, lse2, o_j, l_j, "bhsd")
    want_o, want_l = oa.ring_forward(q.double().cpu(), [t.double().cpu() for t in ks], [t.double().cpu() for t in vs], scale)
    assert rel_l2(out, want_o) < 1e-5 and rel_l2(lse, want_l) < 1e-5
    assert rel_l2(out, out2) < 1e-6 and rel_l2(lse, lse2) < 1e-6


def test_window_attention_with_bias_and_mask(dev):
    """Swin-style windows: (B, nW, heads, N, d) with a (nW, heads, N, N) bias that
    holds -inf entries (shift mask), forward and backward incl. the bias gradient."""
    torch.manual_seed(4)
    B, nW, heads, N, d = 2, 6, 4, 64, 32
    q, k, v = (torch.randn(B, nW, heads, N, d) for _ in range(3))
    bias = torch.randn(nW, heads, N, N) * 0.5
    mask = torch.zeros(nW, 1, N, N)
    mask[1, :, :32, 32:] = float("-inf")
    mask[1, :, 32:, :32] = float("-inf")
    bias = bias + mask
    qd, kd, vd = (t.double().requires_grad_() for t in (q, k, v))
    bd = bias.double().requires_grad_()
    want = oa.window_attention(qd, kd, vd, bd)
    g = torch.randn_like(want)
    want.backward(g)
    qg, kg, vg, bg = (t.to(dev).requires_grad_() for t in (q, k, v, bias))
    out = ja.window_attention(qg, kg, vg, bg)
    assert rel_l2(out, want.detach()) < 1e-5
    out.backward(g.float().to(dev))
    assert rel_l2(qg.grad, qd.grad) < 1e-5 and rel_l2(kg.grad, kd.grad) < 1e-5 and rel_l2(vg.grad, vd.grad) < 1e-5
    assert rel_l2(bg.grad, torch.nan_to_num(bd.grad)) < 1e-5
    # broadcast bias (heads, N, N), bf16 inputs
    out_b = ja.window_attention(qg.detach().bfloat16(), kg.detach().bfloat16(), vg.detach().bfloat16(), bg.detach()[0])
    want_b = oa.window_attention(q.bfloat16().double(), k.bfloat16().double(), v.bfloat16().double(), bias[0].double())
    assert rel_l2(out_b, want_b) < 2e-2


@pytest.mark.parametrize("with_bias", [True, False])
def test_window_kernels_bf16(with_bias, dev):
    """64-token windows, head size 32, bf16: the dedicated window kernels (one wavefront
    per window and head), forward and backward with the bias gradient, against the
    oracle in fp64 on the same bf16 inputs. 15 entries: the last workgroup is ragged."""
    torch.manual_seed(11)
    B, nW, heads, N, d = 1, 5, 3, 64, 32
    q, k, v = (torch.randn(B, nW, heads, N, d).bfloat16() for _ in range(3))
    bias = None
    if with_bias:
        bias = torch.randn(nW, heads, N, N) * 0.5
        bias[2, :, :24, 24:] = float("-inf")
        bias[2, :, 24:, :24] = float("-inf")
    qd, kd, vd = (t.double().requires_grad_() for t in (q, k, v))
    bd = bias.double().requires_grad_() if with_bias else None
    want = oa.window_attention(qd, kd, vd, bd if with_bias else torch.zeros(N, N, dtype=torch.float64))
    g = torch.randn_like(want).bfloat16()
    want.backward(g.double())
    qg, kg, vg = (t.to(dev).requires_grad_() for t in (q, k, v))
    bg = bias.to(dev).requires_grad_() if with_bias else None
    out = ja.window_attention(qg, kg, vg, bg)
    assert out.dtype == torch.bfloat16
    assert rel_l2(out, want.detach()) < 2e-2
    out.backward(g.to(dev))
    assert rel_l2(qg.grad, qd.grad) < 2e-2 and rel_l2(kg.grad, kd.grad) < 2e-2 and rel_l2(vg.grad, vd.grad) < 2e-2
    if with_bias:
        assert rel_l2(bg.grad, torch.nan_to_num(bd.grad)) < 2e-2
        assert (bg.grad[2, :, :24, 24:] == 0).all()
    # lse of the same call through the core interface
    out2, lse = ja.core_forward(qg.detach(), kg.detach(), vg.detach(), d ** -0.5, bias=bg.detach() if with_bias else None)
    s = torch.einsum("bwhqd,bwhkd->bwhqk", q.double(), k.double()) * d ** -0.5
    if with_bias:
        s = s + bias.double()
    assert rel_l2(lse, torch.logsumexp(s, -1)) < 1e-4
    assert torch.equal(out2, out.detach())


def test_core_argument_errors(dev):
    q = torch.zeros(1, 2, 8, 16, device=dev)
    with pytest.raises(NotImplementedError):
        ja.forward(q, q, q, 0.25, 0.0, layout="bshd")
    with pytest.raises(NotImplementedError):
        ja.forward(q, q, q, 0.25, 0.1)
    with pytest.raises(RuntimeError):
        ja.forward(q, q.bfloat16(), q, 0.25)
    with pytest.raises(ValueError):
        ja.forward(q, q[:, :1], q, 0.25)
    wide = torch.zeros(1, 2, 8, 136, device=dev)  # beyond the largest head size the kernels are built for
    with pytest.raises(NotImplementedError):
        ja.forward(wide, wide, wide, 0.25)


@pytest.mark.parametrize("d", [5, 40, 72])
def test_head_sizes_between_the_kernel_sizes_are_zero_padded(d, dev):
    q, k, v = _qkv(1, 2, 33, 47, d, torch.float32)
    scale = d**-0.5
    want_o, want_l = oa.core_forward(q.double(), k.double(), v.double(), scale)
    out, lse, _ = ja.forward(q.to(dev), k.to(dev), v.to(dev), scale)
    assert out.shape == q.shape and rel_l2(out, want_o) < 1e-5 and rel_l2(lse, want_l) < 1e-5
    dout = torch.randn(1, 2, 33, d)
    want = oa.core_backward(dout.double(), q.double(), k.double(), v.double(), want_o, want_l, scale)
    got = ja.backward(dout.to(dev), q.to(dev), k.to(dev), v.to(dev), want_o.float().to(dev), want_l.float().to(dev), scale, 33, 47)
    for g, w in zip(got, want):
        assert g.shape == w.shape and rel_l2(g, w) < 1e-5
