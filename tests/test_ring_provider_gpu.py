"""One rank's seat in the K/V ring (jigsaw_amd.ring.RingSeat) on one GPU, forward and
backward, against the all-ranks ring oracle (oracle.attention.ring_all_ranks, pinned on
the CPU against autograd of full attention).

Every rank of the ring runs in this process, one after the other. The transports are
stand-ins that copy in what the peer would have sent: the K/V hop knows the global chunk
list; the dK/dV partials of the other ranks come from a first, recording pass (the core is
deterministic, so the second pass sends the same partials again). Tolerances: rel-L2 2e-2
for bf16, 1e-5 for fp32 tensors (the reference's ring tests: atol 1e-2 / 1e-3,
tests/modules/attention/test_ring_attention.py:159-368).
"""

import pytest
import torch

from helpers import rel_l2
from jigsaw_amd import ring as jr
from oracle import attention as oa

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


class _Work:
    def __init__(self, log):
        self.log = log

    def wait(self):
        self.log.append(("wait", torch.cuda.current_stream().cuda_stream))


class Peers:
    """Transport stand-ins of one rank. ``partials[src_rank][step]`` = (dk, dv) that rank sent."""

    def __init__(self, rank, ks, vs, with_work, partials=None, sums=None):
        self.rank, self.ks, self.vs, self.P = rank, ks, vs, len(ks)
        self.with_work, self.partials, self.sums = with_work, partials, sums
        self.log, self.sent = [], {}

    def hop(self, src, buf, direction, *, group, async_op, tag):
        # one message per hop: K and V of a chunk as the two halves of a (2, ...) tensor
        assert direction == -1 and async_op and buf.shape == src.shape and buf.data_ptr() != src.data_ptr()
        assert src.shape[0] == 2 and src.is_contiguous() and buf.is_contiguous()
        here, j = (self.rank + tag) % self.P, (self.rank + tag + 1) % self.P
        assert torch.equal(src[0], self.ks[here]) and torch.equal(src[1], self.vs[here]), \
            "the hop must forward the chunk of the current step"
        buf[0].copy_(self.ks[j])
        buf[1].copy_(self.vs[j])
        self.log.append(("hop", tag, torch.cuda.current_stream().cuda_stream))
        return buf, (_Work(self.log) if self.with_work else None)

    def relay(self, src, buf, offset, *, group, async_op, step):
        assert offset == step and 1 <= step < self.P
        self.sent.setdefault(step, []).append(src.clone())
        which = len(self.sent[step]) - 1  # dk first, then dv
        if self.partials is None:
            buf.zero_()
        else:
            buf.copy_(self.partials[(self.rank - step) % self.P][step][which])
        self.log.append(("relay", step, torch.cuda.current_stream().cuda_stream))
        return buf, (_Work(self.log) if self.with_work else None)

    def reduce(self, dk_j, dv_j, step):
        self.sent[step] = (dk_j.clone(), dv_j.clone())
        if self.sums is None:
            return dk_j, dv_j
        return self.sums[step]


def _inputs(shape, P, dtype, dev):
    b, h, n, d = shape
    mk = lambda scale=1.0: [(torch.randn(b, h, n, d) * scale).to(dtype) for _ in range(P)]  # noqa: E731
    qs, ks, vs, douts = mk(d ** -0.5), mk(), mk(), mk()
    gpu = lambda ts: [t.to(dev) for t in ts]  # noqa: E731
    return (qs, ks, vs, douts), tuple(gpu(t) for t in (qs, ks, vs, douts))


CASES = [
    ((1, 2, 256, 64), 4, torch.bfloat16),    # fused step kernel (head size 64)
    ((1, 2, 128, 128), 3, torch.bfloat16),   # head size 128
    ((2, 3, 40, 16), 4, torch.float32),      # generic kernels + merge kernel
    ((1, 1, 128, 64), 1, torch.bfloat16),    # a ring of one: no transfer at all
]


@pytest.mark.parametrize("overlap", [False, True], ids=["plain", "overlapped"])
@pytest.mark.parametrize("scope", ["global", "local"])
@pytest.mark.parametrize("shape,P,dtype", CASES, ids=["d64", "d128", "fp32", "ring-of-one"])
def test_ring_seat_matches_all_ranks_oracle(shape, P, dtype, scope, overlap, dev):
    torch.manual_seed(7)
    (qs, ks, vs, douts), (gq, gk, gv, gd) = _inputs(shape, P, dtype, dev)
    scale = shape[-1] ** -0.5
    dbl = lambda ts: [t.double() for t in ts]  # noqa: E731
    want = oa.ring_all_ranks(dbl(qs), dbl(ks), dbl(vs), dbl(douts), scale, save_scope=scope)
    tol = TOL[dtype]

    def run(partials=None, sums=None):
        res, peers = [], []
        for r in range(P):
            pr = Peers(r, gk, gv, with_work=not overlap, partials=partials, sums=sums)
            seat = jr.RingSeat(r, P, gk[r], pr.hop if P > 1 else None, relay_fn=pr.relay, reduce_fn=pr.reduce,
                               save_scope=scope, overlap=overlap)
            out, lse, saved = seat.forward(gq[r], gk[r], gv[r], scale)
            # a second forward on the same seat: the slots and events are reused
            pr.log.clear()
            out2, lse2, saved = seat.forward(gq[r], gk[r], gv[r], scale)
            torch.cuda.synchronize()
            assert torch.equal(out, out2) and torch.equal(lse, lse2)
            fwd_log = list(pr.log)
            pr.log.clear()
            dq, dk, dv = seat.backward(gd[r], gq[r], out, lse, scale, saved)
            torch.cuda.synchronize()
            res.append((out, lse, dq, dk, dv))
            peers.append((pr, fwd_log, seat))
        return res, peers

    res, peers = run()
    if scope == "local":
        partials = [{s: tuple(pr.sent[s]) for s in pr.sent} for pr, _, _ in peers]
        res, peers = run(partials=partials)
    else:
        sums = {}
        for s in range(P):
            dk = peers[0][0].sent[s][0].clone()
            dv = peers[0][0].sent[s][1].clone()
            for pr, _, _ in peers[1:]:
                dk += pr.sent[s][0]
                dv += pr.sent[s][1]
            sums[s] = (dk, dv)
        res, peers = run(sums=sums)

    for r in range(P):
        out, lse, dq, dk, dv = res[r]
        assert out.dtype == dtype and lse.dtype == torch.float32 and dq.dtype == dtype and dk.dtype == dtype
        for name, got, w in zip(("out", "lse", "dq", "dk", "dv"), (out, lse, dq, dk, dv), (want[i][r] for i in range(5))):
            bound = tol if name != "lse" else max(tol * 0.05, 1e-5)
            assert rel_l2(got, w) < bound, f"rank {r} {name}: {rel_l2(got, w):.3e}"
        pr, fwd_log, seat = peers[r]
        hops = [e for e in fwd_log if e[0] == "hop"]
        assert [e[1] for e in hops] == list(range(P - 1))  # one message (K and V together) per step but the last
        assert [seat.chunk_at(s) for s in range(P)] == [(r + s) % P for s in range(P)]
        main = torch.cuda.current_stream().cuda_stream
        if overlap and P > 1:
            assert all(e[2] != main for e in hops), "the hops belong on the transfer stream"
            assert not any(e[0] == "wait" for e in fwd_log)
        elif P > 1:
            assert all(e[-1] == main for e in fwd_log)
            assert sum(e[0] == "wait" for e in fwd_log) == P - 1  # the host waited for every handle
        if scope == "local":
            relays = [e for e in pr.log if e[0] == "relay"]
            assert [e[1] for e in relays] == [s for s in range(1, P) for _ in (0, 1)]
            assert len([e for e in pr.log if e[0] == "hop"]) == P - 1  # K/V circulate again in the backward
            if overlap and P > 1:
                assert all(e[2] != main for e in relays)
        else:
            assert not [e for e in pr.log if e[0] in ("hop", "relay")]  # saved chunks: nothing travels but the sums


def test_ring_seat_argument_errors(dev):
    k = torch.zeros(1, 1, 128, 64, device=dev, dtype=torch.bfloat16)
    hop = lambda src, buf, direction, **kw: (buf, None)  # noqa: E731
    with pytest.raises(ValueError):
        jr.RingSeat(2, 2, k, hop)
    with pytest.raises(ValueError):
        jr.RingSeat(0, 2, k, None)
    with pytest.raises(ValueError):
        jr.RingSeat(0, 2, k, hop, save_scope="elsewhere")
    seat = jr.RingSeat(0, 2, k, hop, save_scope="local")
    with pytest.raises(ValueError):
        seat.forward(k, k, k[..., :32], 0.125)
    out, lse, saved = seat.forward(k, k, k, 0.125)
    with pytest.raises(ValueError, match="relay_fn"):
        seat.backward(k, k, out, lse, 0.125, saved)


@pytest.mark.parametrize("overlap", [False, True], ids=["plain", "overlapped"])
def test_own_chunk_is_sent_from_where_it_lies_when_v_follows_k(overlap, dev):
    """K and V that are adjacent in memory (the packed projection output) leave as one message
    without a packed copy; separate tensors are packed once. Results are the same either way,
    and the saved chunks of a pass do not alias the slots the next pass writes."""
    torch.manual_seed(3)
    P, shape = 3, (1, 2, 128, 64)
    q = (torch.randn(shape, device=dev) * 0.125).bfloat16()
    kvs = [torch.randn(2, *shape, device=dev).bfloat16() for _ in range(P)]
    first_src = []

    def hop(src, buf, direction, *, group, async_op, tag):
        if tag == 0:
            first_src.append(src.data_ptr())
        buf.copy_(kvs[tag + 1])
        return buf, None

    seat = jr.RingSeat(0, P, kvs[0][0], hop, save_scope="global", overlap=overlap)
    out_a, lse_a, saved_a = seat.forward(q, kvs[0][0], kvs[0][1], 0.125)  # views of one (2, ...) tensor
    k_sep, v_sep = kvs[0][0].clone(), kvs[0][1].clone()
    out_b, lse_b, saved_b = seat.forward(q, k_sep, v_sep, 0.125)          # two tensors of their own
    torch.cuda.synchronize()
    assert first_src[0] == kvs[0].data_ptr(), "adjacent K / V must be sent in place"
    assert first_src[1] not in (k_sep.data_ptr(), kvs[0].data_ptr()), "separate K / V are packed into one message"
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
    for j in range(P):
        for a, b in zip(saved_a[j], saved_b[j]):
            assert torch.equal(a, b) and (j == 0 or a.data_ptr() != b.data_ptr())
        assert torch.equal(saved_a[j][0], kvs[j][0]) and torch.equal(saved_a[j][1], kvs[j][1])
