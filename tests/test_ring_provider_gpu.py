"""Chunk providers of the ring (the K/V hop beside the attention core) on one GPU: the
neighbour's transfer is a device copy of the chunk it would have sent. The provider loop
must visit the chunks in ring order and give exactly what the loop over the chunk list gives
(same kernels, same order: bit-identical), with the hop on the compute thread or on a side
stream."""

import pytest
import torch

from jigsaw_amd import attention as ja
from jigsaw_amd import ring as jr

pytestmark = pytest.mark.gpu


class _Work:
    def __init__(self, log):
        self.log = log

    def wait(self):
        self.log.append("wait")


def _neighbour(ks, vs, rank, log, with_work):
    """send_op_fn of rank ``rank``: what arrives at step tag + 1 is global chunk rank + tag + 1."""
    P = len(ks)

    def send(src, buf, *, direction, group, async_op, tag):
        assert direction == -1 and async_op and buf.shape == src.shape
        j = (rank + tag + 1) % P
        buf.copy_(torch.stack((ks[j], vs[j])))
        log.append(("send", tag, torch.cuda.current_stream().cuda_stream))
        return buf, (_Work(log) if with_work else None)

    return send


@pytest.mark.parametrize("overlap", [False, True], ids=["plain", "side-stream"])
@pytest.mark.parametrize("shape,P,dtype", [
    ((1, 2, 256, 64), 4, torch.bfloat16),    # fused step kernel
    ((1, 2, 128, 128), 3, torch.bfloat16),   # head size 128
    ((2, 3, 40, 16), 4, torch.float32),      # generic kernels + merge kernel
    ((1, 1, 128, 64), 1, torch.bfloat16),    # a ring of one: no transfer at all
])
def test_provider_ring_equals_chunk_list_ring(shape, P, dtype, overlap, dev):
    torch.manual_seed(7)
    b, h, n, d = shape
    scale = d ** -0.5
    q = (torch.randn(b, h, n, d) / d ** 0.5).to(dtype).to(dev)
    ks = [torch.randn(b, h, n, d).to(dtype).to(dev) for _ in range(P)]
    vs = [torch.randn(b, h, n, d).to(dtype).to(dev) for _ in range(P)]
    side = torch.cuda.Stream() if overlap else None
    for rank in range(P):
        log = []
        prov = jr.RingKVProvider(ks[rank], vs[rank], rank, P, _neighbour(ks, vs, rank, log, with_work=not overlap),
                                 comm_stream=side)
        out, lse = jr.ring_forward_from_provider(q, prov, scale)
        want_o, want_l = ja.ring_forward(q, ks, vs, scale, rank=rank)
        torch.cuda.synchronize()
        assert torch.equal(out, want_o) and torch.equal(lse, want_l)
        sends = [e for e in log if e != "wait"]
        assert [e[1] for e in sends] == list(range(P - 1))          # one hop per step but the last
        assert [prov.global_chunk_idx(s) for s in range(P)] == [(rank + s) % P for s in range(P)]
        if overlap:
            assert all(e[2] == side.cuda_stream for e in sends)     # every hop was issued on the side stream
        else:
            assert log.count("wait") == P - 1                       # the host waited for every handle


def test_provider_argument_errors(dev):
    k = torch.zeros(1, 1, 128, 64, device=dev, dtype=torch.bfloat16)
    send = lambda *a, **kw: (a[1], None)  # noqa: E731
    with pytest.raises(ValueError):
        jr.RingKVProvider(k, k[..., :32], 0, 2, send)
    with pytest.raises(ValueError):
        jr.RingKVProvider(k, k, 2, 2, send)
    prov = jr.RingKVProvider(k, k, 0, 2, send)
    with pytest.raises(ValueError):
        prov.get(1)  # step 0 first


def test_provider_ring_in_fp16_with_the_fused_step(dev):
    """fp16 at head size 128 runs the fused step kernel; the provider loop still equals the list loop."""
    torch.manual_seed(8)
    P, shape = 3, (1, 2, 128, 128)
    q = (torch.randn(*shape) / 128 ** 0.5).half().to(dev)
    ks = [torch.randn(*shape).half().to(dev) for _ in range(P)]
    vs = [torch.randn(*shape).half().to(dev) for _ in range(P)]
    side = torch.cuda.Stream()
    prov = jr.RingKVProvider(ks[1], vs[1], 1, P, _neighbour(ks, vs, 1, [], with_work=False), comm_stream=side)
    out, lse = jr.ring_forward_from_provider(q, prov, 128 ** -0.5)
    want_o, want_l = ja.ring_forward(q, ks, vs, 128 ** -0.5, rank=1)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and torch.equal(out, want_o) and torch.equal(lse, want_l)
