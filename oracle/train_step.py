"""Oracle for one training step of the reference's CPU-runnable configuration: the
two-layer halo-convolution model ``DistributedConv2d(3 -> 16, k3, pad 1) -> GELU ->
DistributedConv2d(16 -> 3, k3, pad 1)`` on a 2 x 2 spatial mesh of ``gloo`` ranks, MSE
loss, Adam (lr 1e-3), fp32 (README quick-start model inside the loop of
examples/domain_parallel.py:109-160). Test infrastructure only.

Every rank is a process of its own; what the reference does between ranks is done with
the same collectives:

* halo forward / backward: one uneven ``all_to_all_single`` per split axis, H then W in
  the forward, W then H in the backward, the rank's own span travelling through the
  exchange like everybody else's (_conv/halo.py:66-251, _common/halo.py:7-63);
* weight and bias gradients: SUM all-reduce of ``cat(grads)`` over the H group, then
  the W group (parallel/_sync.py:33-46);
* loss: squared-error sum and element count all-reduced, then divided
  (loss/_regression/functional.py:14-28);
* initial weights: Kaiming-uniform on rank 0 (bound 1/sqrt(fan_in), init.py:115-158),
  broadcast (base.py:223-225); the batch: a GLOBAL tensor seeded by the step, each rank
  keeps its tile (examples/domain_parallel.py:88-106).

``reference_step`` is the same model on the undivided image in plain torch: what the
tiled run must reproduce (the method of tests/test_examples.py:172-217).
"""

from __future__ import annotations

import math
import time

import torch
import torch.distributed as dist
import torch.nn.functional as F

from . import conv as oc
from .halo import needed_input_span

MESH = (2, 2)
K, S, P, D = 3, 1, 1, 1


def _exchange_axis(t, group, rank, size, n_local, axis, gather):
    """One all-to-all along ``axis``. ``gather=True``: every peer gets the rows of this
    rank it needs, the result is the padded span. ``gather=False``: the adjoint."""
    spans = [needed_input_span(r, size, n_local, K, S, P, D) for r in range(size)]
    lo, hi, need, _ = spans[rank]
    moved = t.movedim(axis, 0)
    send, send_sizes, recv_sizes, places = [], [], [], []
    for peer in range(size):
        p_lo, p_hi = spans[peer][0], spans[peer][1]
        if gather:
            # rows of mine inside the peer's span / rows of the peer inside my span
            s0 = max(p_lo, rank * n_local, 0)
            s_cnt = max(min(p_hi, (rank + 1) * n_local, size * n_local) - s0, 0)
            send.append(moved.narrow(0, s0 - rank * n_local, s_cnt))
            r0 = max(lo, peer * n_local, 0)
            r_cnt = max(min(hi, (peer + 1) * n_local, size * n_local) - r0, 0)
            places.append((r0 - lo, r_cnt))
        else:
            # part of my padded gradient that the peer owns / part of the peer's that I own
            s0 = max(lo, peer * n_local, 0)
            s_cnt = max(min(hi, (peer + 1) * n_local, size * n_local) - s0, 0)
            send.append(moved.narrow(0, s0 - lo, s_cnt))
            r0 = max(p_lo, rank * n_local, 0)
            r_cnt = max(min(p_hi, (rank + 1) * n_local, size * n_local) - r0, 0)
            places.append((r0 - rank * n_local, r_cnt))
        send_sizes.append(s_cnt)
        recv_sizes.append(places[-1][1])
    send_cat = torch.cat(send, 0).contiguous()
    recv_cat = send_cat.new_empty((sum(recv_sizes), *send_cat.shape[1:]))
    dist.all_to_all_single(recv_cat, send_cat, recv_sizes, send_sizes, group=group)
    shape = list(moved.shape)
    shape[0] = need if gather else n_local
    out = moved.new_zeros(shape)
    off = 0
    for (start, cnt) in places:
        if cnt:
            if gather:
                out.narrow(0, start, cnt).copy_(recv_cat.narrow(0, off, cnt))
            else:
                out.narrow(0, start, cnt).add_(recv_cat.narrow(0, off, cnt))
        off += cnt
    return out.movedim(0, axis).contiguous()


class _HaloConv(torch.autograd.Function):
    """conv_halo_nway / conv_halo_nway_backward (_conv/distributed.py:212-396) for col = 1."""

    @staticmethod
    def forward(ctx, x, w, b, mesh):
        n_local = x.shape[-2:]
        x_aug = x
        for a, axis in ((0, -2), (1, -1)):
            x_aug = _exchange_axis(x_aug, mesh["groups"][a], mesh["coord"][a], MESH[a], n_local[a], axis, True)
        ctx.save_for_backward(x_aug, w)
        ctx.mesh, ctx.n_local, ctx.has_bias = mesh, n_local, b is not None
        return oc.forward(x_aug, w, b, (S, S), (0, 0), (D, D))

    @staticmethod
    def backward(ctx, g):
        x_aug, w = ctx.saved_tensors
        mesh = ctx.mesh
        gb = oc.grad_bias(g, 2) if ctx.has_bias else None
        gx = oc.dgrad(x_aug.shape, w, g, (S, S), (0, 0), (D, D))
        gw = oc.wgrad(x_aug, w.shape, g, (S, S), (0, 0), (D, D))
        for a, axis in ((1, -1), (0, -2)):
            gx = _exchange_axis(gx, mesh["groups"][a], mesh["coord"][a], MESH[a], ctx.n_local[a], axis, False)
        return gx, gw, gb, None


def _sync_grads(params, mesh):
    flat = torch.cat([p.grad.reshape(-1) for p in params])
    for a in (0, 1):
        dist.all_reduce(flat, op=dist.ReduceOp.SUM, group=mesh["groups"][a])
    off = 0
    for p in params:
        p.grad.copy_(flat[off : off + p.numel()].view_as(p))
        off += p.numel()


def init_params(seed=0):
    """Kaiming-uniform with a = sqrt(5): U(-1/sqrt(fan_in), 1/sqrt(fan_in)); zero biases."""
    g = torch.Generator().manual_seed(seed)

    def ku(*shape):
        fan_in = shape[1] * shape[2] * shape[3]
        return (torch.rand(*shape, generator=g) * 2 - 1) / math.sqrt(fan_in)

    return [ku(16, 3, 3, 3), torch.zeros(16), ku(3, 16, 3, 3), torch.zeros(3)]


def make_batch(step, batch=4, size=512):
    g = torch.Generator().manual_seed(1000 + step)
    return torch.randn(batch, 3, size, size, generator=g), torch.randn(batch, 3, size, size, generator=g)


def make_mesh(rank):
    """Groups of a 2 x 2 mesh, rank = 2 * row + col; every rank creates every group."""
    coord = (rank // 2, rank % 2)
    h_groups = [dist.new_group([c, 2 + c]) for c in range(2)]     # same column: split along H
    w_groups = [dist.new_group([2 * r, 2 * r + 1]) for r in range(2)]  # same row: split along W
    return {"coord": coord, "groups": (h_groups[coord[1]], w_groups[coord[0]])}


def rank_steps(rank, steps, batch=4, size=512, warmup=0):
    """Run ``steps`` training steps on this rank (process group already initialised, world 4).
    Returns ``(losses, seconds per timed step, params)``."""
    mesh = make_mesh(rank)
    params = [p.clone() for p in init_params()]
    for p in params:
        dist.broadcast(p, src=0)
        p.requires_grad_()
    opt = torch.optim.Adam(params, lr=1e-3)
    losses, t0 = [], None
    tile = size // 2
    for step in range(warmup + steps):
        if step == warmup:
            dist.barrier()
            t0 = time.perf_counter()
        x, y = make_batch(step, batch, size)
        r, c = mesh["coord"]
        sl = (slice(None), slice(None), slice(r * tile, (r + 1) * tile), slice(c * tile, (c + 1) * tile))
        x, y = x[sl].contiguous(), y[sl].contiguous()
        h = F.gelu(_HaloConv.apply(x, params[0], params[1], mesh))
        out = _HaloConv.apply(h, params[2], params[3], mesh)
        stats = torch.stack([((out - y) ** 2).sum(), torch.tensor(float(out.numel()))])
        # sum and count reduced, then divided; the graph keeps the local sum
        total = stats.detach().clone()
        dist.all_reduce(total, op=dist.ReduceOp.SUM)
        loss = stats[0] / total[1]
        opt.zero_grad()
        loss.backward()
        _sync_grads(params, mesh)
        opt.step()
        losses.append(float(total[0] / total[1]))
    dist.barrier()
    sec = (time.perf_counter() - t0) / steps
    return losses, sec, [p.detach().clone() for p in params]


def reference_step(steps, batch=4, size=512):
    """The same model on the undivided image, plain torch."""
    params = [p.clone().requires_grad_() for p in init_params()]
    opt = torch.optim.Adam(params, lr=1e-3)
    losses = []
    for step in range(steps):
        x, y = make_batch(step, batch, size)
        out = F.conv2d(F.gelu(F.conv2d(x, params[0], params[1], padding=1)), params[2], params[3], padding=1)
        loss = F.mse_loss(out, y)
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    return losses, [p.detach().clone() for p in params]


def _worker(rank, port, steps, warmup, batch, size, threads, queue):
    torch.set_num_threads(threads)
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank, world_size=4)
    try:
        losses, sec, params = rank_steps(rank, steps, batch, size, warmup)
        queue.put((rank, losses, sec, [p.numpy() for p in params]))
    finally:
        dist.destroy_process_group()


def run_four_ranks(steps=1, warmup=0, batch=4, size=512, threads=1, timeout=300.0):
    """Spawn the four ranks as fresh processes (nothing GPU-related is touched in them) and
    return ``{rank: (losses, seconds per step, params)}``."""
    import socket

    import torch.multiprocessing as mp

    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    ctx = mp.get_context("spawn")
    queue = ctx.Queue()
    procs = [ctx.Process(target=_worker, args=(r, port, steps, warmup, batch, size, threads, queue)) for r in range(4)]
    for p in procs:
        p.start()
    out = {}
    try:
        for _ in range(4):
            rank, losses, sec, params = queue.get(timeout=timeout)
            out[rank] = (losses, sec, [torch.from_numpy(a) for a in params])
    finally:
        for p in procs:
            p.join(timeout=30)
            if p.is_alive():
                p.kill()
    return out
