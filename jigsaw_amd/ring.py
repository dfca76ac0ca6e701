"""One rank's seat in a K/V ring: the hops beside the attention core, forward and backward.

What the reference spreads over its chunk providers and the ring loops
(jigsaw/modules/attention/_functional/forward.py:172-199, backward.py:169-312,
forward_chunk_provider.py, backward_chunk_provider.py) is here one object, :class:`RingSeat`,
built once per layer and reused by every pass. It owns what a pass needs besides the
tensors of the caller: the receive slots, the transfer streams and a fixed set of events, so a
pass allocates no stream or event and (with ``save_scope="local"``) no receive buffer.

Schedule of a pass over ``P`` chunks. At step ``s`` the rank holds global chunk
``(rank + s) % P`` (forward_chunk_provider.py:190-192) in slot ``s % 2``; step 0 reads the
caller's own tensors. Per step, in this order on the host:

1. the compute stream waits for ``landed[s % 2]`` (the hop that filled the slot);
2. the attention core of step ``s`` is enqueued (fused with the merge into the fp32
   accumulator where the kernel covers the shape);
3. ``idle[s % 2]`` is recorded behind it on the compute stream;
4. the hop for step ``s + 1`` is issued on the transfer stream: it sends the slot the core
   is reading (two readers, no hazard) and receives into slot ``(s + 1) % 2``, which the core
   of step ``s - 1`` may still be reading, so the transfer stream first waits for
   ``idle[(s + 1) % 2]`` -- that one event, not for the compute stream as a whole -- and then
   records ``landed[(s + 1) % 2]`` behind the transfer.

The core is enqueued before the hop is issued, so the host cost of issuing the hop sits
behind a running kernel instead of in front of it, and the transfer of step ``s + 1`` runs
while step ``s`` computes. K and V travel as two messages from the tensors they live in
(no packed copy). Without a transfer stream (``overlap=False``) the same steps run on the
compute stream and the host waits on the handle the transport returns.

The transport is the caller's, with the reference's signatures:

* ``hop_fn(src, buf, direction, *, group, async_op, tag) -> (buf, work or None)`` --
  ``RingAttentionConfig.send_op_fn`` as the forward ring calls it
  (jigsaw/modules/attention/_config.py:250-269): send ``src`` to ``rank + direction``,
  receive into ``buf`` from ``rank - direction``;
* ``relay_fn(src, buf, offset, *, group, async_op, step) -> (buf, work or None)`` --
  ``p2p_fn`` as the backward calls it for the dK/dV partials of re-circulated chunks
  (backward.py:514-538): send to ``rank + offset``, receive from ``rank - offset``;
* ``reduce_fn(dk_j, dv_j, step) -> (dk_j, dv_j)`` -- the per-step SUM all-reduce of the
  default configuration (saved chunks, backward.py:272-277).

With ``torch.distributed`` these are batched isend / irecv pairs and an all-reduce; a
single-GPU harness passes functions that copy in what the peers would have sent.
"""

from __future__ import annotations

from collections.abc import Callable, Sequence
from typing import Any

import torch

from .attention import attend_step_, core_backward

HopFn = Callable[..., "tuple[torch.Tensor, Any]"]


class RingSeat:
    """Rank ``rank`` of a ring of ``world`` ranks; see the module docstring for the schedule.

    ``like`` is a tensor with the shape, dtype and device of one K (or V) chunk.
    ``save_scope`` is ``"global"`` (the forward keeps every chunk for the backward, the
    reference's default with ``SEND_DKV``: per-step ``reduce_fn``) or ``"local"`` (only the
    own chunk is kept; the backward circulates K/V again and relays each step's dK/dV
    partial to the chunk's owner through ``relay_fn``)."""

    def __init__(self, rank: int, world: int, like: torch.Tensor, hop_fn: HopFn | None, *, group: Any = None,
                 relay_fn: HopFn | None = None, reduce_fn: Callable | None = None, save_scope: str = "global",
                 overlap: bool = True) -> None:
        if not 0 <= rank < world:
            raise ValueError(f"rank {rank} outside a ring of {world}")
        if save_scope not in ("global", "local"):
            raise ValueError(f"save_scope must be 'global' or 'local', got {save_scope!r}")
        if world > 1 and hop_fn is None:
            raise ValueError("a ring of more than one rank needs a hop_fn")
        self.rank, self.world, self.group, self.save_scope = int(rank), int(world), group, save_scope
        self._hop, self._relay, self._reduce = hop_fn, relay_fn, reduce_fn
        self._like = like
        on_gpu = like.is_cuda
        self._wire = torch.cuda.Stream(device=like.device) if (overlap and on_gpu and world > 1) else None
        # slot i holds (k, v) of the steps with s % 2 == i; allocated on first use, then kept
        self._slots: list[tuple[torch.Tensor, torch.Tensor] | None] = [None, None]
        if self._wire is not None:
            self._landed = [torch.cuda.Event(), torch.cuda.Event()]
            self._idle = [torch.cuda.Event(), torch.cuda.Event()]
            self._start = torch.cuda.Event()
            # the dK/dV partials go to other peers than the K/V hops (other links), on a stream of their own
            self._wire_back = torch.cuda.Stream(device=like.device) if save_scope == "local" else None
            self._ready = [torch.cuda.Event(), torch.cuda.Event()]
            self._arrived = [torch.cuda.Event(), torch.cuda.Event()]

    # ------------------------------------------------------------------ chunk bookkeeping
    def chunk_at(self, step: int) -> int:
        """Global index of the chunk the rank holds at ``step`` while chunks circulate."""
        return (self.rank + step) % self.world

    def _slot(self, i: int, fresh: bool) -> tuple[torch.Tensor, torch.Tensor]:
        if fresh:
            return torch.empty_like(self._like), torch.empty_like(self._like)
        if self._slots[i] is None:
            self._slots[i] = (torch.empty_like(self._like), torch.empty_like(self._like))
        return self._slots[i]

    # ------------------------------------------------------------------ the hop
    def _issue_hop(self, held: tuple, into: tuple, step: int) -> Any:
        """Send ``held`` towards ``rank - 1`` and receive the chunk of ``step + 1`` into ``into``."""
        works = []
        for src, buf in zip(held, into):
            _, work = self._hop(src, buf, -1, group=self.group, async_op=True, tag=step)
            if work is not None:
                works.append(work)
        return works

    def _circulate(self, k: torch.Tensor, v: torch.Tensor, keep: bool):
        """Generator over ``(step, k_s, v_s)``; the consumer enqueues its kernels for a step
        and then resumes the generator, which issues the hop for the next step behind them."""
        P, wire = self.world, self._wire
        held = (k, v)
        if wire is not None:
            compute = torch.cuda.current_stream(self._like.device)
            # the transfers come behind whatever produced k and v and behind every earlier pass
            self._start.record(compute)
            wire.wait_event(self._start)
        pending: list = []
        for s in range(P):
            if s > 0:
                if wire is not None:
                    compute.wait_event(self._landed[s % 2])
                else:
                    for w in pending:
                        w.wait()
            yield s, held[0], held[1]
            if s + 1 == P:
                break
            into = self._slot((s + 1) % 2, fresh=keep)
            if wire is None:
                pending = self._issue_hop(held, into, s)
            else:
                self._idle[s % 2].record(compute)
                if s >= 1 and not keep:
                    wire.wait_event(self._idle[(s + 1) % 2])  # the core of step s - 1 has left that slot
                with torch.cuda.stream(wire):
                    for w in self._issue_hop(held, into, s):
                        w.wait()  # a torch.distributed handle makes the CURRENT stream wait, not the host
                    self._landed[(s + 1) % 2].record(wire)
                # No record_stream() on the tensors the transfer touched: the compute stream waits for
                # `landed` before the pass ends, so whatever it frees or reuses afterwards is ordered
                # behind every access of the transfer stream (and record_stream is slow on the host).
            held = into

    # ------------------------------------------------------------------ forward
    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float):
        """``(out, lse, saved)``: the loop of ``ring_forward`` (forward.py:160-199) with the hops
        beside it. ``out`` in ``q.dtype`` (fp32 accumulator, cast once), ``lse`` fp32.
        ``saved`` is what :meth:`backward` wants back: every chunk by global index
        (``save_scope="global"``) or the own chunk only."""
        if k.shape != v.shape or k.dtype != v.dtype or k.shape != self._like.shape:
            raise ValueError("k and v must have the shape and dtype this seat was built for")
        acc = torch.promote_types(q.dtype, torch.float32)
        out = torch.zeros(q.shape, device=q.device, dtype=acc)
        lse = torch.full(q.shape[:-1], float("-inf"), device=q.device, dtype=acc)
        keep = self.save_scope == "global"
        chunks: list = [None] * self.world
        for s, ks, vs in self._circulate(k.contiguous(), v.contiguous(), keep):
            out, lse = attend_step_(q, ks.to(q.dtype), vs.to(q.dtype), scale, out, lse)
            if keep:
                chunks[self.chunk_at(s)] = (ks, vs)
        return out.to(q.dtype), lse, (chunks if keep else [(k, v)])

    # ------------------------------------------------------------------ backward
    def backward(self, dout: torch.Tensor, q: torch.Tensor, out: torch.Tensor, lse: torch.Tensor, scale: float,
                 saved: Sequence):
        """``(dq, dk, dv)`` of this rank: the loop of ``ring_backward`` (backward.py:169-312)
        from the GLOBAL ``out`` / ``lse``. ``dq`` is summed over the chunks in fp32 and cast
        to ``q.dtype`` once (the reference adds in ``q.dtype``, backward.py:184, 269). dK/dV:

        * ``"global"``: step ``s`` takes saved chunk ``s`` (backward.py:97-98); ``reduce_fn``
          sums its partial over the ranks and the owner (``rank == s``) keeps the sum;
        * ``"local"``: K/V circulate as in the forward; the partial of step ``s`` belongs to
          rank ``rank + s`` and goes there through ``relay_fn`` with offset ``s``, while the
          partial for the own chunk arrives from ``rank - s``; the owner adds them in step
          order to its own step-0 partial (backward.py:484-538). The relay of step ``s`` is
          issued behind the core of step ``s`` and its sum is taken one step later, so the
          transfer runs under the core of step ``s + 1``."""
        core = q.dtype
        dout, out = dout.to(core), out.to(core)
        dq = torch.zeros(q.shape, device=q.device, dtype=torch.float32)
        P = self.world
        if self.save_scope == "global":
            if len(saved) != P:
                raise ValueError(f"expected the {P} chunks the forward saved, got {len(saved)}")
            dk_own = dv_own = None
            for s, (ks, vs) in enumerate(saved):
                dq_j, dk_j, dv_j = core_backward(dout, q, ks.to(core), vs.to(core), out, lse, scale)
                dq += dq_j
                if self._reduce is not None:
                    dk_j, dv_j = self._reduce(dk_j, dv_j, s)
                if s == self.rank:
                    dk_own, dv_own = dk_j, dv_j
            return dq.to(core), dk_own, dv_own

        (k, v), = saved
        if P > 1 and self._relay is None:
            raise ValueError("save_scope='local' relays the dK/dV partials: pass relay_fn")
        dk_own = dv_own = None
        inbox: tuple | None = None  # (recv_dk, recv_dv, works or event) of the previous step's relay
        keep_alive: list = []       # partials a transfer may still be reading; dropped after the last `arrived` wait
        wire = self._wire_back if self._wire is not None else None
        if wire is not None:
            compute = torch.cuda.current_stream(q.device)

        def take(box):
            nonlocal dk_own, dv_own
            r_dk, r_dv, handle = box
            if wire is not None:
                compute.wait_event(handle)
            else:
                for w in handle:
                    w.wait()
            dk_own += r_dk
            dv_own += r_dv

        for s, ks, vs in self._circulate(k.contiguous(), v.contiguous(), keep=False):
            dq_j, dk_j, dv_j = core_backward(dout, q, ks.to(core), vs.to(core), out, lse, scale)
            dq += dq_j
            if inbox is not None:  # behind this step's core: its transfer ran under it
                take(inbox)
                inbox = None
            if s == 0:
                dk_own, dv_own = dk_j.float(), dv_j.float()
                continue
            r_dk, r_dv = torch.empty_like(dk_j), torch.empty_like(dv_j)
            if wire is None:
                works = [w for src, buf in ((dk_j, r_dk), (dv_j, r_dv))
                         for w in [self._relay(src, buf, s, group=self.group, async_op=True, step=s)[1]] if w is not None]
                inbox = (r_dk, r_dv, works)
            else:
                ready, arrived = self._ready[s % 2], self._arrived[s % 2]
                ready.record(compute)
                with torch.cuda.stream(wire):
                    wire.wait_event(ready)
                    for src, buf in ((dk_j, r_dk), (dv_j, r_dv)):
                        _, w = self._relay(src, buf, s, group=self.group, async_op=True, step=s)
                        if w is not None:
                            w.wait()
                    arrived.record(wire)
                keep_alive.append((dk_j, dv_j))  # read by the transfer stream until `arrived`
                inbox = (r_dk, r_dv, arrived)
        if inbox is not None:
            take(inbox)
        return dq.to(core), dk_own.to(core), dv_own.to(core)


__all__ = ["RingSeat"]
