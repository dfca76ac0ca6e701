"""One rank's seat in a K/V ring: the hops beside the attention core, forward and backward.

What the reference spreads over its chunk providers and the ring loops
(jigsaw/modules/attention/_functional/forward.py:172-199, backward.py:169-312,
forward_chunk_provider.py, backward_chunk_provider.py) is here one object, :class:`RingSeat`,
built once per layer and reused by every pass. It owns what a pass needs besides the
tensors of the caller: the receive slots, the transfer streams and a fixed set of events, so a
pass allocates no stream or event and (with ``save_scope="local"``) no receive buffer.

Schedule of a pass over ``P`` chunks. At step ``s`` the rank holds global chunk
``(rank + s) % P`` (forward_chunk_provider.py:190-192); step 0 reads the caller's own
tensors, step ``s > 0`` receive slot ``s - 1``. A chunk travels as ONE message: K and V of a
slot are the two halves of one ``(2, ...)`` buffer, and the caller's own pair is sent from
where it lies when V follows K in memory (the packed projection output), else from one
packed copy. There are ``P - 1`` slots (memory is not what a 288 GB device is short of), so
within a pass no transfer has to wait for a core to leave a slot. On the host:

1. ``start`` is recorded on the compute stream (behind whatever produced K and V and behind
   every earlier pass), the transfer stream waits for it once, hop 0 is issued and the
   attention core of step 0 is enqueued;
2. the other ``P - 2`` hops are issued on the transfer stream: hop ``s`` sends the chunk of
   step ``s`` (the caller's pair, then slot ``s - 1``: stream order makes it wait for the hop
   that filled it) and receives into slot ``s``, then records ``landed[s]``. The host is done
   with the transfers while step 0 still computes;
3. per later step the compute stream waits for ``landed[s - 1]`` and the core is enqueued
   (fused with the merge into the fp32 accumulator where the kernel covers the shape).

Every cross-stream wait and every change of the current stream costs the host 7-10 us here,
about a fifth of what one core of configuration 4 takes on the GPU: the schedule above needs
one wait per step and one change of stream per pass. Without a transfer stream
(``overlap=False``) the same steps run on the compute stream, the hop for step ``s + 1``
behind the core of step ``s``, and the host waits on the handle the transport returns.

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

from .attention import attend_step_, backward_chunks, core_backward

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
        # slot i holds the chunk of step i + 1, K and V as the halves of one buffer; allocated on first use, then kept
        self._slots: list = [None] * max(self.world - 1, 0)
        if self._wire is not None:
            self._landed = [torch.cuda.Event() for _ in range(self.world - 1)]
            self._start = torch.cuda.Event()
            # the dK/dV partials go to other peers than the K/V hops (other links), on a stream of their own
            self._wire_back = torch.cuda.Stream(device=like.device) if save_scope == "local" else None
            self._ready = [torch.cuda.Event(), torch.cuda.Event()]
            self._arrived = [torch.cuda.Event(), torch.cuda.Event()]

    # ------------------------------------------------------------------ chunk bookkeeping
    def chunk_at(self, step: int) -> int:
        """Global index of the chunk the rank holds at ``step`` while chunks circulate."""
        return (self.rank + step) % self.world

    def _slot(self, i: int, fresh: bool) -> torch.Tensor:
        shape = (2, *self._like.shape)
        if fresh:
            return self._like.new_empty(shape)
        if self._slots[i] is None:
            self._slots[i] = self._like.new_empty(shape)
        return self._slots[i]

    @staticmethod
    def _packed(k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """``(2, ...)`` tensor with ``k`` then ``v``: a view when ``v`` follows ``k`` in memory, else a copy."""
        if (k.is_contiguous() and v.is_contiguous() and v.storage_offset() == k.storage_offset() + k.numel()
                and k.untyped_storage().data_ptr() == v.untyped_storage().data_ptr()):
            return torch.as_strided(k, (2, *k.shape), (k.numel(), *k.stride()))
        return torch.stack((k, v))

    # ------------------------------------------------------------------ the hops
    def _circulate(self, k: torch.Tensor, v: torch.Tensor, keep: bool):
        """Generator over ``(step, k_s, v_s)``; the consumer enqueues its kernels for a step
        and then resumes the generator."""
        P, wire = self.world, self._wire
        if P == 1:
            yield 0, k, v
            return
        held = self._packed(k, v)
        if wire is None:
            ks, vs = k, v
            for s in range(P):
                yield s, ks, vs
                if s + 1 == P:
                    break
                into = self._slot(s, fresh=keep)
                _, work = self._hop(held, into, -1, group=self.group, async_op=True, tag=s)
                if work is not None:
                    work.wait()
                held, ks, vs = into, into[0], into[1]
            return
        compute = torch.cuda.current_stream(self._like.device)
        slots = [self._slot(s, fresh=keep) for s in range(P - 1)]  # allocated while the compute stream is current
        self._start.record(compute)
        wire.wait_event(self._start)

        def issue(first: int, last: int, held: torch.Tensor) -> torch.Tensor:
            torch.cuda.set_stream(wire)  # (a `with torch.cuda.stream` block costs several times as much host time)
            try:
                for s in range(first, last):
                    _, work = self._hop(held, slots[s], -1, group=self.group, async_op=True, tag=s)
                    if work is not None:
                        work.wait()  # a torch.distributed handle makes the CURRENT stream wait, not the host
                    self._landed[s].record(wire)
                    held = slots[s]
            finally:
                torch.cuda.set_stream(compute)
            return held

        held = issue(0, 1, held)  # the first transfer starts before the host turns to the core of step 0
        yield 0, k, v
        issue(1, P - 1, held)
        # No record_stream() on the tensors the transfers touch: the compute stream waits for every
        # `landed` before the pass ends, so whatever it frees or reuses afterwards is ordered behind
        # every access of the transfer stream (and record_stream is slow on the host).
        for s in range(1, P):
            compute.wait_event(self._landed[s - 1])
            yield s, slots[s - 1][0], slots[s - 1][1]

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
            # every chunk is resident: one pass over all of them where the kernels cover it
            one_pass = backward_chunks(dout, q, out, lse, [c[0].to(core) for c in saved], [c[1].to(core) for c in saved], scale)
            if one_pass is not None:
                dq_all, dks, dvs = one_pass
                dk_own = dv_own = None
                for s in range(P):
                    dk_j, dv_j = dks[s], dvs[s]
                    if self._reduce is not None:
                        dk_j, dv_j = self._reduce(dk_j, dv_j, s)
                    if s == self.rank:
                        dk_own, dv_own = dk_j, dv_j
                return dq_all, dk_own, dv_own
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
                wire.wait_event(ready)
                torch.cuda.set_stream(wire)
                try:
                    for src, buf in ((dk_j, r_dk), (dv_j, r_dv)):
                        _, w = self._relay(src, buf, s, group=self.group, async_op=True, step=s)
                        if w is not None:
                            w.wait()
                    arrived.record(wire)
                finally:
                    torch.cuda.set_stream(compute)
                keep_alive.append((dk_j, dv_j))  # read by the transfer stream until `arrived`
                inbox = (r_dk, r_dv, arrived)
        if inbox is not None:
            take(inbox)
        return dq.to(core), dk_own.to(core), dv_own.to(core)


__all__ = ["RingSeat"]
