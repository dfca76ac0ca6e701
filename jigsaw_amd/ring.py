"""The K/V hop of ring attention beside the attention core: chunk providers.

Host-side mirror of the forward chunk providers of the plain ring that circulates the
packed K/V tensor (``_RingForwardChunkProvider`` and its overlap variant,
jigsaw/modules/attention/_functional/forward_chunk_provider.py:147-244) and of the
side-stream helpers they use (``_comm_overlap.py:21-79``). A provider hands the ring loop
the chunk of step ``s`` -- the global chunk ``(rank + s) % P`` -- and meanwhile has the chunk
of step ``s + 1`` on its way:

* plain: the transfer is issued on the compute stream's thread and its ``work`` handle is
  waited for on the host before the chunk is used;
* overlapped: the transfer is issued on a side stream that first waits for the compute
  stream (the source must be complete), the compute stream later waits for an event
  recorded behind the transfer, and two receive buffers alternate, so the hop of step
  ``s + 1`` runs while the core of step ``s`` computes.

The transfer itself is the caller's: ``send_op_fn(src, buf, direction=-1, group=...,
async_op=True, tag=step) -> (buf, work or None)``, the signature of the reference's
``config.send_op_fn`` (forward_chunk_provider.py:222-229). With ``torch.distributed`` it
is a batched isend / irecv to the ring neighbours; a single-GPU harness passes a device
copy of the chunk the neighbour would have sent.
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch

from .attention import attend_step_

SendOp = Callable[..., "tuple[torch.Tensor, Any]"]


def issue_on_comm_stream(comm_stream: torch.cuda.Stream, produce: Callable[[], tuple], keep_alive: tuple = ()):
    """Run ``produce() -> (recv_buf, work)`` on ``comm_stream`` once the compute stream's work so
    far is done; returns ``(recv_buf, work, event)`` with the event recorded behind the transfer
    (_comm_overlap.py:21-63). ``work.wait()`` is called under the side stream, so for a
    ``torch.distributed`` handle it is that stream, not the host, that waits."""
    compute = torch.cuda.current_stream()
    comm_stream.wait_stream(compute)
    with torch.cuda.stream(comm_stream):
        recv_buf, work = produce()
        if work is not None:
            work.wait()
    for t in keep_alive:
        t.record_stream(comm_stream)  # the caching allocator must not hand the memory out while the transfer runs
    event = torch.cuda.Event()
    event.record(comm_stream)
    return recv_buf, work, event


def consume(event: torch.cuda.Event, *bufs: torch.Tensor) -> None:
    """The compute stream waits for ``event`` and takes over ``bufs`` (_comm_overlap.py:66-79)."""
    compute = torch.cuda.current_stream()
    compute.wait_event(event)
    for b in bufs:
        b.record_stream(compute)


class RingKVProvider:
    """K/V chunks of one rank's ring, the packed ``(2, ...)`` K/V tensor circulating towards
    ``rank - 1`` (``direction=-1``), so that step ``s`` holds global chunk ``(rank + s) % P``.

    ``comm_stream=None`` gives the plain provider, a side stream the overlapped one."""

    def __init__(self, k_local: torch.Tensor, v_local: torch.Tensor, rank: int, world_size: int, send_op_fn: SendOp,
                 group: Any = None, comm_stream: torch.cuda.Stream | None = None) -> None:
        if k_local.shape != v_local.shape or k_local.dtype != v_local.dtype:
            raise ValueError("k and v chunks must agree in shape and dtype")
        if not 0 <= rank < world_size:
            raise ValueError(f"rank {rank} outside a ring of {world_size}")
        self.rank, self.world_size, self.group = rank, world_size, group
        self._send, self._cs = send_op_fn, comm_stream
        self._kv = torch.stack((k_local, v_local)).contiguous()  # the circulated tensor
        self._bufs = [torch.empty_like(self._kv), torch.empty_like(self._kv)]
        self._pending = 0          # buffer the next get() adopts
        self._work: Any = None
        self._event: torch.cuda.Event | None = None
        self._next = 0             # step the next get() must ask for
        if world_size > 1:
            self._kick(self._kv, into=0, tag=0)

    def global_chunk_idx(self, step: int) -> int:
        """Global index of the chunk held at ``step`` (forward_chunk_provider.py:190-192)."""
        return (self.rank + step) % self.world_size

    def _kick(self, src: torch.Tensor, into: int, tag: int) -> None:
        buf = self._bufs[into]

        def produce():
            return self._send(src, buf, direction=-1, group=self.group, async_op=True, tag=tag)

        if self._cs is None:
            _, self._work = produce()
            self._event = None
        else:
            _, self._work, self._event = issue_on_comm_stream(self._cs, produce, keep_alive=(src, buf))
        self._pending = into

    def get(self, step: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Key and value of step ``step`` (steps are asked for in order, once each); receives the
        chunk sent during the previous step and relays it onwards before returning."""
        if step != self._next or step >= self.world_size:
            raise ValueError(f"ring steps are taken in order: expected {self._next}, got {step}")
        self._next += 1
        if step > 0:
            recv = self._bufs[self._pending]
            if self._cs is None:
                if self._work is not None:
                    self._work.wait()
            else:
                consume(self._event, recv)
            self._kv = recv
            if step + 1 < self.world_size:
                # relay into the other buffer; an overlapped kick first waits for the compute stream,
                # i.e. for the core of step - 1 that still reads that buffer
                self._kick(self._kv, into=1 - self._pending, tag=step)
        return self._kv[0], self._kv[1]


def ring_forward_from_provider(q: torch.Tensor, provider: RingKVProvider, scale: float):
    """``(out, lse)`` of ``q`` over the provider's ``P`` chunks: the loop of ring_forward
    (jigsaw/modules/attention/_functional/forward.py:172-199) with the chunk fetch in the
    provider. fp32 accumulator, cast to ``q.dtype`` once at the end."""
    acc = torch.promote_types(q.dtype, torch.float32)
    out = torch.zeros(q.shape, device=q.device, dtype=acc)
    lse = torch.full(q.shape[:-1], float("-inf"), device=q.device, dtype=acc)
    for step in range(provider.world_size):
        kj, vj = provider.get(step)
        out, lse = attend_step_(q, kj.to(q.dtype), vj.to(q.dtype), scale, out, lse)
    return out.to(q.dtype), lse


__all__ = ["RingKVProvider", "consume", "issue_on_comm_stream", "ring_forward_from_provider"]
