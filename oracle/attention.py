"""Oracle for the ring-attention step: math core, online-softmax merge, and the
forward / backward loops over K/V chunks for one rank's queries. Test
infrastructure only."""

from __future__ import annotations

import torch


def core_forward(q, k, v, scale):
    """``(out, logsumexp)`` of one chunk; ``bhsd`` tensors.

    Follows cores/math.forward, jigsaw/modules/attention/_functional/cores/math.py:69-78
    (dropout 0): scores = (q @ k^T) * scale; natural-log logsumexp over keys;
    softmax; out = p @ v.
    """
    scores = (q @ k.mT) * scale
    logsumexp = scores.logsumexp(dim=-1)
    p = torch.softmax(scores, dim=-1)
    return p @ v, logsumexp


def core_backward(grad_out, q, k, v, out, logsumexp, scale):
    """``(dq, dk, dv)`` of one chunk from the GLOBAL ``out`` / ``logsumexp``.

    Follows cores/math.backward, jigsaw/modules/attention/_functional/cores/math.py:125-149:
    p = exp(scores - lse) is already globally normalised; D = rowsum(dO * O).
    """
    attn = (q @ k.mT) * scale
    p = torch.exp(attn - logsumexp.unsqueeze(-1).to(attn.dtype))
    dv = p.mT @ grad_out
    dp = grad_out @ v.mT
    d = (grad_out * out).sum(dim=-1, keepdim=True)
    d_attn = p * (dp - d) * scale
    dq = d_attn @ k
    dk = d_attn.mT @ q
    return dq, dk, dv


def merge_(o1, l1, o2, l2, layout="bhsd", form="eager"):
    """Merge ``(o2, l2)`` into ``(o1, l1)``; returns ``(o1, l_new)``; o1 in place.

    ``form="eager"`` follows _online_softmax_merge_,
    jigsaw/modules/attention/_functional/forward.py:56-61
    (``o1.mul_(1 - w).addcmul_(w, o2)``, ``logaddexp``); ``form="fused"`` follows the
    Triton kernel, _merge_kernel.py:70-82 (``a + w * (b - a)``,
    ``max + log(1 + exp(-|l1 - l2|))``).
    """
    w = torch.sigmoid(l2 - l1)
    if layout == "bshd":
        w = w.transpose(1, 2)
    w = w.unsqueeze(-1)
    if form == "eager":
        o1.mul_(1 - w).addcmul_(w, o2.to(o1.dtype))
        return o1, torch.logaddexp(l1, l2)
    a = o1.float()
    o1.copy_((a + w * (o2.float() - a)).to(o1.dtype))
    mx = torch.maximum(l1, l2)
    return o1, mx + torch.log(1.0 + torch.exp(-(l1 - l2).abs()))


def ring_forward(q, k_chunks, v_chunks, scale, rank=0):
    """``(out, lse)`` for one rank's queries over all P chunks.

    Follows ring_forward, jigsaw/modules/attention/_functional/forward.py:160-199:
    fp32 accumulator ``out = 0``, ``lse = -inf`` (:161-167); step ``s`` attends
    chunk ``(rank + s) % P`` (forward_chunk_provider.py:190-192); per step the
    core runs in ``q.dtype`` and the result is merged (:64-96); ``out`` is cast
    to ``q.dtype`` once at the end (:199).
    """
    P = len(k_chunks)
    acc = torch.promote_types(q.dtype, torch.float32)
    out = torch.zeros(q.shape, dtype=acc)
    lse = torch.full(q.shape[:-1], float("-inf"), dtype=acc)
    for step in range(P):
        j = (rank + step) % P
        out_j, l_j = core_forward(q, k_chunks[j].to(q.dtype), v_chunks[j].to(q.dtype), scale)
        out, lse = merge_(out, lse, out_j, l_j.to(acc))
    return out.to(q.dtype), lse


def ring_backward(dout, q, out, lse, k_chunks, v_chunks, scale):
    """``(dq, [dk_j], [dv_j])`` of one rank's queries against every chunk.

    Follows ring_backward, jigsaw/modules/attention/_functional/backward.py:176-270:
    ``dout, q, out`` in ``q.dtype``, ``lse`` stays fp32 (:179-183); ``dq``
    accumulates in ``q.dtype`` (:184, 269); the default configuration visits chunk
    ``s`` at step ``s`` (:97-98). The cross-rank sum of dK/dV is left out: the
    per-chunk contributions of this rank are returned.
    """
    core = q.dtype
    dout, out = dout.to(core), out.to(core)
    dq = torch.zeros_like(q)
    dks, dvs = [], []
    for j in range(len(k_chunks)):
        dq_j, dk_j, dv_j = core_backward(dout, q, k_chunks[j].to(core), v_chunks[j].to(core), out, lse, scale)
        dq += dq_j
        dks.append(dk_j)
        dvs.append(dv_j)
    return dq, dks, dvs


def ring_all_ranks(qs, ks, vs, douts, scale, save_scope="global"):
    """Every rank of a ring of ``P = len(qs)`` ranks, forward and backward, with the
    cross-rank dK/dV sums: ``([out_r], [lse_r], [dq_r], [dk_r], [dv_r])``.

    Rank ``r`` holds ``qs[r], ks[r], vs[r]``. Forward as :func:`ring_forward`. Backward
    per rank as :func:`ring_backward`; the owner of chunk ``r`` then sums what the ranks
    computed for it:

    * ``"global"`` (saved chunks, SEND_DKV; backward.py:272-277): a SUM all-reduce of
      each step's partial, i.e. the contributions of ranks 0 .. P-1 added in the core dtype;
    * ``"local"`` (re-circulated chunks, SEND_DKV; backward.py:484-538): the own step-0
      partial first, then at step ``s`` the partial received from rank ``r - s``
      (which holds chunk ``r`` at its step ``s``), added in arrival order.
    """
    P = len(qs)
    outs, lses, dqs, parts = [], [], [], []
    for r in range(P):
        o, l = ring_forward(qs[r], ks, vs, scale, rank=r)
        dq, dkj, dvj = ring_backward(douts[r], qs[r], o, l, ks, vs, scale)
        outs.append(o), lses.append(l), dqs.append(dq), parts.append((dkj, dvj))
    dks, dvs = [], []
    for r in range(P):
        if save_scope == "global":
            order = list(range(P))
        elif save_scope == "local":
            order = [(r - s) % P for s in range(P)]
        else:
            raise ValueError(save_scope)
        dk = parts[order[0]][0][r].clone()
        dv = parts[order[0]][1][r].clone()
        for src in order[1:]:
            dk += parts[src][0][r]
            dv += parts[src][1][r]
        dks.append(dk), dvs.append(dv)
    return outs, lses, dqs, dks, dvs


def window_attention(q, k, v, bias):
    """Windowed attention with an additive bias / mask, as the Swin example calls
    ``F.scaled_dot_product_attention(q, k, v, attn_mask=bias)`` (examples/swin.py:148-151):
    softmax(q k^T / sqrt(d) + bias) v."""
    scale = q.shape[-1] ** -0.5
    s = (q @ k.mT) * scale + bias
    return torch.softmax(s, dim=-1) @ v
