#!/usr/bin/env python3
"""Benchmark of the per-rank hot path on one MI355X.

One "step" is one pass of the halo-exchange convolution of BASELINE.json's
configuration 2 for one rank: pack the 8 strips, assemble the padded tile from
the (seeded, locally held) neighbour strips, convolution forward, then dgrad
(writing the owned cells and the halo gradients to send in one pass), wgrad with
the bias gradient from the same pass, and the fold of the neighbours' halo
gradients into the border. All inputs are resident in HBM before the
timed region. ``value`` is the convolution's algorithmic FLOPs (fwd + dgrad +
wgrad) divided by the whole step time, halo movement included.

Prints ONE JSON line (see the keys below). ``--gpus`` above 1 is refused: this
build runs one rank's share on one GPU and has no collectives.
"""

from __future__ import annotations

import argparse
import gc
import itertools
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E
PEAK_FP32_TFLOPS = 157.3  # MI355X dense fp32 MFMA (and vector FMA)

METRIC = "halo-conv fwd+bwd & ring-attn step TFLOP/s on 1 GPU; % MFMA peak; halo GB/s"

# HBM bytes per launch of the three convolution kernels of the step (FETCH_SIZE + WRITE_SIZE
# from rocprofv3 --pmc, scaled by a copy kernel of known size).
CONV_TRAFFIC_BYTES = {"fwd": 2.24e9, "dgrad_fold": 2.87e9, "wgrad_bias": 2.31e9}  # wgrad: 2.23 GB + 0.08 GB for its reduction
CONV_KERNEL_NAMES = {
    "fwd": "conv3x3_mfma_kernel (forward, config 2)",
    "dgrad_fold": "conv3x3_mfma_kernel (dgrad with the fold epilogue, config 2)",
    "wgrad_bias": "wgrad3x3_mfma_kernel + reduction (weight and bias gradient, config 2)",
}


def _events():
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def time_gpu(fn, iters: int, warmup: int = 2) -> float:
    """Average milliseconds per call, HIP events on the stream the kernels run on
    (the library launches on torch's current stream)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    # a full collection of the interpreter's garbage collector takes tens of milliseconds
    # in a process this size and would land inside one of these short loops
    gc.collect()
    gc.disable()
    try:
        e0, e1 = _events()
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
    finally:
        gc.enable()
    return e0.elapsed_time(e1) / iters


def build_conv2_workload(dev, batch=8, ch=64, tile=1024):
    """Configuration 2: one rank's 1024x1024 tile of a 2048x2048 domain, batch 8,
    64 -> 64 channels, 3x3, pad 1; bf16 N(0,1) activations, Kaiming-uniform weights.
    The 8 neighbour strips (width 1) are seeded stand-ins for the neighbours' edges."""
    from jigsaw_amd.halo import HaloGeometry

    g = torch.Generator(device=dev).manual_seed(0)
    geom = HaloGeometry((tile, tile), (1, 1), (1, 1))
    lead = (batch, ch)
    x = torch.randn(*lead, tile, tile, device=dev, generator=g).bfloat16()
    bound = 1.0 / (ch * 9) ** 0.5
    w = ((torch.rand(ch, ch, 3, 3, device=dev, generator=g) * 2 - 1) * bound).bfloat16()
    b = ((torch.rand(ch, device=dev, generator=g) * 2 - 1) * bound).bfloat16()
    gout = torch.randn(*lead, tile, tile, device=dev, generator=g).bfloat16()
    strips_fwd = {
        o: torch.randn(*lead, *geom.strip_extent(o, "assemble"), device=dev, generator=g).bfloat16()
        for o in geom.offsets()
    }
    strips_bwd = {
        o: torch.randn(*lead, *geom.strip_extent(o, "fold"), device=dev, generator=g).bfloat16()
        for o in geom.offsets()
    }
    from jigsaw_amd import conv as jc

    bands = jc.frame_bands(x, geom, w.shape)
    if bands is None:
        raise RuntimeError("the framed kernels should cover configuration 2")
    return {"geom": geom, "x": x, "w": w, "b": b, "g": gout, "strips_fwd": strips_fwd, "strips_bwd": strips_bwd,
            "bands": bands}


def conv_step_buffers(wl) -> dict:
    """Every tensor one step writes, and the three workspaces, allocated once: the timed steps then
    allocate nothing (``out=`` / ``workspace=`` of the host functions)."""
    from jigsaw_amd import conv as jc
    from jigsaw_amd.halo import halo_assemble, halo_pack

    geom, x, w, g = wl["geom"], wl["x"], wl["w"], wl["g"]
    dev = x.device
    ws = lambda: torch.empty(256 << 20, dtype=torch.uint8, device=dev)  # noqa: E731  (more than any of the three asks for)
    buf = {"ws_fwd": ws(), "ws_dgrad": ws(), "ws_wgrad": ws()}
    buf["pack"] = halo_pack(x, geom, from_padded=False)
    buf["x_aug"] = halo_assemble(x, wl["strips_fwd"], geom)
    buf["y"] = jc.conv_nd(buf["x_aug"], w, wl["b"])
    buf["gx_send"] = jc.conv_nd_input_fold(geom, w, g)
    buf["gw_gb"] = jc.conv_nd_weight(buf["x_aug"], w.shape, g, with_bias_grad=True)
    return buf


def conv_step(wl, buf, kernel_events=None):
    """The hot path of one rank for one batch (see the module docstring). The backward
    uses the fused forms, each with the bits of the separate steps it replaces: dgrad
    writes the owned cells and the strips it sends in one pass, wgrad adds up the bias
    gradient on the way, and the received strips are added to the border afterwards.
    ``kernel_events`` maps a name to (start, end) HIP events, made before the loop, recorded here on the
    launch stream around the three convolution launches of the step."""
    from jigsaw_amd import conv as jc
    from jigsaw_amd.halo import halo_assemble, halo_fold_border_, halo_pack

    geom, x, w, b, g = wl["geom"], wl["x"], wl["w"], wl["b"], wl["g"]

    def bracket(name, fn):
        if kernel_events is None:
            return fn()
        e0, e1 = kernel_events[name]
        e0.record()
        out = fn()
        e1.record()
        return out

    halo_pack(x, geom, from_padded=False, out=buf["pack"])  # strips this rank sends
    x_aug = halo_assemble(x, wl["strips_fwd"], geom, out=buf["x_aug"])
    y = bracket("fwd", lambda: jc.conv_nd(x_aug, w, b, out=buf["y"], workspace=buf["ws_fwd"]))
    # owned cells + halo gradients this rank sends
    gx, _send = bracket("dgrad_fold", lambda: jc.conv_nd_input_fold(geom, w, g, out=buf["gx_send"], workspace=buf["ws_dgrad"]))
    # one pass over g for the weight and the bias gradient
    gw, gb = bracket("wgrad_bias", lambda: jc.conv_nd_weight(x_aug, w.shape, g, with_bias_grad=True, out=buf["gw_gb"],
                                                             workspace=buf["ws_wgrad"]))
    halo_fold_border_(gx, wl["strips_bwd"], geom)
    return y, gx, gw, gb


def timed_conv_steps(wl, steps: int, warmup: int) -> dict:
    """W warm-up steps, then exactly K timed steps with the collector off and nothing allocated:
    HIP events around every step and around its three convolution launches (all events made
    before the loop), a synchronisation on both sides. Returns per-step and per-kernel times."""
    buf = conv_step_buffers(wl)
    names = ("fwd", "dgrad_fold", "wgrad_bias")
    step_ev = [_events() for _ in range(steps)]
    kern_ev = [{n: _events() for n in names} for _ in range(steps)]
    for _ in range(warmup):
        conv_step(wl, buf)
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()
    try:
        t0 = time.perf_counter()
        for i in range(steps):
            step_ev[i][0].record()
            conv_step(wl, buf, kern_ev[i])
            step_ev[i][1].record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
    finally:
        gc.enable()
    per_step = [a.elapsed_time(b) for a, b in step_ev]
    span_ms = step_ev[0][0].elapsed_time(step_ev[-1][1])  # first step's start to last step's end, gaps included
    per_kernel = {n: [ev[n][0].elapsed_time(ev[n][1]) for ev in kern_ev] for n in names}
    return {"per_step": per_step, "span_ms": span_ms, "wall_ms": wall_ms, "per_kernel": per_kernel, "buf": buf}


def _median(v):
    v = sorted(v)
    n = len(v)
    return v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])


def ln_statistics_calls(dev, g, big_rows: int = 1 << 18, cols: int = 256):
    """The sharded LayerNorm's two statistics passes (forward: one tensor read; backward: g and x_hat read,
    column partials for the weight / bias gradient and their reduction) on 2 ** 18 rows of configuration 4's
    local width, over six different 134 MB tensors in turn: one alone would stay in the 256 MB last-level
    cache and the figure would not be an HBM rate. The C entry points are called on buffers made once, so that
    the host's share of such short kernels (two allocations a call) stays out of the figure. Returns the two
    callables and the number of calls after which the inputs repeat."""
    from jigsaw_amd import _lib

    lib = _lib.load()
    xls = [torch.randn(big_rows, cols, device=dev, generator=g).bfloat16() for _ in range(6)]
    mean_b, var_b = torch.empty(big_rows, device=dev), torch.empty(big_rows, device=dev)
    bf16 = _lib.dtype_code(torch.bfloat16)
    turn = itertools.count()
    w_ln = torch.ones(cols, device=dev, dtype=torch.bfloat16)
    gw_b, gb_b = torch.empty(cols, device=dev), torch.empty(cols, device=dev)
    ws_bytes = int(lib.jg_ln_bwd_workspace_bytes(big_rows, cols))
    ws_ln = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def stats_fwd():
        t = xls[next(turn) % len(xls)]
        _lib.check(lib.jg_ln_partial_fwd(_lib.ptr(mean_b), _lib.ptr(var_b), _lib.ptr(t), big_rows, cols, bf16,
                                         _lib.stream_ptr(dev)), "jg_ln_partial_fwd")

    def stats_bwd():
        i = next(turn) % (len(xls) // 2)
        _lib.check(lib.jg_ln_partial_bwd(_lib.ptr(mean_b), _lib.ptr(var_b), _lib.ptr(gw_b), _lib.ptr(gb_b), _lib.ptr(xls[2 * i]),
                                         _lib.ptr(xls[2 * i + 1]), _lib.ptr(w_ln), big_rows, cols, bf16, _lib.ptr(ws_ln), ws_bytes,
                                         _lib.stream_ptr(dev)), "jg_ln_partial_bwd")

    return stats_fwd, stats_bwd, len(xls)


def attention_figures(dev, iters: int) -> dict:
    """Configuration 4: one rank's ring-attention step. 8 local heads, 4096 local
    queries, one K/V chunk of 4096 keys per step (4 steps), head size 64, bf16.
    Forward = flash core with the LSE merge fused in; backward = dQ + dK/dV kernels
    from the global out / lse. Also the sharded LayerNorm statistics (dim 512, 256 local)."""
    from jigsaw_amd import attention as ja
    from jigsaw_amd import layernorm as jl

    b, h, n, d, P = 1, 8, 4096, 64, 4
    g = torch.Generator(device=dev).manual_seed(0)
    q = (torch.randn(b, h, n, d, device=dev, generator=g) / 8).bfloat16()
    ks = [(torch.randn(b, h, n, d, device=dev, generator=g) / 8).bfloat16() for _ in range(P)]
    vs = [(torch.randn(b, h, n, d, device=dev, generator=g) / 8).bfloat16() for _ in range(P)]
    dout = torch.randn(b, h, n, d, device=dev, generator=g).bfloat16()
    scale = d**-0.5
    acc = torch.zeros(b, h, n, d, device=dev)
    lse = torch.full((b, h, n), float("-inf"), device=dev)
    f_fwd = 4 * b * h * n * n * d
    f_bwd = 10 * b * h * n * n * d
    ms_f = time_gpu(lambda: ja.core_forward(q, ks[0], vs[0], scale, out_acc=acc, lse_acc=lse, want_out=False), iters)
    out, l = ja.ring_forward(q, ks, vs, scale)
    ms_b = time_gpu(lambda: ja.core_backward(dout, q, ks[0], vs[0], out, l, scale), iters)
    ms_ring = time_gpu(lambda: ja.ring_forward(q, ks, vs, scale), iters)
    # The same ring with the hops in the loop (jigsaw_amd.ring.RingSeat): every step forwards the chunk
    # it holds and receives the next one, on the compute stream or on the seat's transfer stream. The
    # neighbour's transfer is a device copy of the 8 MiB (K and V of a chunk in one message); "link" puts a spinning one-thread kernel of
    # about the time the message takes over one 153 GB/s xGMI link in front of it (a transfer over the
    # link, unlike a big device copy, occupies neither the compute units nor HBM).
    from jigsaw_amd import ring as jr

    cal = 2_000_000
    ms_cal = time_gpu(lambda: torch.cuda._sleep(cal), 5)
    link_cycles = int(cal * (ks[0].numel() * 2 / 153e9 * 1e3) / ms_cal)  # one K or V message

    kvs = [torch.stack((k, v)) for k, v in zip(ks, vs)]  # a chunk travels as one message: K and V together

    def seat_for(link, overlap, scope):
        def hop(src, buf, direction, *, group, async_op, tag):
            if link:
                torch.cuda._sleep(2 * link_cycles)
            buf.copy_(kvs[(tag + 1) % P])
            return buf, None

        def relay(src, buf, offset, *, group, async_op, step):
            if link:
                torch.cuda._sleep(link_cycles)
            buf.copy_(src)  # the partial the peer would have sent: same size
            return buf, None

        return jr.RingSeat(0, P, ks[0], hop, relay_fn=relay, save_scope=scope, overlap=overlap)

    hop, hop_bwd = {}, {}
    for name, link, overlap in (("ms_copy_inline", False, False), ("ms_copy_overlapped", False, True),
                                ("ms_link_inline", True, False), ("ms_link_overlapped", True, True)):
        seat = seat_for(link, overlap, "local")
        k0, v0 = kvs[0][0], kvs[0][1]  # V behind K in memory, as the packed projection leaves them: sent from where they lie
        hop[name] = time_gpu(lambda: seat.forward(q, k0, v0, scale), iters)
        _, _, saved = seat.forward(q, k0, v0, scale)
        hop_bwd[name] = time_gpu(lambda: seat.backward(dout, q, out, l, scale, saved), iters)
    hop["ms_no_hop"] = ms_ring
    hop_bwd["ms_no_hop"] = time_gpu(lambda: ja.ring_backward(dout, q, out, l, ks, vs, scale), iters)
    x = torch.randn(b, n, 256, device=dev, generator=g).bfloat16()
    ms_ln = time_gpu(lambda: jl.partial_stats(x), iters)
    # the same statistics, and the backward's partial sums, on a shard that fills the chip
    stats_fwd, stats_bwd, n_turn = ln_statistics_calls(dev, g)
    ms_ln_big = time_gpu(stats_fwd, max(iters, 2 * n_turn), warmup=n_turn)
    ms_ln_bwd = time_gpu(stats_bwd, max(iters, 2 * n_turn), warmup=n_turn)
    del stats_fwd, stats_bwd
    # the separate LSE merge (what a step runs when its core cannot fuse it): fp32 accumulator read and
    # written, the step's bf16 output read; at the step's size and at 16 x the heads
    merge = {}
    for name, hh in (("lse_merge_step", h), ("lse_merge_128_heads", 16 * h)):
        o1 = torch.randn(b, hh, n, d, device=dev, generator=g)
        l1 = torch.randn(b, hh, n, device=dev, generator=g)
        o2 = torch.randn(b, hh, n, d, device=dev, generator=g).bfloat16()
        l2 = torch.randn(b, hh, n, device=dev, generator=g)
        ms_m = time_gpu(lambda: ja.fused_online_softmax_merge_(o1, l1, o2, l2, "bhsd"), iters)
        nbytes = o1.numel() * (4 + 4 + 2) + l1.numel() * 12
        merge[name] = {"ms": ms_m, "GBps": nbytes / (ms_m * 1e-3) / 1e9, "bytes": nbytes,
                       "frac_hbm_peak": nbytes / (ms_m * 1e-3) / 1e9 / PEAK_HBM_GBPS}
        del o1, l1, o2, l2
    # the ring step on fp32 inputs: the fp32 matrix-core kernels (peak 157.3 TFLOP/s)
    q32, k32, v32, do32 = q.float(), ks[0].float(), vs[0].float(), dout.float()
    acc32, lse32 = torch.zeros(b, h, n, d, device=dev), torch.full((b, h, n), float("-inf"), device=dev)
    ms_f32 = time_gpu(lambda: ja.core_forward(q32, k32, v32, scale, out_acc=acc32, lse_acc=lse32, want_out=False), iters)
    o32, l32 = ja.core_forward(q32, k32, v32, scale)
    ms_b32 = time_gpu(lambda: ja.core_backward(do32, q32, k32, v32, o32, l32, scale), iters)
    tf = lambda f, ms: f / (ms * 1e-3) / 1e12  # noqa: E731
    return {
        "attn_fwd_step": {"ms": ms_f, "tflops": tf(f_fwd, ms_f), "frac_mfma_peak": tf(f_fwd, ms_f) / PEAK_BF16_TFLOPS},
        "attn_bwd_step": {"ms": ms_b, "tflops": tf(f_bwd, ms_b), "frac_mfma_peak": tf(f_bwd, ms_b) / PEAK_BF16_TFLOPS},
        "attn_ring_fwd_4_steps": {"ms": ms_ring, "tflops": tf(4 * f_fwd, ms_ring)},
        "attn_ring_fwd_4_steps_with_hop": hop,
        "attn_ring_bwd_4_steps_with_hop_and_dkv_relay": hop_bwd,
        "attn_fp32_fwd_step": {"ms": ms_f32, "tflops": tf(f_fwd, ms_f32), "frac_fp32_mfma_peak": tf(f_fwd, ms_f32) / PEAK_FP32_TFLOPS},
        "attn_fp32_bwd_step": {"ms": ms_b32, "tflops": tf(f_bwd, ms_b32), "frac_fp32_mfma_peak": tf(f_bwd, ms_b32) / PEAK_FP32_TFLOPS},
        **merge,
        "ln_partial_stats": {"ms": ms_ln, "GBps": x.numel() * 2 / (ms_ln * 1e-3) / 1e9, "bytes": x.numel() * 2},
        "ln_partial_stats_262144_rows": {"ms": ms_ln_big, "GBps": (1 << 18) * 256 * 2 / (ms_ln_big * 1e-3) / 1e9,
                                         "bytes": (1 << 18) * 256 * 2, "frac_hbm_peak": (1 << 18) * 256 * 2 / (ms_ln_big * 1e-3) / 1e9 / PEAK_HBM_GBPS},
        "ln_partial_bwd_262144_rows_with_column_reduction": {
            "ms": ms_ln_bwd, "GBps": 2 * (1 << 18) * 256 * 2 / (ms_ln_bwd * 1e-3) / 1e9, "bytes": 2 * (1 << 18) * 256 * 2,
            "frac_hbm_peak": 2 * (1 << 18) * 256 * 2 / (ms_ln_bwd * 1e-3) / 1e9 / PEAK_HBM_GBPS},
    }


def conv3d_figures(dev, iters: int) -> dict:
    """Configuration 3: one rank's 128^3 tile of a 256^3 volume, batch 2, 32 -> 32
    channels, 3x3x3, pad 1, bf16; 26 seeded halo strips of width 1."""
    from jigsaw_amd import conv as jc
    from jigsaw_amd.halo import HaloGeometry, halo_assemble, halo_fold, halo_fold_border_, halo_pack

    g = torch.Generator(device=dev).manual_seed(1)
    n, lead, ch = (128, 128, 128), (2, 32), 32
    geom = HaloGeometry(n, (1, 1, 1), (1, 1, 1))
    x = torch.randn(*lead, *n, device=dev, generator=g).bfloat16()
    bound = 1.0 / (ch * 27) ** 0.5
    w = ((torch.rand(ch, ch, 3, 3, 3, device=dev, generator=g) * 2 - 1) * bound).bfloat16()
    gout = torch.randn(*lead, *n, device=dev, generator=g).bfloat16()
    sf = {o: torch.randn(*lead, *geom.strip_extent(o, "assemble"), device=dev, generator=g).bfloat16() for o in geom.offsets()}
    sb = {o: torch.randn(*lead, *geom.strip_extent(o, "fold"), device=dev, generator=g).bfloat16() for o in geom.offsets()}
    x_aug = halo_assemble(x, sf, geom)
    gx_aug = jc.conv_nd_input(x_aug.shape, w, gout)
    flop = 2 * lead[0] * ch * ch * 27 * n[0] * n[1] * n[2]
    nbytes = (x.numel() + x_aug.numel()) * 2
    ms = {
        "fwd": time_gpu(lambda: jc.conv_nd(x_aug, w, None), iters),
        "dgrad": time_gpu(lambda: jc.conv_nd_input(x_aug.shape, w, gout), iters),
        "wgrad": time_gpu(lambda: jc.conv_nd_weight(x_aug, w.shape, gout), iters),
    }
    gx = torch.empty_like(x)
    ms_asm = time_gpu(lambda: halo_assemble(x, sf, geom, out=x_aug), iters)
    ms_fold = time_gpu(lambda: halo_fold(gx_aug, sb, geom, out=gx), iters)
    out = {f"conv3d_{k}": {"ms": v, "tflops": flop / (v * 1e-3) / 1e12, "frac_mfma_peak": flop / (v * 1e-3) / 1e12 / PEAK_BF16_TFLOPS} for k, v in ms.items()}
    out["halo3d_assemble"] = {"ms": ms_asm, "GBps": nbytes / (ms_asm * 1e-3) / 1e9, "frac_hbm_peak": nbytes / (ms_asm * 1e-3) / 1e9 / PEAK_HBM_GBPS}
    out["halo3d_fold"] = {"ms": ms_fold, "GBps": nbytes / (ms_fold * 1e-3) / 1e9, "frac_hbm_peak": nbytes / (ms_fold * 1e-3) / 1e9 / PEAK_HBM_GBPS}
    # the fused backward the layer runs by default, and its small companions
    ms_fused = time_gpu(lambda: jc.conv_nd_input_fold(geom, w, gout), iters)
    ms_border = time_gpu(lambda: halo_fold_border_(gx, sb, geom), iters)
    ms_pack = time_gpu(lambda: halo_pack(x, geom, from_padded=False), iters)
    out["conv3d_dgrad_fused_with_pack_and_fold"] = {"ms": ms_fused, "tflops": flop / (ms_fused * 1e-3) / 1e12}
    out["halo3d_fold_border"] = {"ms": ms_border}
    out["halo3d_pack"] = {"ms": ms_pack}
    return out


def groupnorm_figures(dev, iters: int) -> dict:
    """GroupNorm over a spatially sharded activation of configuration 2's shape
    (8 x 64 x 1024^2 bf16, 8 groups), one rank's passes: forward = sum, centred squares,
    normalise + affine (reads x three times, writes y and x_norm); backward = partial
    sums over g and x_norm, then the input gradient."""
    from jigsaw_amd import groupnorm as jgn

    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(8, 64, 1024, 1024, device=dev, generator=g).bfloat16().requires_grad_()
    w = (1 + 0.1 * torch.randn(64, device=dev, generator=g)).bfloat16().requires_grad_()
    b = (0.1 * torch.randn(64, device=dev, generator=g)).bfloat16().requires_grad_()
    gy = torch.randn(8, 64, 1024, 1024, device=dev, generator=g).bfloat16()
    nbytes = x.numel() * 2
    ms_fwd = time_gpu(lambda: jgn.group_norm(x.detach(), 8, w.detach(), b.detach(), (), 1e-5), iters)

    def fwd_bwd():
        x.grad = None
        jgn.group_norm(x, 8, w, b, (), 1e-5).backward(gy)

    ms_both = time_gpu(fwd_bwd, max(3, iters // 2))
    ms_bwd = ms_both - ms_fwd
    return {
        "groupnorm_fwd": {"ms": ms_fwd, "GBps": 5 * nbytes / (ms_fwd * 1e-3) / 1e9, "bytes": 5 * nbytes},
        "groupnorm_bwd": {"ms": ms_bwd, "GBps": 5 * nbytes / (ms_bwd * 1e-3) / 1e9, "bytes": 5 * nbytes},
    }


def attention_wide_figures(dev, iters: int) -> dict:
    """The attention core at head size 128 (its own MFMA kernels): 32 heads, 4096 queries x 4096
    keys, bf16; forward, and backward (dQ + dK/dV) from the global out / lse."""
    from jigsaw_amd import attention as ja

    h, n, d = 32, 4096, 128
    g = torch.Generator(device=dev).manual_seed(5)
    q = (torch.randn(1, h, n, d, device=dev, generator=g) / d**0.5).bfloat16()
    k = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    v = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    dout = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    out, lse = ja.core_forward(q, k, v, d**-0.5)
    ms_f = time_gpu(lambda: ja.core_forward(q, k, v, d**-0.5), iters)
    ms_b = time_gpu(lambda: ja.core_backward(dout, q, k, v, out, lse, d**-0.5), iters)
    f_fwd = 4.0 * h * n * n * d
    tf = lambda f, ms: f / (ms * 1e-3) / 1e12  # noqa: E731
    return {
        "attn_d128_fwd": {"ms": ms_f, "tflops": tf(f_fwd, ms_f), "frac_mfma_peak": tf(f_fwd, ms_f) / PEAK_BF16_TFLOPS},
        "attn_d128_bwd": {"ms": ms_b, "tflops": tf(2.5 * f_fwd, ms_b), "frac_mfma_peak": tf(2.5 * f_fwd, ms_b) / PEAK_BF16_TFLOPS},
    }


def projection_figures(dev, iters: int) -> dict:
    """The projections around the attention core with the head split / merge fused into the
    GEMM addressing, on 8 sequences of configuration 4 (32768 tokens, 512 channels, 8 heads
    of 64, bf16): qkv projection writing (3, b, h, s, d), output projection reading
    (b, h, s, d); the qkv backward is the input gradient (one GEMM) plus the weight and
    bias gradient (one GEMM contracted over the tokens and its reduction)."""
    from jigsaw_amd import projection as jp

    g = torch.Generator(device=dev).manual_seed(4)
    bsz, s, c, heads = 8, 4096, 512, 8
    x = torch.randn(bsz, s, c, device=dev, generator=g).bfloat16().requires_grad_()
    w = (torch.randn(3 * c, c, device=dev, generator=g) / c ** 0.5).bfloat16().requires_grad_()
    b = (0.1 * torch.randn(3 * c, device=dev, generator=g)).bfloat16().requires_grad_()
    wo = (torch.randn(c, c, device=dev, generator=g) / c ** 0.5).bfloat16()
    o = torch.randn(bsz, heads, s, c // heads, device=dev, generator=g).bfloat16()
    gy = torch.randn(3, bsz, heads, s, c // heads, device=dev, generator=g).bfloat16()
    flops = 2.0 * bsz * s * c * 3 * c
    ms_qkv = time_gpu(lambda: jp.qkv_projection(x.detach(), w.detach(), b.detach(), heads), iters)
    ms_out = time_gpu(lambda: jp.heads_projection(o, wo, None), iters)
    y = jp.qkv_projection(x, w, b, heads)
    ms_bwd = time_gpu(lambda: torch.autograd.grad(y, (x, w, b), gy, retain_graph=True), iters)
    return {
        "qkv_projection_fwd": {"ms": ms_qkv, "TFLOPs": flops / (ms_qkv * 1e-3) / 1e12},
        "heads_projection_fwd": {"ms": ms_out, "TFLOPs": flops / 3 / (ms_out * 1e-3) / 1e12},
        "qkv_projection_bwd": {"ms": ms_bwd, "TFLOPs": 2 * flops / (ms_bwd * 1e-3) / 1e12},
    }


def _swin_step(dev):
    """Configuration 5's block, its inputs and ``step()`` = one forward + backward under bf16 autocast."""
    from jigsaw_amd import projection as jp
    from jigsaw_amd import swin as js
    from jigsaw_amd.conv import TileGroup

    # the bf16 copies of the fp32 parameters are kept between steps, as a training loop whose optimizer
    # updates the parameters in place would ask for (nothing here writes through ``.data``)
    jp.remember_casts(True)
    g = torch.Generator(device=dev).manual_seed(2)
    slabs = {}

    def comm(data, buffer, direction, *, group, async_op):
        # the neighbour's slab: a seeded stand-in, made once per slab shape (the exchange itself
        # is not part of this figure, so it should not add kernels of its own to the step)
        key = (tuple(buffer.shape), direction, id(group))
        if key not in slabs:
            slabs[key] = torch.randn(buffer.shape, device=dev, generator=g).to(buffer.dtype)
        return slabs[key], None

    n, dim = (256, 256), 128
    groups = (TileGroup(2, 0), TileGroup(2, 1))
    block = js.SwinBlock(dim, 4, 8, n, groups, comm, shift=4, device=dev)
    x = torch.randn(1, *n, dim, device=dev, generator=g).bfloat16().requires_grad_()
    gout = torch.randn(1, *n, dim, device=dev, generator=g).bfloat16()
    leaves = [x, *block.parameters()]

    def step():
        for t in leaves:  # what optimizer.zero_grad() does: the backward then assigns instead of adding
            t.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = block(x)
        y.backward(gout)

    return step, x


def swin_figures(dev, iters: int) -> dict:
    """Configuration 5: one rank's Swin block on a 256x256-token tile, dim 128, 4 heads,
    8x8 windows, shift 4, bf16 autocast; the roll's cross-tile slabs are seeded."""
    from jigsaw_amd import roll as jr

    step, x = _swin_step(dev)
    # a host-bound step of ~40 launches: a handful of cold iterations says little, so more of them
    ms = time_gpu(step, max(20, iters), warmup=5)
    xr = x.detach()
    ms_roll = time_gpu(lambda: jr.roll(xr, (-4, -4), (1, 2)), iters)
    return {
        "swin_block_fwd_bwd": {"ms": ms},
        "roll": {"ms": ms_roll, "GBps": 2 * xr.numel() * 2 / (ms_roll * 1e-3) / 1e9, "bytes": 2 * xr.numel() * 2},
    }


def _cpu_conv2_step(batch: int, tile: int, dtype: torch.dtype):
    """One step of configuration 2 for rank (0, 0) of a 2 x 2 mesh on the oracle (the torch CPU
    operators the reference calls): halo gather of the whole mesh, conv forward, bias gradient,
    dgrad on the padded tile, wgrad, scatter-add. Returns seconds."""
    from oracle import conv as oc
    from oracle import halo as oh

    ch = 64
    torch.manual_seed(0)
    mesh, k, s, p, d = (2, 2), (3, 3), (1, 1), (1, 1), (1, 1)
    glob = torch.randn(batch, ch, 2 * tile, 2 * tile).to(dtype)
    w = ((torch.rand(ch, ch, 3, 3) * 2 - 1) / 24).to(dtype)
    b = ((torch.rand(ch) * 2 - 1) / 24).to(dtype)
    gout = torch.randn(batch, ch, tile, tile).to(dtype)
    tiles = oh.split_global(glob, mesh)
    del glob
    t0 = time.perf_counter()
    aug = oh.gather_mesh(tiles, mesh, k, s, p, d)
    lp = oh.local_padding(p, mesh)
    y = oc.forward(aug[(0, 0)], w, b, s, lp, d)
    gb = oc.grad_bias(gout, 2)
    gx_aug = {c: oc.dgrad(aug[c].shape, w, gout, s, lp, d) if c == (0, 0) else torch.zeros_like(aug[c]) for c in aug}
    gw = oc.wgrad(aug[(0, 0)], w.shape, gout, s, lp, d)
    gx = oh.scatter_add_mesh(gx_aug, mesh, k, s, p, d, (tile, tile))
    sec = time.perf_counter() - t0
    del y, gb, gx_aug, gw, gx, aug
    return sec


def cpu_baseline(seconds_budget: float = 25.0) -> dict:
    """The oracle (the reference's torch CPU operators) timed on the host cores. Runs BEFORE this
    process touches the GPU (its second leg starts child processes).

    Leg 1, the ``value``: configuration 2 at its real tile (1024 x 1024 of 2048 x 2048, 64 -> 64,
    bf16, rank (0, 0) of the 2 x 2 mesh; the gather and the scatter-add move the whole mesh). A
    small probe step estimates the rate; the batch (8 in the configuration) is cut to what fits
    the time budget and reported, the tile is not cut.
    Leg 2: configuration 1 as the reference runs it: four gloo ranks (fresh processes), one
    training step of the 3 -> 16 -> 3 model on 512 x 512 images, batch 4, fp32, with the halo
    all-to-alls, the loss and gradient all-reduces and Adam."""
    from oracle import train_step as ots

    cores = torch.get_num_threads()
    dtype = torch.bfloat16
    flop = lambda batch, tile: 3 * 2 * batch * 64 * 64 * 9 * tile * tile  # noqa: E731
    _cpu_conv2_step(1, 128, dtype)  # warm-up (thread pools, oneDNN primitive cache)
    probe = _cpu_conv2_step(1, 256, dtype)
    per_batch_entry = probe * 16.0  # a 1024^2 tile is 16 times the probe
    batch = int(max(1, min(8, seconds_budget / 2 / max(per_batch_entry, 1e-3))))
    secs = [_cpu_conv2_step(batch, 1024, dtype)]
    while sum(secs) + secs[-1] < seconds_budget / 2 and len(secs) < 5:
        secs.append(_cpu_conv2_step(batch, 1024, dtype))
    sec = sorted(secs)[len(secs) // 2]
    c1 = {}
    try:
        ranks = ots.run_four_ranks(steps=3, warmup=1, batch=4, size=512, threads=max(1, cores // 4), timeout=240.0)
        c1 = {"config1_ms_per_step": max(r[1] for r in ranks.values()) * 1e3, "config1_ranks": 4,
              "config1_threads_per_rank": max(1, cores // 4), "config1_loss": ranks[0][0][-1]}
    except Exception as exc:  # the CPU leg must not take the GPU figures down with it
        c1 = {"config1_error": repr(exc)}
    return {
        "value": flop(batch, 1024) / sec / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"configuration 2 on the oracle (torch CPU operators): halo gather + conv fwd/dgrad/wgrad/bias-grad + "
        f"scatter-add, bf16, real 1024x1024 tile of a 2x2 mesh, 64->64, batch {batch} of 8 "
        f"({flop(batch, 1024) / 1e9:.1f} of the step's {flop(8, 1024) / 1e9:.1f} GFLOP), {len(secs)} timed step(s) of "
        f"{sec:.2f} s, torch {torch.__version__}, {cores} threads of {os.cpu_count()} logical cores; "
        "configuration 1: one training step of 4 gloo ranks (see config1_* keys)",
        **c1,
    }


def conv2_extras(wl, x_aug, it: int, flop_one: int, flop_step: int, ms_fwd: float) -> dict:
    """Per-operator figures of configuration 2 beside the forward kernel: the separate
    dgrad / wgrad / fold, the fused forms the step uses, and the framed-input variants."""
    from jigsaw_amd import conv as jc
    from jigsaw_amd.halo import halo_assemble, halo_fold

    geom = wl["geom"]
    tf = lambda ms: flop_one / (ms * 1e-3) / 1e12  # noqa: E731
    gx_aug = jc.conv_nd_input(x_aug.shape, wl["w"], wl["g"])
    ms_fwd_loop = time_gpu(lambda: jc.conv_nd(x_aug, wl["w"], wl["b"]), it)  # launched back to back
    ms_dgrad = time_gpu(lambda: jc.conv_nd_input(x_aug.shape, wl["w"], wl["g"]), it)
    ms_wgrad = time_gpu(lambda: jc.conv_nd_weight(x_aug, wl["w"].shape, wl["g"]), it)
    gx_buf = torch.empty_like(wl["x"])
    ms_asm = time_gpu(lambda: halo_assemble(wl["x"], wl["strips_fwd"], geom, out=x_aug), it)
    ms_fold = time_gpu(lambda: halo_fold(gx_aug, wl["strips_bwd"], geom, out=gx_buf), it)
    ms_dgrad_fold = time_gpu(lambda: jc.conv_nd_input_fold(geom, wl["w"], wl["g"]), it)
    from jigsaw_amd.halo import halo_fold_border_

    ms_border = time_gpu(lambda: halo_fold_border_(gx_buf, wl["strips_bwd"], geom), it)
    x_frame = halo_assemble(wl["x"], wl["strips_fwd"], geom, bands=wl["bands"])
    ms_frame = time_gpu(lambda: halo_assemble(wl["x"], wl["strips_fwd"], geom, out=x_frame, bands=wl["bands"]), it)
    ms_fwd_framed = time_gpu(lambda: jc.conv_nd_framed(x_frame, wl["x"], geom, wl["w"], wl["b"]), it)
    ms_wgrad_framed = time_gpu(
        lambda: jc.conv_nd_weight_framed(x_frame, wl["x"], geom, wl["w"].shape, wl["g"], with_bias_grad=True), it
    )
    # transposed convolution of the same shape (k3 s1 p1, 64 -> 64): the mirror image of the
    # step, on the same kernels (forward = dgrad with the fold epilogue + border fold,
    # backward = assemble + plain conv + weight gradient with the operands exchanged)
    def convt_fwd():
        y_t, _ = jc.conv_nd_input_fold(geom, wl["w"], wl["x"])
        halo_fold_border_(y_t, wl["strips_bwd"], geom)

    def convt_bwd():
        g_raw = halo_assemble(wl["g"], wl["strips_fwd"], geom, out=x_aug)
        jc.conv_nd(g_raw, wl["w"], None)
        jc.conv_nd_weight(g_raw, wl["w"].shape, wl["x"])

    ms_convt_fwd = time_gpu(convt_fwd, it)
    ms_convt_bwd = time_gpu(convt_bwd, it)
    es = wl["x"].element_size()
    strip_bytes = sum(t.numel() for t in wl["strips_fwd"].values()) * es
    halo_bytes = (wl["x"].numel() + x_aug.numel()) * es + strip_bytes  # read tile + strips, write padded tile
    gbps = lambda ms: halo_bytes / (ms * 1e-3) / 1e9  # noqa: E731

    return {
        "conv_fwd_back_to_back": {"ms": ms_fwd_loop, "tflops": tf(ms_fwd_loop)},
        "conv_dgrad": {"ms": ms_dgrad, "tflops": tf(ms_dgrad), "frac_mfma_peak": tf(ms_dgrad) / PEAK_BF16_TFLOPS},
        "conv_wgrad": {"ms": ms_wgrad, "tflops": tf(ms_wgrad), "frac_mfma_peak": tf(ms_wgrad) / PEAK_BF16_TFLOPS},
        "conv_fwd_bwd_kernels_only": {
            "ms": ms_fwd + ms_dgrad + ms_wgrad,
            "tflops": flop_step / ((ms_fwd + ms_dgrad + ms_wgrad) * 1e-3) / 1e12,
            "frac_mfma_peak": flop_step / ((ms_fwd + ms_dgrad + ms_wgrad) * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        },
        "halo_assemble": {"ms": ms_asm, "GBps": gbps(ms_asm), "frac_hbm_peak": gbps(ms_asm) / PEAK_HBM_GBPS, "bytes": halo_bytes},
        "halo_fold": {"ms": ms_fold, "GBps": gbps(ms_fold), "frac_hbm_peak": gbps(ms_fold) / PEAK_HBM_GBPS, "bytes": halo_bytes},
        "conv_dgrad_fused_with_pack_and_fold": {"ms": ms_dgrad_fold, "tflops": tf(ms_dgrad_fold)},
        "halo_fold_border": {"ms": ms_border},
        "halo_assemble_frame": {"ms": ms_frame},
        "conv_fwd_framed": {"ms": ms_fwd_framed, "tflops": tf(ms_fwd_framed)},
        "conv_wgrad_framed_with_bias_grad": {"ms": ms_wgrad_framed, "tflops": tf(ms_wgrad_framed)},
        "conv_transpose_fwd": {"ms": ms_convt_fwd, "tflops": tf(ms_convt_fwd)},
        "conv_transpose_bwd": {"ms": ms_convt_bwd, "tflops": 2 * tf(ms_convt_bwd)},
    }


# --------------------------------------------------------------------------- #
# Launch-only modes for rocprofv3 (``--profile MODE``): each runs a few repetitions of one group of
# kernels and prints no figures, so that a kernel trace or a counter run of the command holds those
# launches and little else.
# --------------------------------------------------------------------------- #
def profile_conv2_attention(reps: int = 3) -> None:
    """Every hot kernel of configuration 2 (the step as the benchmark runs it, then the separate
    operators the fused ones replace) and the attention core of configuration 4, plus a plain device copy
    of known size that calibrates the FETCH_SIZE / WRITE_SIZE counters."""
    from jigsaw_amd import attention as ja
    from jigsaw_amd import conv as jc
    from jigsaw_amd.halo import halo_fold, halo_fold_border_

    dev = torch.device("cuda:0")
    wl = build_conv2_workload(dev)
    buf = conv_step_buffers(wl)
    geom, x, w, gout = wl["geom"], wl["x"], wl["w"], wl["g"]
    x_aug = buf["x_aug"]
    gx_aug = jc.conv_nd_input(x_aug.shape, w, gout)
    gx = torch.empty_like(x)
    copy_dst = torch.empty_like(x)  # calibration copy: reads and writes x.numel() * 2 bytes
    g = torch.Generator(device=dev).manual_seed(0)
    q = (torch.randn(1, 8, 4096, 64, device=dev, generator=g) / 8).bfloat16()
    k = torch.randn(1, 8, 4096, 64, device=dev, generator=g).bfloat16()
    v = torch.randn(1, 8, 4096, 64, device=dev, generator=g).bfloat16()
    dout = torch.randn(1, 8, 4096, 64, device=dev, generator=g).bfloat16()
    acc = torch.zeros(1, 8, 4096, 64, device=dev)
    lse = torch.full((1, 8, 4096), float("-inf"), device=dev)
    out, l = ja.core_forward(q, k, v, 0.125)
    for _ in range(reps):
        copy_dst.copy_(x)
        conv_step(wl, buf)
        # the separate steps the fused ones replace
        jc.conv_nd_input(x_aug.shape, w, gout)
        jc.sum_grad_bias(gout, 2)
        halo_fold(gx_aug, wl["strips_bwd"], geom, out=gx)
        halo_fold_border_(gx, wl["strips_bwd"], geom)
        ja.core_forward(q, k, v, 0.125, out_acc=acc, lse_acc=lse, want_out=False)
        ja.core_backward(dout, q, k, v, out, l, 0.125)
    torch.cuda.synchronize()


def profile_around_attention(reps: int = 3) -> None:
    """The kernels either side of the ring step: the attention core at head size 128 (32 heads, 4096 x 4096
    tokens) and the qkv / output projections with the head split fused in (8 x 4096 tokens, 512 channels, 8 heads)."""
    from jigsaw_amd import attention as ja
    from jigsaw_amd import projection as jp

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(1)
    h, n, d = 32, 4096, 128
    q = (torch.randn(1, h, n, d, device=dev, generator=g) / d**0.5).bfloat16()
    k = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    v = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    dout = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    out, lse = ja.core_forward(q, k, v, d**-0.5)
    bsz, c, heads = 8, 512, 8
    x = torch.randn(bsz, n, c, device=dev, generator=g).bfloat16().requires_grad_()
    w = (torch.randn(3 * c, c, device=dev, generator=g) / c**0.5).bfloat16().requires_grad_()
    b = (0.1 * torch.randn(3 * c, device=dev, generator=g)).bfloat16().requires_grad_()
    wo = (torch.randn(c, c, device=dev, generator=g) / c**0.5).bfloat16()
    o = torch.randn(bsz, heads, n, c // heads, device=dev, generator=g).bfloat16()
    gy = torch.randn(3, bsz, heads, n, c // heads, device=dev, generator=g).bfloat16()
    for _ in range(reps):
        ja.core_forward(q, k, v, d**-0.5)
        ja.core_backward(dout, q, k, v, out, lse, d**-0.5)
        y = jp.qkv_projection(x, w, b, heads)
        torch.autograd.grad(y, (x, w, b), gy)
        jp.heads_projection(o, wo, None)
    torch.cuda.synchronize()


def profile_ring(reps: int = 3) -> None:
    """Configuration 4's ring, forward and backward over the four resident chunks (no hops)."""
    from jigsaw_amd import attention as ja

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    b, h, n, d, P = 1, 8, 4096, 64, 4
    q = (torch.randn(b, h, n, d, device=dev, generator=g) / 8).bfloat16()
    ks = [(torch.randn(b, h, n, d, device=dev, generator=g) / 8).bfloat16() for _ in range(P)]
    vs = [(torch.randn(b, h, n, d, device=dev, generator=g) / 8).bfloat16() for _ in range(P)]
    dout = torch.randn(b, h, n, d, device=dev, generator=g).bfloat16()
    for _ in range(reps):
        out, l = ja.ring_forward(q, ks, vs, d**-0.5)
        ja.ring_backward(dout, q, out, l, ks, vs, d**-0.5)  # one pass over the four chunks
        ja.core_backward(dout, q, ks[0], vs[0], out, l, d**-0.5)  # one chunk by itself, for comparison
    torch.cuda.synchronize()


def profile_swin_block(reps: int = 5) -> None:
    """Forward + backward of one Swin block of configuration 5 (256 x 256 token tile, dim 128, 4 heads,
    8 x 8 windows, shift 4, bf16 autocast; the neighbours' roll slabs are random stand-ins made once)."""
    step = _swin_step(torch.device("cuda:0"))[0]
    for _ in range(reps):
        step()
    torch.cuda.synchronize()


def profile_attention_fp32(reps: int = 3) -> None:
    """The attention core forward + backward on fp32 inputs (8 heads, 4096 x 4096 tokens) at head sizes 64, 128, 32."""
    from jigsaw_amd import attention as ja

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(4)
    for d in (64, 128, 32):
        b, h, n = 1, 8, 4096
        q, k, v, dout = (torch.randn(b, h, n, d, device=dev, generator=g) / 8 for _ in range(4))
        scale = d**-0.5
        for _ in range(reps):
            out, lse = ja.core_forward(q, k, v, scale)
            ja.core_backward(dout, q, k, v, out, lse, scale)
        torch.cuda.synchronize()


def profile_sharded_layernorm(reps: int = 3) -> None:
    """Forward + backward of the channel-sharded LayerNorm on one shard's rows, bf16: 2 ** 18 rows of 256
    channels (configuration 4's local width at a row count that fills the chip), 2 ** 20 rows of 64, and, for
    the kernels that walk a row, 2 ** 18 rows of 132."""
    from jigsaw_amd import layernorm as jl

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(3)
    for rows, cols in ((1 << 18, 256), (1 << 20, 64), (1 << 18, 132)):
        x = torch.randn(rows, cols, device=dev, generator=g).bfloat16().requires_grad_()
        w = torch.ones(cols, device=dev, dtype=torch.bfloat16, requires_grad=True)
        b = torch.zeros(cols, device=dev, dtype=torch.bfloat16, requires_grad=True)
        gout = torch.randn(rows, cols, device=dev, generator=g).bfloat16()
        for _ in range(reps):
            x.grad = w.grad = b.grad = None
            jl.layer_norm(x, w, b, None).backward(gout)
        torch.cuda.synchronize()
        del x, gout
    # the two statistics kernels by themselves, as bench.py's figures time them (inputs in turn, read-only
    # neighbours): in the layer above each runs right behind a kernel that leaves 268 MB of written lines behind
    stats_fwd, stats_bwd, n_turn = ln_statistics_calls(dev, g)
    for _ in range(2 * n_turn):
        stats_fwd()
    for _ in range(2 * n_turn):
        stats_bwd()
    torch.cuda.synchronize()


def profile_conv3d(reps: int = 3) -> None:
    """Configuration 3: pack, assemble, forward, fused dgrad, wgrad, border fold and the separate fold."""
    conv3d_figures(torch.device("cuda:0"), reps)


PROFILE_MODES = {
    "conv2-attention": profile_conv2_attention,
    "around-attention": profile_around_attention,
    "ring": profile_ring,
    "swin-block": profile_swin_block,
    "attention-fp32": profile_attention_fp32,
    "sharded-layernorm": profile_sharded_layernorm,
    "conv3d": profile_conv3d,
}

EXTRA_GROUPS = ("conv2", "attention", "conv3d", "swin", "groupnorm", "projection", "attention-wide")


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--cpu-baseline-only", action="store_true", help="run only the CPU leg and print its JSON object")
    ap.add_argument("--no-extras", action="store_true",
                    help="only the timed steps and the roofline kernel (a kernel trace of this run then "
                    "holds the forward kernel's launches under a name of their own)")
    ap.add_argument("--only", default=None, metavar="GROUPS",
                    help="comma-separated groups of the figures under `extra` to run (default: all): " + ", ".join(EXTRA_GROUPS))
    ap.add_argument("--profile", default=None, choices=sorted(PROFILE_MODES),
                    help="launch one group of kernels a few times and print no figures (for rocprofv3 runs)")
    ns = ap.parse_args()
    if ns.gpus != 1:
        print(
            "bench.py: this build runs one rank's share on ONE GPU and has no collectives; "
            f"--gpus {ns.gpus} is not supported (use --gpus 1).",
            file=sys.stderr,
        )
        return 2
    if ns.cpu_baseline_only:
        print(json.dumps(cpu_baseline()))
        return 0
    groups = set(EXTRA_GROUPS)
    if ns.only is not None:
        groups = {v.strip() for v in ns.only.split(",") if v.strip()}
        if groups - set(EXTRA_GROUPS):
            print(f"bench.py: unknown group(s) {sorted(groups - set(EXTRA_GROUPS))}; known: {', '.join(EXTRA_GROUPS)}", file=sys.stderr)
            return 2
    if ns.no_extras:
        groups = set()
    if ns.profile is not None:
        if not torch.cuda.is_available():
            print("bench.py: no GPU visible; the HIP kernels have no CPU fallback.", file=sys.stderr)
            return 2
        import jigsaw_amd

        jigsaw_amd.load()
        PROFILE_MODES[ns.profile]()
        print(f"bench.py --profile {ns.profile}: done", file=sys.stderr)
        return 0
    # The CPU leg runs first, in a child process of its own, before this process has touched
    # the GPU: it starts further processes (the gloo ranks), and its thread pools and buffers
    # would otherwise stay behind in the process that issues the GPU work.
    cpu = None
    if not ns.no_cpu_baseline:
        import subprocess

        try:
            done = subprocess.run([sys.executable, os.path.abspath(__file__), "--cpu-baseline-only"],
                                  capture_output=True, text=True, timeout=900)
            cpu = json.loads(done.stdout.strip().splitlines()[-1])
        except Exception as exc:
            cpu = {"value": None, "unit": "TFLOP/s", "cores": None, "kind": "port", "sample": f"CPU leg failed: {exc!r}"}
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback.", file=sys.stderr)
        return 2

    import jigsaw_amd

    jigsaw_amd.load()  # fail loudly if the library is not built
    dev = torch.device("cuda:0")
    wl = build_conv2_workload(dev)
    batch, ch, tile = wl["x"].shape[0], wl["x"].shape[1], wl["x"].shape[-1]
    flop_one = 2 * batch * ch * ch * 9 * tile * tile  # fwd = dgrad = wgrad
    flop_step = 3 * flop_one

    # ---- the timed region: W warm-up steps, then exactly K steps
    timed = timed_conv_steps(wl, ns.steps, ns.warmup)
    per_step = timed["per_step"]
    ms_per_step = _median(per_step)
    ms_mean = max(timed["span_ms"], timed["wall_ms"]) / ns.steps  # host-side gaps count too
    if max(per_step) > 2 * ms_per_step:
        worst = max(range(len(per_step)), key=per_step.__getitem__)
        print(f"bench.py: step {worst} took {per_step[worst]:.3f} ms against a median of {ms_per_step:.3f} ms "
              f"(per-kernel brackets of that step: " + ", ".join(f"{k} {v[worst]:.3f}" for k, v in timed["per_kernel"].items()) + ")",
              file=sys.stderr)
    value = flop_step / (ms_per_step * 1e-3) / 1e12

    # ---- per-kernel figures: the three convolution launches of the timed steps (the small weight
    # re-layout and reduction launches that belong to each are inside its bracket), median over the
    # steps; the roofline entry is the DOMINANT one: the longest
    x_aug = timed["buf"]["x_aug"]
    it = max(5, ns.steps)
    ms_kernel = {k: _median(v) for k, v in timed["per_kernel"].items()}
    ms_fwd = ms_kernel["fwd"]
    dominant = max(ms_kernel, key=ms_kernel.get)
    tf = lambda ms: flop_one / (ms * 1e-3) / 1e12  # noqa: E731
    roofline = {
        "kernel": CONV_KERNEL_NAMES[dominant],
        "bound": "mfma",
        "achieved": tf(ms_kernel[dominant]),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": tf(ms_kernel[dominant]) / PEAK_BF16_TFLOPS,
        "traffic": CONV_TRAFFIC_BYTES[dominant],
    }
    extra = {f"conv_{k}_in_step": {"ms": v, "ms_mean": sum(timed["per_kernel"][k]) / ns.steps, "ms_max": max(timed["per_kernel"][k]),
                                   "tflops": tf(v), "frac_mfma_peak": tf(v) / PEAK_BF16_TFLOPS}
             for k, v in ms_kernel.items()}
    del timed
    if "conv2" in groups:
        extra.update(conv2_extras(wl, x_aug, it, flop_one, flop_step, ms_fwd))
    del x_aug
    if "attention" in groups:
        extra.update(attention_figures(dev, max(10, it)))
    if "conv3d" in groups:
        extra.update(conv3d_figures(dev, it))
    if "swin" in groups:
        extra.update(swin_figures(dev, it))
    if "groupnorm" in groups:
        extra.update(groupnorm_figures(dev, it))
    if "projection" in groups:
        extra.update(projection_figures(dev, it))
    if "attention-wide" in groups:
        extra.update(attention_wide_figures(dev, it))

    line = {
        "metric": METRIC,
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": ns.steps,
        "warmup": ns.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_stat": "median of the timed steps' HIP-event brackets",
        "ms_per_step_mean": ms_mean,
        "ms_per_step_max": max(per_step),
        "ms_per_step_min": min(per_step),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "config 2: one rank's 1024x1024 tile of a 2048x2048 domain, batch 8, 64->64 ch, 3x3, pad 1; "
            "halo pack + assemble + conv fwd + dgrad (fused with the halo pack and the own part of the fold) + wgrad (fused with bias-grad) + border fold",
            "flop_per_step": flop_step,
            "frac_mfma_peak": value / PEAK_BF16_TFLOPS,
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
