"""The allocation-free variant of the LayerNorm backward partials, through the C ABI (GPU).

``jg_ln_partial_bwd_static`` keeps its column partials in a device array built into the
library instead of a caller's workspace. Checked against ``jg_ln_partial_bwd`` (bit for bit:
same kernels, same order of additions) on two calls in a row, the second with a smaller
input, so that what the first call left in the shared array cannot leak into the second;
and the size limit is an error, not a fault.
"""

import ctypes

import pytest
import torch

import jigsaw_amd
from jigsaw_amd import _lib

pytestmark = pytest.mark.gpu

DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _call(lib, name, g, xh, w, with_ws):
    rows, cols = g.shape
    dev = g.device
    mean = torch.full((rows,), float("nan"), device=dev)
    dot = torch.full((rows,), float("nan"), device=dev)
    gw = torch.full((cols,), float("nan"), device=dev)
    gb = torch.full((cols,), float("nan"), device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [mean.data_ptr(), dot.data_ptr(), gw.data_ptr(), gb.data_ptr(), g.data_ptr(), xh.data_ptr(), w.data_ptr(),
            rows, cols, DT[g.dtype]]
    if with_ws:
        nbytes = int(lib.jg_ln_bwd_workspace_bytes(rows, cols))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        args += [ws.data_ptr(), nbytes]
    rc = getattr(lib, name)(*args, stream)
    assert rc == 0, lib.jg_last_error().decode()
    torch.cuda.synchronize()
    return mean, dot, gw, gb


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_matches_workspace_variant_twice(dtype, dev):
    lib = jigsaw_amd.load()
    torch.manual_seed(0)
    # first the shape of the ViT configuration (4096 rows, 256 local columns), then a smaller,
    # ragged one that reuses the front of the same scratch array
    for rows, cols in ((4096, 256), (77, 100)):
        print(f"jg_ln_partial_bwd_static rows={rows} cols={cols} {dtype}", flush=True)
        g = torch.randn(rows, cols, device=dev).to(dtype)
        xh = torch.randn(rows, cols, device=dev).to(dtype)
        w = (1 + 0.2 * torch.randn(cols, device=dev)).to(dtype)
        want = _call(lib, "jg_ln_partial_bwd", g, xh, w, with_ws=True)
        got = _call(lib, "jg_ln_partial_bwd_static", g, xh, w, with_ws=False)
        for name, a, b in zip(("mean_gxn", "dot", "gw", "gb"), got, want):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), f"{name} differs at {rows} x {cols}"
        # and against plain torch, so that both being wrong alike would show
        gf, xf, wf = g.float(), xh.float(), w.float()
        gxn = (gf * wf).to(dtype).float()
        torch.testing.assert_close(got[0], gxn.mean(-1), atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(got[2], (gf * xf).sum(0), atol=2e-2, rtol=1e-3)
        torch.testing.assert_close(got[3], gf.sum(0), atol=2e-2, rtol=1e-3)


def test_static_scratch_rejects_what_does_not_fit(dev):
    lib = jigsaw_amd.load()
    rows, cols = 8192, 2048  # 1024 blocks x 2 x 2048 x 4 B = 16 MiB of partials
    g = torch.zeros(rows, cols, device=dev)
    mean = torch.zeros(rows, device=dev)
    gw = torch.zeros(cols, device=dev)
    rc = lib.jg_ln_partial_bwd_static(mean.data_ptr(), mean.data_ptr(), gw.data_ptr(), gw.data_ptr(), g.data_ptr(),
                                      g.data_ptr(), gw.data_ptr(), rows, cols, 0, None)
    assert rc == -4 and b"built-in scratch" in lib.jg_last_error()
    # without column sums nothing is staged, so any size is fine
    rc = lib.jg_ln_partial_bwd_static(mean.data_ptr(), mean.data_ptr(), None, None, g.data_ptr(), g.data_ptr(),
                                      gw.data_ptr(), rows, cols, 0, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.jg_last_error().decode()
    torch.cuda.synchronize()
