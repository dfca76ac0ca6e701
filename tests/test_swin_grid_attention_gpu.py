"""The Swin window-attention kernels that work on the token grid itself
(jigsaw_amd.attention.swin_grid_attention: windows addressed in place, relative-position bias and
shift mask formed in the kernel) against plain fp64 attention over explicitly partitioned windows
with an explicit (nW, heads, N, N) bias, built from the pinned oracle helpers (oracle/swin.py).
Tolerance: rel-L2 2e-2 (bf16 operands), the bar of the other bf16 attention tests."""

import pytest
import torch

from helpers import rel_l2
from jigsaw_amd import attention as ja
from jigsaw_amd import swin as js
from jigsaw_amd.conv import TileGroup
from oracle import swin as osw

pytestmark = pytest.mark.gpu


def _reference(q, k, v, table, mask, grid, window):
    """fp64: partition, bias = table[index] (+ mask), softmax attention, un-partition."""
    b, heads, s, d = q.shape
    gh, gw = grid

    def part(t):  # (B, heads, S, d) -> (B, heads, nW, N, d)
        t = t.view(b * heads, gh, gw, d)
        return osw.windows(t, window).view(b, heads, -1, window * window, d)

    qw, kw, vw = part(q), part(k), part(v)
    index = osw.relative_position_index(window)
    bias = table[index.view(-1)].view(window * window, window * window, heads).permute(2, 0, 1)  # (heads, N, N)
    scores = qw @ kw.transpose(-1, -2) * d**-0.5 + bias[None, :, None]
    if mask is not None:
        scores = scores + mask[None, None]
    out = torch.softmax(scores, -1) @ vw
    return osw.unwindows(out.reshape(b * heads, -1, window * window, d), gh, gw, window).reshape(b, heads, s, d)


@pytest.mark.parametrize("grid,heads,shift,tiling", [
    ((16, 24), 4, 0, None),
    ((16, 16), 3, 4, (1, 0, 1, 0)),       # undivided grid: last window row / column mixed
    ((32, 16), 4, 3, (2, 1, 2, 1)),       # the lower right tile of a 2 x 2 tiling
    ((32, 16), 2, 4, (2, 0, 2, 0)),       # the upper left one: no window crosses a border
])
def test_swin_grid_attention_forward_backward(grid, heads, shift, tiling, dev):
    torch.manual_seed(3)
    b, d, window = 2, 32, 8
    gh, gw = grid
    s = gh * gw
    q, k, v, dout = (torch.randn(b, heads, s, d).bfloat16() for _ in range(4))
    table = torch.randn(225, heads) * 0.5
    side = mask = None
    if shift:
        groups = (TileGroup(tiling[0], tiling[1]), TileGroup(tiling[2], tiling[3]))
        side = js.border_sides(gh, gw, window, shift, groups).to(torch.uint8)
        mask = js.shift_mask(gh, gw, window, shift, groups).double()
    qd, kd, vd, td = (t.double().requires_grad_() for t in (q, k, v, table))
    want = _reference(qd, kd, vd, td, mask, grid, window)
    want.backward(dout.double())

    gq, gk, gv = (t.to(dev).requires_grad_() for t in (q, k, v))
    gt = table.to(dev).requires_grad_()
    out = ja.swin_grid_attention(gq, gk, gv, gt, None if side is None else side.to(dev), grid)
    out.backward(dout.to(dev))
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and gt.grad.dtype == torch.float32
    assert rel_l2(out, want) < 2e-2
    for name, got, w in (("dq", gq.grad, qd.grad), ("dk", gk.grad, kd.grad), ("dv", gv.grad, vd.grad), ("dtable", gt.grad, td.grad)):
        assert rel_l2(got, w) < 2e-2, f"{name}: {rel_l2(got, w):.3e}"
    # the table gradient adds up in a fixed order: a second run gives the same bits
    gt2 = table.to(dev).requires_grad_()
    ja.swin_grid_attention(gq.detach(), gk.detach(), gv.detach(), gt2, None if side is None else side.to(dev), grid).backward(dout.to(dev))
    assert torch.equal(gt.grad, gt2.grad)


def test_swin_grid_attention_argument_errors(dev):
    q = torch.zeros(1, 2, 64, 32, device=dev, dtype=torch.bfloat16)
    table = torch.zeros(225, 2, device=dev)
    with pytest.raises(NotImplementedError):
        ja.swin_grid_attention(q.float(), q.float(), q.float(), table, None, (8, 8))
    with pytest.raises(ValueError):
        ja.swin_grid_attention(q, q, q, table[:, :1], None, (8, 8))
    with pytest.raises(ValueError):
        ja.swin_grid_attention(q, q, q, table, torch.zeros(1, 64, device=dev), (8, 8))
