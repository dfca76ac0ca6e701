"""HIP convolution kernels against the oracle (torch CPU operators in fp64) (GPU).

Tolerances (rel-L2 of the whole tensor): fp32 tensors 1e-5 and bf16 tensors 2e-2, as the north-star
states, fp16 tensors 2e-3; the reference's own conv tests use atol/rtol 1e-4 for
y / dx / db and a looser bound for dw (tests/modules/convolution/conv/test_conv2d_multi_spatial.py:207-233).
"""

import itertools

import pytest
import torch

from helpers import conv_geometry, mesh_coords, neighbour, rel_l2
from jigsaw_amd import conv as jc
from jigsaw_amd.halo import halo_pack
from oracle import conv as oc
from oracle import halo as oh

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-3}

PRIM_CASES = [
    # (N, Cin, Cout, in spatial, kernel, stride, padding, dilation)
    (2, 3, 16, (18, 18), (3, 3), (1, 1), (0, 0), (1, 1)),
    (2, 16, 3, (18, 20), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 5, 7, (13, 11), (3, 2), (2, 1), (1, 0), (1, 2)),
    (2, 4, 4, (9, 9), (1, 1), (1, 1), (0, 0), (1, 1)),
    (2, 4, 6, (12, 12), (5, 5), (1, 1), (2, 2), (1, 1)),
    (1, 3, 5, (40,), (3,), (1,), (1,), (1,)),
    (1, 4, 6, (8, 9, 10), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
    (2, 3, 4, (7, 8, 9), (3, 1, 2), (1, 2, 1), (1, 0, 1), (1, 1, 1)),
    (2, 64, 64, (18, 34), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 32, 32, (10, 10, 18), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
    (1, 64, 64, (20, 70), (3, 3), (1, 1), (1, 1), (1, 1)),
    (3, 64, 64, (37, 53), (3, 3), (1, 1), (0, 0), (1, 1)),
    # several stages per workgroup, strips that start in the middle of a workgroup's range
    (2, 64, 64, (260, 131), (3, 3), (1, 1), (0, 0), (1, 1)),
    (2, 32, 32, (6, 70, 130), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
    (1, 32, 64, (131, 200), (3, 3), (1, 1), (1, 1), (1, 1)),
    # row lengths of whole cache lines: the input gradient's tile grid moves so that its staged rows start on
    # a line (an odd distance: staged from one pixel earlier), the first tile column mostly hangs out of the tensor
    (2, 32, 32, (20, 128), (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 64, 64, (35, 192), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 32, 16, (4, 18, 64), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    # weight gradient: several stages per workgroup with column strips of unequal cost (windows that stick out
    # across W, a last strip with fewer columns), odd padding across even rows (staged one pixel early)
    (2, 64, 64, (150, 330), (3, 3), (1, 1), (1, 1), (1, 1)),
    (2, 32, 32, (140, 200), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 32, 32, (5, 40, 136), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    # weight gradient without padding over whole stages (even rows, 64-column strips), every window inside x: the
    # kernel without the border path, whose stage loop loads and stores without conditions. One stage per
    # workgroup, two or three (the load cursor stops at the last one), each channel blocking
    (2, 64, 64, (4, 66), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 64, 64, (1030, 66), (3, 3), (1, 1), (0, 0), (1, 1)),
    (2, 64, 64, (8, 130), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 32, 64, (262, 130), (3, 3), (1, 1), (0, 0), (1, 1)),
    (2, 64, 32, (6, 66), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 32, 32, (518, 66), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 32, 32, (5, 260, 66), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
    # channel counts beyond one group of LDS-resident weights, and produced channels that are
    # not a multiple of the 32-row MFMA tile (padded with zero weight rows, not stored)
    (1, 128, 128, (20, 70), (3, 3), (1, 1), (1, 1), (1, 1)),
    (2, 16, 3, (37, 66), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 48, 80, (33, 40), (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 256, 64, (18, 34), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 96, 32, (5, 18, 34), (3, 3, 3), (1, 1, 1), (1, 0, 1), (1, 1, 1)),
    (1, 80, 16, (4, 20, 36), (3, 3, 3), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
    # contraction channels that are not a multiple of the 16-channel MFMA step (first / last layers)
    (2, 69, 64, (37, 66), (3, 3), (1, 1), (0, 0), (1, 1)),
    (1, 64, 69, (20, 70), (3, 3), (1, 1), (1, 1), (1, 1)),
    (2, 20, 24, (5, 18, 34), (3, 3, 3), (1, 1, 1), (1, 0, 1), (1, 1, 1)),
    # non-overlapping kernels (patch embeddings, 1 x 1): a GEMM over the patches in bf16
    (2, 8, 16, (16, 24), (4, 4), (4, 4), (0, 0), (1, 1)),
    (2, 16, 32, (9, 11), (1, 1), (1, 1), (0, 0), (1, 1)),
    (2, 8, 8, (17, 19), (4, 4), (4, 4), (0, 0), (1, 1)),
    (1, 4, 8, (4, 8, 10), (2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
    (3, 72, 264, (64, 48), (8, 8), (8, 8), (0, 0), (1, 1)),
    (2, 16, 32, (20, 36), (2, 2), (2, 2), (0, 0), (1, 1)),
    # extents 1 or 3 at stride 1: embedded in the 3 x 3 (x 3) MFMA kernels
    (2, 64, 64, (20, 70), (1, 1), (1, 1), (0, 0), (1, 1)),
    (1, 16, 24, (19, 33), (1, 3), (1, 1), (0, 1), (1, 1)),
    (2, 8, 5, (12, 40), (3, 1), (1, 1), (1, 0), (1, 1)),
    (1, 16, 16, (5, 10, 34), (1, 1, 1), (1, 1, 1), (0, 0, 0), (1, 1, 1)),
    (1, 8, 8, (6, 9, 20), (3, 1, 3), (1, 1, 1), (1, 0, 0), (1, 1, 1)),
    # strided 3 x 3 (down-sampling): the stride-1 kernels, sampled / zero-stuffed
    (2, 16, 32, (33, 40), (3, 3), (2, 2), (1, 1), (1, 1)),
    (1, 8, 8, (20, 31), (3, 3), (2, 3), (0, 1), (1, 1)),
    (1, 8, 16, (7, 12, 18), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),
    (2, 8, 8, (16, 16), (1, 1), (2, 2), (0, 0), (1, 1)),
    # dilated 3-tap kernels whose padding is a multiple of the dilation: the residue images as batch
    # entries of the undilated MFMA kernels (extents that the dilation does and does not divide)
    (2, 32, 64, (33, 47), (3, 3), (1, 1), (2, 3), (2, 3)),
    (1, 64, 64, (40, 64), (3, 3), (1, 1), (0, 0), (2, 2)),
    (2, 16, 8, (21, 30), (3, 3), (1, 1), (4, 0), (2, 1)),
    (1, 8, 16, (9, 3), (3, 1), (1, 1), (4, 0), (4, 5)),
    (1, 32, 32, (6, 19, 34), (3, 3, 3), (1, 1, 1), (1, 2, 2), (1, 2, 2)),
    (2, 16, 32, (33, 40), (3, 3), (2, 2), (2, 2), (2, 2)),   # strided and dilated
    (1, 4, 6, (17, 23), (3, 3), (1, 1), (1, 1), (2, 2)),     # padding not a multiple: the direct kernels
    # more than three taps on an axis: tap blocks of three as channel blocks of a three-tap layer
    (1, 16, 32, (20, 33), (5, 5), (1, 1), (2, 2), (1, 1)),
    (2, 8, 8, (15, 18), (7, 7), (1, 1), (3, 3), (1, 1)),
    (1, 8, 16, (12, 14), (4, 4), (2, 2), (1, 1), (1, 1)),
    (1, 6, 4, (13, 16), (1, 5), (1, 1), (0, 0), (1, 1)),
    (2, 4, 6, (11, 9), (5, 2), (1, 1), (4, 1), (1, 1)),
    (1, 4, 6, (6, 9, 10), (5, 3, 3), (1, 1, 1), (2, 1, 1), (1, 1, 1)),
    (1, 3, 5, (14, 14), (7, 7), (2, 2), (3, 3), (1, 1)),     # a 7 x 7 stem at stride 2
    # grouped layers (ninth entry: groups), depthwise among them: the direct kernels
    (2, 8, 12, (13, 17), (3, 3), (1, 1), (1, 1), (1, 1), 4),
    (1, 32, 32, (20, 22), (3, 3), (1, 1), (1, 1), (1, 1), 32),
    (2, 6, 9, (11, 14), (3, 5), (2, 1), (1, 2), (1, 2), 3),
    (1, 16, 16, (5, 9, 10), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 2),
    (2, 64, 64, (18, 34), (3, 3), (1, 1), (0, 0), (1, 1), 2),   # a shape the MFMA kernels would take ungrouped
    (1, 12, 8, (30,), (5,), (1,), (2,), (1,), 4),
    # dilated kernels of more than three taps (residue images on the tap-block route), a padding that is no multiple of
    # the dilation (the remainder as a rim of zeros around the input), two taps an axis (a block with a zero tap in front)
    (2, 3, 5, (15, 18), (5, 3), (1, 1), (4, 2), (2, 2)),
    (1, 4, 6, (13, 17), (3, 3), (1, 1), (1, 3), (2, 2)),
    (2, 5, 4, (14, 15), (3, 3), (2, 2), (1, 1), (2, 3)),
    (1, 6, 7, (9, 11), (2, 2), (1, 1), (1, 0), (1, 1)),
    (1, 3, 4, (6, 7, 8), (1, 2, 2), (1, 1, 1), (0, 1, 1), (1, 1, 1)),
    (2, 4, 4, (12, 12), (2, 2), (1, 1), (0, 0), (2, 2)),
    # groups of at least 8 channels a side: each group as an ungrouped layer of its own (matrix cores, and the routes above)
    (2, 48, 32, (20, 22), (3, 3), (2, 2), (1, 1), (1, 1), 2),
    (1, 32, 64, (17, 19), (5, 5), (1, 1), (2, 2), (1, 1), 4),
    (1, 24, 24, (6, 10, 12), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 2, 2), 3),
]


def _pid(c):
    name = "n{}_ci{}_co{}_in{}_k{}_s{}_p{}_d{}".format(c[0], c[1], c[2], *["x".join(map(str, v)) for v in c[3:8]])
    return name + (f"_g{c[8]}" if len(c) > 8 else "")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", PRIM_CASES, ids=_pid)
def test_conv_primitives_match_oracle(case, dtype, dev):
    N, cin, cout, insp, k, s, p, d = case[:8]
    groups = case[8] if len(case) > 8 else 1
    torch.manual_seed(0)
    x = torch.randn(N, cin, *insp).to(dtype)
    fan_in = cin // groups * int(torch.tensor(k).prod())
    w = ((torch.rand(cout, cin // groups, *k) * 2 - 1) / fan_in**0.5).to(dtype)
    b = (torch.randn(cout) * 0.1).to(dtype)
    xd, wd, bd = x.double(), w.double(), b.double()
    y_want = oc.forward(xd, wd, bd, s, p, d, groups)
    g = torch.randn_like(y_want).to(dtype)
    gd = g.double()
    gx_want = oc.dgrad(x.shape, wd, gd, s, p, d, groups)
    gw_want = oc.wgrad(xd, w.shape, gd, s, p, d, groups)
    gb_want = oc.grad_bias(gd, len(k))

    xg, wg, bg, gg = x.to(dev), w.to(dev), b.to(dev), g.to(dev)
    kw = dict(stride=s, padding=p, dilation=d, groups=groups)
    y = jc.conv_nd(xg, wg, bg, **kw)
    assert y.dtype == dtype and y.shape == y_want.shape
    assert rel_l2(y, y_want) < TOL[dtype], f"fwd rel-L2 {rel_l2(y, y_want):.3e}"
    y0 = jc.conv_nd(xg, wg, None, **kw)
    assert rel_l2(y0, oc.forward(xd, wd, None, s, p, d, groups)) < TOL[dtype]
    gx = jc.conv_nd_input(x.shape, wg, gg, **kw)
    assert rel_l2(gx, gx_want) < TOL[dtype], f"dgrad rel-L2 {rel_l2(gx, gx_want):.3e}"
    gw = jc.conv_nd_weight(xg, w.shape, gg, **kw)
    assert gw.shape == w.shape
    assert rel_l2(gw, gw_want) < TOL[dtype], f"wgrad rel-L2 {rel_l2(gw, gw_want):.3e}"
    gb = jc.sum_grad_bias(gg, len(k))
    assert rel_l2(gb, gb_want) < TOL[dtype], f"bias grad rel-L2 {rel_l2(gb, gb_want):.3e}"
    # both gradients from one pass over g (falls back to the two kernels where not covered)
    gw2, gb2 = jc.conv_nd_weight(xg, w.shape, gg, with_bias_grad=True, **kw)
    assert torch.equal(gw2, gw)
    assert gb2.dtype == dtype and rel_l2(gb2, gb_want) < TOL[dtype], f"fused bias grad rel-L2 {rel_l2(gb2, gb_want):.3e}"


def test_partial_channel_step_ignores_what_lies_behind_the_last_channel(dev):
    """3 input channels fill 3 of the 16 slots of an MFMA step; the slots behind them are read
    from whatever follows in memory (the next batch entry) and must not reach the result:
    batch entry 1 is all NaN, batch entry 0 must still match the oracle (and stay finite)."""
    torch.manual_seed(3)
    x = torch.randn(2, 3, 40, 70).bfloat16()
    x[1] = float("nan")
    w = ((torch.rand(16, 3, 3, 3) * 2 - 1) / 27**0.5).bfloat16()
    y = jc.conv_nd(x.to(dev), w.to(dev), None)
    assert torch.isfinite(y[0]).all() and torch.isnan(y[1]).all()
    assert rel_l2(y[0:1], oc.forward(x[0:1].double(), w.double(), None, (1, 1), (0, 0), (1, 1))) < TOL[torch.bfloat16]
    g = torch.randn(2, 3, 38, 68).bfloat16()  # gradient of a 16 -> 3 layer: dgrad contracts over 3 channels
    g[1] = float("nan")
    wt = ((torch.rand(3, 16, 3, 3) * 2 - 1) / 12).bfloat16()
    gx = jc.conv_nd_input((2, 16, 40, 70), wt.to(dev), g.to(dev))
    assert torch.isfinite(gx[0]).all()
    assert rel_l2(gx[0:1], oc.dgrad((1, 16, 40, 70), wt.double(), g[0:1].double(), (1, 1), (0, 0), (1, 1))) < TOL[torch.bfloat16]


def test_conv_argument_errors(dev):
    x = torch.zeros(1, 4, 8, 8, device=dev)
    w = torch.zeros(4, 4, 3, 3, device=dev)
    with pytest.raises(NotImplementedError):
        jc.conv_nd(x, w, padding="same")
    with pytest.raises(RuntimeError):  # 4 input channels against a weight that takes 4 per group, two groups
        jc.conv_nd(x, w, groups=2)
    with pytest.raises(ValueError):
        jc.conv_nd(x, w, groups=3)
    with pytest.raises(RuntimeError):
        jc.conv_nd(x, w.bfloat16())
    with pytest.raises(RuntimeError):
        jc.conv_nd(x[:, :3], w)
    with pytest.raises(RuntimeError):
        jc.conv_nd(x.cpu(), w.cpu())
    with pytest.raises(RuntimeError):
        jc.conv_nd(x[:, :, :2, :2], w)


class TableExchange:
    """HaloExchange stand-in on one GPU: the strips the neighbours would send are
    computed beforehand (by packing the neighbours' tensors) and handed over."""

    def __init__(self, fwd, bwd):
        self.fwd, self.bwd = fwd, bwd
        self.sent_fwd = self.sent_bwd = None

    def forward(self, send):
        self.sent_fwd = send
        return self.fwd

    def backward(self, send):
        self.sent_bwd = send
        return self.bwd


def _recv_tables(tensors, geoms, mesh, from_padded):
    """For every rank: offset -> strip received from the neighbour at that offset."""
    ns = len(mesh)
    out = {}
    for c in mesh_coords(mesh):
        tab = {}
        for o in itertools.product((-1, 0, 1), repeat=ns):
            nb = neighbour(c, o, mesh) if any(o) else None
            if nb is None:
                continue
            back = tuple(-v for v in o)
            tab[o] = halo_pack(tensors[nb], geoms[nb], from_padded=from_padded, present=[back])[back]
        out[c] = tab
    return out


DIST_CASES = [
    # mesh, local spatial, N, Cin, Cout, kernel, padding, dtype
    ((2, 2), (32, 32), 2, 3, 16, (3, 3), (1, 1), torch.float32),
    ((2, 2), (32, 32), 2, 16, 3, (3, 3), (1, 1), torch.float32),
    # the reference's CPU-runnable configuration at its real size: 2 x 2 mesh of 256 x 256 tiles, batch 4, fp32
    ((2, 2), (256, 256), 4, 3, 16, (3, 3), (1, 1), torch.float32),
    ((2, 2), (256, 256), 4, 16, 3, (3, 3), (1, 1), torch.float32),
    ((3, 3), (8, 12), 1, 4, 5, (5, 3), (2, 1), torch.float32),
    ((2, 1), (16, 20), 2, 4, 4, (3, 3), (1, 1), torch.float32),
    ((2, 2), (32, 64), 1, 64, 64, (3, 3), (1, 1), torch.bfloat16),
    ((2, 2, 2), (8, 8, 16), 1, 32, 32, (3, 3, 3), (1, 1, 1), torch.bfloat16),
    ((2, 2, 2), (6, 6, 6), 1, 3, 4, (3, 3, 3), (1, 1, 1), torch.float32),
    # strided / dilated halos (needed_input_span with s > 1, d > 1): one-sided and 2-wide halos
    ((2, 2), (8, 12), 2, 4, 6, (3, 3), (1, 1), torch.float32, (2, 2), (1, 1)),
    ((3, 2), (8, 10), 1, 3, 5, (3, 3), (2, 2), torch.float32, (1, 1), (2, 2)),
    ((2, 2), (16, 32), 1, 32, 32, (3, 3), (1, 2), torch.bfloat16, (2, 1), (1, 2)),
    ((2, 1, 2), (4, 6, 8), 1, 2, 3, (3, 3, 3), (1, 1, 2), torch.float32, (2, 1, 1), (1, 1, 2)),
    # need spans that drift against the tiles (halo.py:49-63 with out_local * stride != n): the widths change from rank to rank
    ((2, 2), (16, 20), 2, 4, 6, (3, 3), (0, 0), torch.float32),                    # no padding: (0, 1) and (1, 0)
    ((4, 2), (6, 12), 1, 3, 5, (5, 3), (0, 1), torch.float32),                     # four ranks: (r, 3 - r)
    ((2, 2), (8, 8), 1, 3, 4, (6, 6), (0, 0), torch.float32, (2, 2), (1, 1)),      # strided and drifting
    ((2, 2), (16, 32), 1, 32, 32, (3, 3), (0, 0), torch.bfloat16),                 # MFMA path, fused fold, framed forward
    ((2, 1, 2), (4, 6, 8), 1, 2, 3, (3, 3, 5), (0, 1, 1), torch.float32),
    # grouped layers (eleventh entry: groups) through the distributed functions
    ((2, 2), (8, 12), 2, 6, 9, (3, 3), (1, 1), torch.float32, (1, 1), (1, 1), 3),
    ((2, 2), (16, 32), 1, 32, 32, (3, 3), (1, 1), torch.bfloat16, (1, 1), (1, 1), 32),
    ((2, 2), (16, 32), 2, 32, 48, (3, 3), (1, 1), torch.bfloat16, (1, 1), (1, 1), 2),   # 16 -> 24 channels a group: each group on the matrix cores
]


@pytest.mark.parametrize("case", DIST_CASES, ids=lambda c: f"mesh{'x'.join(map(str, c[0]))}_{c[3]}to{c[4]}_{str(c[7]).split('.')[-1]}" + (f"_s{''.join(map(str, c[8]))}_d{''.join(map(str, c[9]))}" if len(c) > 8 else "") + (f"_g{c[10]}" if len(c) > 10 else ""))
def test_distributed_conv_matches_global_conv(case, dev):
    """The reference's parity method: every rank's y / dx and the summed dw / db equal
    the serial conv on the gathered tensor (test_conv2d_multi_spatial.py:73-233)."""
    # bf16 cases also take the framed forward (only the frame of the padded tile is built)
    _run_mesh_case(case, dev, framed=case[7] == torch.bfloat16, autocast=None)


@pytest.mark.parametrize("framed", [False, True], ids=["assembled", "framed"])
@pytest.mark.parametrize("case", [
    ((2, 2), (32, 64), 1, 64, 64, (3, 3), (1, 1), torch.float32),
    ((2, 2, 2), (8, 8, 16), 1, 32, 32, (3, 3, 3), (1, 1, 1), torch.float32),
], ids=["2d", "3d"])
def test_distributed_conv_under_autocast(case, framed, dev):
    """fp32 leaves under bf16 autocast: the forward casts x / w / b down
    (_core/autocast.py:44-66, functional.py:53), the backward runs outside autocast in the
    weight's dtype on the saved bf16 padded tile (functional.py:126-129). Gradients come
    back in the leaves' dtype. Bar: bf16 (the forward's operands are rounded to it)."""
    _run_mesh_case(case, dev, framed=framed, autocast=torch.bfloat16)


def _run_mesh_case(case, dev, framed, autocast):
    mesh, n, N, cin, cout, k, p, dtype = case[:8]
    ns = len(mesh)
    s, d = (case[8], case[9]) if len(case) > 8 else ((1,) * ns, (1,) * ns)
    conv_groups = case[10] if len(case) > 10 else 1
    torch.manual_seed(0)
    gshape = tuple(a * b for a, b in zip(n, mesh))
    X = torch.randn(N, cin, *gshape).to(dtype)
    fan_in = cin // conv_groups * int(torch.tensor(k).prod())
    W = ((torch.rand(cout, cin // conv_groups, *k) * 2 - 1) / fan_in**0.5).to(dtype)
    B = (torch.randn(cout) * 0.1).to(dtype)
    Xd = X.double().requires_grad_()
    Wd = W.double().requires_grad_()
    Bd = B.double().requires_grad_()
    Y = oc.forward(Xd, Wd, Bd, s, p, d, conv_groups)
    G = torch.randn_like(Y).to(dtype)
    Y.backward(G.double())

    tiles = {c: t.to(dev) for c, t in oh.split_global(X, mesh).items()}
    gtiles = {c: t.to(dev) for c, t in oh.split_global(G, mesh).items()}
    geoms = {c: conv_geometry(n, mesh, c, k, s, p, d) for c in tiles}
    if autocast is not None:
        # the strips travel in the autocast dtype; the upstream gradient arrives rounded to it
        fwd_tabs = _recv_tables({c: t.to(autocast) for c, t in tiles.items()}, geoms, mesh, from_padded=False)
        gtiles = {c: t.to(autocast).to(dtype) for c, t in gtiles.items()}
    else:
        fwd_tabs = _recv_tables(tiles, geoms, mesh, from_padded=False)
    Wg, Bg = W.to(dev), B.to(dev)

    # pass 1: forward of every rank, and the padded dgrad every rank will send from
    cfgs, outs, leaves, gx_need = {}, {}, {}, {}
    for c in mesh_coords(mesh):
        cfgs[c] = jc.HipConvNdConfig.for_rank(ns, Bg, TableExchange(fwd_tabs[c], None), groups=conv_groups, framed=framed)
        groups = tuple(jc.TileGroup(mesh[a], c[a]) for a in range(ns))
        xl = tiles[c].clone().requires_grad_()
        wl, bl = Wg.clone().requires_grad_(), Bg.clone().requires_grad_()
        with torch.autocast("cuda", dtype=autocast or torch.bfloat16, enabled=autocast is not None):
            y, x_aug = jc._ConvNd.apply(xl, wl, bl, s, p, d, groups, None, cfgs[c])
        outs[c], leaves[c] = y, (xl, wl, bl)
        assert not x_aug.requires_grad
        assert y.dtype == (autocast or dtype) and x_aug.dtype == (autocast or dtype)
        lp = oh.local_padding(p, mesh)
        gx_need[c] = jc.conv_nd_input(x_aug.shape, Wg, gtiles[c], stride=s, padding=lp, dilation=d, groups=conv_groups)
    bwd_tabs = _recv_tables(gx_need, geoms, mesh, from_padded=True)

    # pass 2: backward of every rank
    gw_sum = torch.zeros_like(W, dtype=torch.float64)
    gb_sum = torch.zeros_like(B, dtype=torch.float64)
    tol = TOL[autocast or dtype]
    for c in mesh_coords(mesh):
        cfgs[c].halo_exchange.bwd = bwd_tabs[c]
        outs[c].backward(gtiles[c].to(outs[c].dtype))
        xl, wl, bl = leaves[c]
        assert xl.grad.dtype == dtype and wl.grad.dtype == dtype and bl.grad.dtype == dtype
        sl = (slice(None), slice(None)) + tuple(slice(c[a] * n[a], (c[a] + 1) * n[a]) for a in range(ns))
        no = tuple(Y.shape[2 + a] // mesh[a] for a in range(ns))  # output rows per rank
        so = (slice(None), slice(None)) + tuple(slice(c[a] * no[a], (c[a] + 1) * no[a]) for a in range(ns))
        assert rel_l2(outs[c], Y.detach()[so]) < tol, f"y of rank {c}: {rel_l2(outs[c], Y.detach()[so]):.3e}"
        assert rel_l2(xl.grad, Xd.grad[sl]) < tol, f"dx of rank {c}: {rel_l2(xl.grad, Xd.grad[sl]):.3e}"
        gw_sum += wl.grad.double().cpu()
        gb_sum += bl.grad.double().cpu()
    # replicated weights: gradients are summed over the spatial ranks (parallel/_sync.py:33-46)
    assert rel_l2(gw_sum, Wd.grad) < tol, f"dw: {rel_l2(gw_sum, Wd.grad):.3e}"
    assert rel_l2(gb_sum, Bd.grad) < tol, f"db: {rel_l2(gb_sum, Bd.grad):.3e}"


GENERAL_SPAN_CASES = [
    # mesh, local spatial, N, Cin, Cout, kernel, padding, dtype, stride, dilation: need spans that leave out owned
    # rows or reach past the adjacent rank (halo.py:49-63, 134-154): one split axis at a time
    ((2, 2), (9, 9), 2, 3, 4, (3, 3), (0, 0), torch.float32, (2, 2), (1, 1)),
    ((3, 2), (2, 8), 1, 4, 5, (7, 3), (3, 1), torch.float32, (1, 1), (1, 1)),
    ((4, 1), (3, 10), 2, 2, 3, (9, 3), (4, 1), torch.float32, (1, 1), (1, 1)),
    ((3, 2), (2, 16), 1, 16, 16, (3, 3), (3, 1), torch.bfloat16, (1, 1), (3, 1)),
    ((2, 3, 1), (4, 2, 5), 1, 2, 3, (5, 7, 3), (2, 3, 1), torch.float32, (1, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("case", GENERAL_SPAN_CASES, ids=lambda c: "mesh" + "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[5])) + "_" + str(c[7]).split(".")[-1])
def test_distributed_conv_with_general_spans(case, dev):
    """``conv_halo_nway`` and ``conv_halo_nway_backward`` on every rank of the mesh (in lockstep, one thread a rank)
    where the need spans do not fit the strip exchange: y, dx of every rank and the summed dw, db against the
    serial conv on the gathered tensor (the parity method of test_conv2d_multi_spatial.py:73-233). The two
    functions are called directly: the autograd engine runs every rank's backward node on its one device thread,
    where ranks that wait for each other cannot meet."""
    from helpers import LockstepMesh
    from jigsaw_amd.halo import spans_fit_the_strips

    mesh, n, N, cin, cout, k, p, dtype, s, d = case
    ns = len(mesh)
    assert not spans_fit_the_strips(n, k, s, p, d, mesh)
    torch.manual_seed(1)
    gshape = tuple(a * b for a, b in zip(n, mesh))
    X = torch.randn(N, cin, *gshape).to(dtype)
    W = ((torch.rand(cout, cin, *k) * 2 - 1) / (cin * int(torch.tensor(k).prod())) ** 0.5).to(dtype)
    B = (torch.randn(cout) * 0.1).to(dtype)
    Xd, Wd, Bd = X.double().requires_grad_(), W.double().requires_grad_(), B.double().requires_grad_()
    Y = oc.forward(Xd, Wd, Bd, s, p, d)
    G = torch.randn_like(Y).to(dtype)
    Y.backward(G.double())
    tiles = oh.split_global(X, mesh)
    gtiles = oh.split_global(G, mesh)
    lock = LockstepMesh(mesh)

    def rank(c, exchange):
        cfg = jc.HipConvNdConfig.for_rank(ns, B.to(dev), exchange)
        groups = tuple(jc.TileGroup(mesh[a], c[a]) for a in range(ns))
        xl, wl, bl = tiles[c].to(dev), W.to(dev), B.to(dev)
        y, x_aug = jc.conv_halo_nway(xl, wl, bl, s, p, d, groups, None, cfg)
        gx, gw, gb = jc.conv_halo_nway_backward(gtiles[c].to(dev), x_aug, wl, s, p, d, n, groups, None, cfg, need=(True, True, True))
        return y.cpu(), gx.cpu(), gw.double().cpu(), gb.double().cpu()

    got = lock.run(rank)
    tol = TOL[dtype]
    gw_sum, gb_sum = torch.zeros_like(Wd), torch.zeros_like(Bd)
    for c in mesh_coords(mesh):
        y, gx, gw, gb = got[c]
        sl = (slice(None), slice(None)) + tuple(slice(c[a] * n[a], (c[a] + 1) * n[a]) for a in range(ns))
        no = tuple(Y.shape[2 + a] // mesh[a] for a in range(ns))
        so = (slice(None), slice(None)) + tuple(slice(c[a] * no[a], (c[a] + 1) * no[a]) for a in range(ns))
        assert rel_l2(y, Y.detach()[so]) < tol, f"y of rank {c}: {rel_l2(y, Y.detach()[so]):.3e}"
        assert rel_l2(gx, Xd.grad[sl]) < tol, f"dx of rank {c}: {rel_l2(gx, Xd.grad[sl]):.3e}"
        gw_sum += gw
        gb_sum += gb
    assert rel_l2(gw_sum, Wd.grad) < tol and rel_l2(gb_sum, Bd.grad) < tol
    # the exchange ran once per split axis and direction on every rank, forward first to last, backward last to first
    per_rank = [call for call in lock.calls if call[0] == (0,) * ns]
    split = [a for a in range(ns) if mesh[a] > 1]
    assert [(a, b) for _, a, b, _ in per_rank] == [(a, False) for a in split] + [(a, True) for a in reversed(split)]


def test_frame_without_its_tile_is_refused(dev):
    """A caller that keeps only ``x_aug`` (as the reference's own autograd function does)
    cannot take the weight gradient from a frame: the backward says so instead of
    reading the undefined interior."""
    torch.manual_seed(0)
    mesh, n = (2, 2), (32, 64)
    X = torch.randn(1, 64, 64, 128).bfloat16()
    tiles = {c: t.to(dev) for c, t in oh.split_global(X, mesh).items()}
    geoms = {c: conv_geometry(n, mesh, c, (3, 3), (1, 1), (1, 1), (1, 1)) for c in tiles}
    tabs = _recv_tables(tiles, geoms, mesh, from_padded=False)
    c = (0, 1)
    cfg = jc.HipConvNdConfig.for_rank(2, None, TableExchange(tabs[c], {}), framed=True)
    groups = tuple(jc.TileGroup(mesh[a], c[a]) for a in range(2))
    w = (torch.randn(64, 64, 3, 3) / 24).bfloat16().to(dev)
    y, x_aug = jc.conv_halo_nway(tiles[c], w, None, (1, 1), (1, 1), (1, 1), groups, None, cfg)
    with pytest.raises(RuntimeError, match="x_tile"):
        jc.conv_halo_nway_backward(torch.ones_like(y), x_aug, w, (1, 1), (1, 1), (1, 1), n, groups, None, cfg)


def test_first_layer_skips_dgrad(dev):
    """needs_input_grad gating (functional.py:131-148): no input grad -> no dgrad, no fold."""
    cfg = jc.HipConvNdConfig.for_rank(2, None, TableExchange({}, {}))
    x = torch.randn(1, 3, 8, 8, device=dev)
    w = torch.randn(4, 3, 3, 3, device=dev, requires_grad=True)
    groups = (jc.TileGroup(1, 0), jc.TileGroup(1, 0))
    y, _ = jc._ConvNd.apply(x, w, None, (1, 1), (1, 1), (1, 1), groups, None, cfg)
    y.sum().backward()
    assert w.grad is not None and cfg.halo_exchange.sent_bwd is None


def test_string_padding_is_rejected(dev):
    cfg = jc.HipConvNdConfig.for_rank(2, None, TableExchange({}, {}))
    x = torch.randn(1, 3, 8, 8, device=dev)
    w = torch.randn(4, 3, 3, 3, device=dev)
    with pytest.raises(NotImplementedError):
        jc.conv_halo_nway(x, w, None, (1, 1), "same", (1, 1), (None, None), None, cfg)


FUSED_CASES = [
    # size, lo, hi, conv padding on the padded tile, N, channels, strips that exist
    ((32, 64), (1, 1), (1, 1), (0, 0), 2, 64, "all"),
    ((40, 72), (1, 1), (1, 1), (0, 0), 1, 64, "some"),
    ((24, 40), (0, 2), (2, 0), (0, 0), 1, 32, "all"),
    ((16, 96), (1, 0), (1, 0), (0, 1), 1, 64, "all"),     # W axis not split: the conv pads it itself
    ((48, 128), (1, 1), (1, 1), (0, 0), 2, 64, "all"),    # rows of g are whole cache lines: the tile grid is shifted
    ((20, 192), (1, 1), (1, 1), (0, 0), 1, 32, "some"),
    ((8, 8, 16), (1, 1, 1), (1, 1, 1), (0, 0, 0), 1, 32, "all"),
    ((6, 10, 24), (1, 0, 1), (1, 0, 1), (0, 1, 0), 1, 32, "some"),
]


@pytest.mark.parametrize("case", FUSED_CASES, ids=lambda c: f"{'x'.join(map(str, c[0]))}_lo{''.join(map(str, c[1]))}_hi{''.join(map(str, c[2]))}")
def test_fused_dgrad_fold_has_the_bits_of_the_three_steps(case, dev):
    """conv_nd_input_fold + halo_fold_border_ == conv_nd_input + halo_pack + halo_fold, bit for bit."""
    from jigsaw_amd.halo import HaloGeometry, halo_fold, halo_fold_border_

    size, lo, hi, pad, N, ch, which = case
    ns = len(size)
    geom = HaloGeometry(size, lo, hi)
    torch.manual_seed(3)
    k = (3,) * ns
    out_sp = tuple(geom.padded[a] + 2 * pad[a] - 2 for a in range(ns))
    w = ((torch.rand(ch, ch, *k, device=dev) * 2 - 1) / (ch * 3**ns) ** 0.5).bfloat16()
    g = torch.randn(N, ch, *out_sp, device=dev).bfloat16()
    g[0, 0].zero_()          # exact zeros: the fold clears the sign of -0.0
    g[0, 1] = -g[0, 1].abs() * 1e-30
    offs = [o for o in geom.offsets() if all(geom.strip_extent(o, "fold")[a] > 0 for a in range(ns))]
    if which == "some":
        offs = offs[::2]
    recv = {o: torch.randn(N, ch, *geom.strip_extent(o, "fold"), device=dev).bfloat16() for o in offs}

    gx_aug = jc.conv_nd_input((N, ch, *geom.padded), w, g, padding=pad)
    send_u = halo_pack(gx_aug, geom, from_padded=True)
    gx_u = halo_fold(gx_aug, recv, geom)

    fused = jc.conv_nd_input_fold(geom, w, g, padding=pad)
    assert fused is not None, "the MFMA path should cover this case"
    gx_f, send_f = fused
    halo_fold_border_(gx_f, recv, geom)
    assert torch.equal(gx_f.view(torch.int16), gx_u.view(torch.int16))
    assert set(send_f) == set(send_u)
    for o in send_u:
        assert torch.equal(send_f[o].view(torch.int16), send_u[o].view(torch.int16)), f"strip {o}"


def test_fused_dgrad_fold_declines_what_the_mfma_kernel_does_not_cover(dev):
    from jigsaw_amd.halo import HaloGeometry

    geom = HaloGeometry((8, 8), (1, 1), (1, 1))
    w = torch.randn(4, 3, 3, 3, device=dev)
    g = torch.randn(1, 4, 8, 8, device=dev)
    assert jc.conv_nd_input_fold(geom, w, g, padding=(0, 0)) is None


FRAMED_CASES = [
    # size, lo, hi, conv padding on the padded tile, N, channels
    ((96, 256), (1, 1), (1, 1), (0, 0), 2, 64),
    ((70, 200), (1, 1), (1, 1), (0, 0), 1, 64),
    ((40, 330), (1, 0), (1, 0), (0, 1), 1, 32),       # W axis not split: the conv pads it itself
    ((66, 130), (0, 2), (2, 0), (0, 0), 1, 64),
    ((4, 40, 140), (1, 1, 1), (1, 1, 1), (0, 0, 0), 1, 32),
]


@pytest.mark.parametrize("case", FRAMED_CASES, ids=lambda c: f"{'x'.join(map(str, c[0]))}_lo{''.join(map(str, c[1]))}_hi{''.join(map(str, c[2]))}")
def test_framed_conv_has_the_bits_of_the_assembled_tile(case, dev):
    """Forward and weight gradient that read the own tile directly, plus a frame of the padded
    tile near the edges, equal the kernels on the fully assembled tile bit for bit; what lies
    outside the frame is never read (it holds NaN here)."""
    from jigsaw_amd.halo import HaloGeometry, halo_assemble

    size, lo, hi, pad, N, ch = case
    ns = len(size)
    geom = HaloGeometry(size, lo, hi)
    torch.manual_seed(5)
    k = (3,) * ns
    x = torch.randn(N, ch, *size, device=dev).bfloat16()
    strips = {o: torch.randn(N, ch, *geom.strip_extent(o, "assemble"), device=dev).bfloat16() for o in geom.offsets()}
    w = ((torch.rand(ch, ch, *k, device=dev) * 2 - 1) / (ch * 3**ns) ** 0.5).bfloat16()
    b = (torch.randn(ch, device=dev) * 0.1).bfloat16()
    x_aug = halo_assemble(x, strips, geom)
    y_ref = jc.conv_nd(x_aug, w, b, padding=pad)
    g = torch.randn_like(y_ref)
    gw_ref, gb_ref = jc.conv_nd_weight(x_aug, w.shape, g, padding=pad, with_bias_grad=True)

    bands = jc.frame_bands(x, geom, w.shape, padding=pad)
    if bands is None:
        # the framed weight-gradient kernel needs an even padding along W; callers assemble the whole tile then
        assert pad[-1] % 2 == 1
        return
    frame = torch.full_like(x_aug, float("nan"))
    halo_assemble(x, strips, geom, out=frame, bands=bands)
    # the frame holds exactly the band cells of the assembled tile
    inside = torch.ones(geom.padded, dtype=torch.bool, device=dev)
    for a in range(ns):
        idx = torch.arange(geom.padded[a], device=dev)
        in_band = (idx < bands[0][a]) | (idx >= geom.padded[a] - bands[1][a])
        shape = [1] * ns
        shape[a] = -1
        inside &= ~in_band.view(shape)
    assert torch.equal(frame[..., ~inside].view(torch.int16), x_aug[..., ~inside].view(torch.int16))
    assert torch.isnan(frame[..., inside]).all()

    y = jc.conv_nd_framed(frame, x, geom, w, b, padding=pad)
    assert y is not None and torch.equal(y.view(torch.int16), y_ref.view(torch.int16))
    gw, gb = jc.conv_nd_weight_framed(frame, x, geom, w.shape, g, padding=pad, with_bias_grad=True)
    assert torch.equal(gw.view(torch.int16), gw_ref.view(torch.int16))
    assert torch.equal(gb.view(torch.int16), gb_ref.view(torch.int16))


def _crop_check(y, x_aug, w, b, windows, what):
    """Output windows of the full-size result against the oracle on the matching input
    crops (a k=3, pad-0 conv: output rows h0..h0+H come from input rows h0..h0+H+2)."""
    ns = y.dim() - 2
    for n, *org in windows:
        ext = (32,) * (ns - 1) + (64,)
        ext = tuple(min(e, y.shape[2 + a] - org[a]) for a, e in enumerate(ext))
        osl = (n, slice(None)) + tuple(slice(o, o + e) for o, e in zip(org, ext))
        isl = (slice(n, n + 1), slice(None)) + tuple(slice(o, o + e + 2) for o, e in zip(org, ext))
        want = oc.forward(x_aug[isl].float().cpu(), w.float().cpu(), None if b is None else b.float().cpu(),
                          (1,) * ns, (0,) * ns, (1,) * ns)[0]
        assert rel_l2(y[osl], want) < 2e-2, f"{what}: window {n, *org}"


def test_config2_full_size_properties(dev):
    """Configuration 2 at full size (8 x 64 x 1024^2 bf16, all 8 neighbours live): output
    windows from the corners, edges and interior of several batch entries against the oracle
    on the matching crops; the fused backward against the separate steps bit for bit; the
    weight gradient as the sum of per-entry weight gradients, one of them against the oracle;
    the bias gradient against the plain sum."""
    from jigsaw_amd.halo import HaloGeometry, halo_assemble, halo_fold, halo_fold_border_

    torch.manual_seed(0)
    N, C, T = 8, 64, 1024
    geom = HaloGeometry((T, T), (1, 1), (1, 1))
    x = torch.randn(N, C, T, T, device=dev).bfloat16()
    w = ((torch.rand(C, C, 3, 3, device=dev) * 2 - 1) / 24).bfloat16()
    b = ((torch.rand(C, device=dev) * 2 - 1) / 24).bfloat16()
    g = torch.randn(N, C, T, T, device=dev).bfloat16()
    sf = {o: torch.randn(N, C, *geom.strip_extent(o, "assemble"), device=dev).bfloat16() for o in geom.offsets()}
    sb = {o: torch.randn(N, C, *geom.strip_extent(o, "fold"), device=dev).bfloat16() for o in geom.offsets()}

    x_aug = halo_assemble(x, sf, geom)
    y = jc.conv_nd(x_aug, w, b)
    wins = [(0, 0, 0), (0, 0, T - 64), (3, T - 32, 0), (7, T - 32, T - 64), (5, 496, 480), (2, 16, 960), (6, 1000, 64)]
    _crop_check(y, x_aug, w, b, wins, "forward")

    # backward: fused == separate, and the padded gradient against the oracle (dgrad of a
    # k=3 conv is the conv of the zero-padded g with the flipped, transposed weight)
    gx_aug = jc.conv_nd_input(x_aug.shape, w, g)
    wt = w.flip(-1, -2).transpose(0, 1).contiguous()
    g_pad = torch.nn.functional.pad(g, (2, 2, 2, 2))
    wins_aug = [(0, 0, 0), (1, 0, T + 2 - 64), (4, T + 2 - 32, 0), (7, T + 2 - 32, T + 2 - 64), (3, 500, 500)]
    _crop_check(gx_aug, g_pad, wt, None, wins_aug, "dgrad")
    gx_u = halo_fold(gx_aug, sb, geom)
    send_u = halo_pack(gx_aug, geom, from_padded=True)
    del gx_aug, g_pad
    gx_f, send_f = jc.conv_nd_input_fold(geom, w, g)
    halo_fold_border_(gx_f, sb, geom)
    assert torch.equal(gx_f.view(torch.int16), gx_u.view(torch.int16))
    for o in send_u:
        assert torch.equal(send_f[o].view(torch.int16), send_u[o].view(torch.int16)), f"strip {o}"
    del gx_u, gx_f

    gw, gb = jc.conv_nd_weight(x_aug, w.shape, g, with_bias_grad=True)
    parts = [jc.conv_nd_weight(x_aug[n:n + 1], w.shape, g[n:n + 1]).float() for n in range(N)]
    assert rel_l2(gw, sum(parts)) < 1e-2
    want1 = oc.wgrad(x_aug[5:6].float().cpu(), w.shape, g[5:6].float().cpu(), (1, 1), (0, 0), (1, 1))
    assert rel_l2(parts[5], want1) < 2e-2
    assert rel_l2(gb, g.float().sum((0, 2, 3))) < 1e-2


def test_config3_full_size_properties(dev):
    """Configuration 3 at full size (2 x 32 x 128^3 bf16, 26 neighbours): forward and padded
    gradient windows against the oracle on crops, the fused backward against the separate
    steps bit for bit, the weight gradient of one entry against the oracle."""
    from jigsaw_amd.halo import HaloGeometry, halo_assemble, halo_fold, halo_fold_border_

    torch.manual_seed(1)
    N, C, T = 2, 32, 128
    geom = HaloGeometry((T, T, T), (1, 1, 1), (1, 1, 1))
    x = torch.randn(N, C, T, T, T, device=dev).bfloat16()
    w = ((torch.rand(C, C, 3, 3, 3, device=dev) * 2 - 1) / 864 ** 0.5).bfloat16()
    b = ((torch.rand(C, device=dev) * 2 - 1) / 864 ** 0.5).bfloat16()
    g = torch.randn(N, C, T, T, T, device=dev).bfloat16()
    sf = {o: torch.randn(N, C, *geom.strip_extent(o, "assemble"), device=dev).bfloat16() for o in geom.offsets()}
    sb = {o: torch.randn(N, C, *geom.strip_extent(o, "fold"), device=dev).bfloat16() for o in geom.offsets()}

    x_aug = halo_assemble(x, sf, geom)
    y = jc.conv_nd(x_aug, w, b)
    wins = [(0, 0, 0, 0), (1, T - 32, T - 32, T - 64), (0, 0, T - 32, 64), (1, 96, 0, 0), (0, 50, 50, 30)]
    _crop_check(y, x_aug, w, b, wins, "forward")

    gx_aug = jc.conv_nd_input(x_aug.shape, w, g)
    wt = w.flip(-1, -2, -3).transpose(0, 1).contiguous()
    g_pad = torch.nn.functional.pad(g, (2,) * 6)
    wins_aug = [(0, 0, 0, 0), (1, T + 2 - 32, T + 2 - 32, T + 2 - 64), (0, 40, 98, 66), (1, 0, 98, 0)]
    _crop_check(gx_aug, g_pad, wt, None, wins_aug, "dgrad")
    gx_u = halo_fold(gx_aug, sb, geom)
    send_u = halo_pack(gx_aug, geom, from_padded=True)
    fused = jc.conv_nd_input_fold(geom, w, g)
    assert fused is not None
    gx_f, send_f = fused
    halo_fold_border_(gx_f, sb, geom)
    assert torch.equal(gx_f.view(torch.int16), gx_u.view(torch.int16))
    for o in send_u:
        assert torch.equal(send_f[o].view(torch.int16), send_u[o].view(torch.int16)), f"strip {o}"

    gw, gb = jc.conv_nd_weight(x_aug, w.shape, g, with_bias_grad=True)
    parts = [jc.conv_nd_weight(x_aug[n:n + 1], w.shape, g[n:n + 1]).float() for n in range(N)]
    assert rel_l2(gw, sum(parts)) < 1e-2
    want0 = oc.wgrad(x_aug[0:1].float().cpu(), w.shape, g[0:1].float().cpu(), (1, 1, 1), (0, 0, 0), (1, 1, 1))
    assert rel_l2(parts[0], want0) < 2e-2
    assert rel_l2(gb, g.float().sum((0, 2, 3, 4))) < 1e-2
