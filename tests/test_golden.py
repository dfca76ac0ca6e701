"""Known-answer fixtures of tests/golden (derived independently of the oracle and of the
kernels, see tests/golden/make_fixtures.py) against the oracle and the host logic (CPU)
and against the HIP kernels through the C ABI (GPU)."""

import json
from pathlib import Path

import pytest
import torch

from oracle import attention as oa
from oracle import conv_transpose as oct_
from oracle import halo as oh
from oracle import layernorm as ol

GOLDEN = Path(__file__).parent / "golden"
SPANS = json.loads((GOLDEN / "spans.json").read_text())
CASES = json.loads((GOLDEN / "float_cases.json").read_text())
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


def test_span_tables_oracle_and_host():
    from jigsaw_amd import conv_transpose as jct
    from jigsaw_amd import halo as jh

    for G, n, k, s, p, d, r, lo, hi, out_local in SPANS["conv_need_span"]:
        assert oh.needed_input_span(r, G, n, k, s, p, d) == (lo, hi, hi - lo, out_local)
        assert jh.needed_input_span(r, G, n, k, s, p, d)[:2] == (lo, hi)
    for G, n, k, s, p, d, r, base, wloc, out_local, gout in SPANS["convt_raw_span"]:
        assert oct_.produced_output_span(r, G, n, k, s, p, d) == (base, wloc, out_local, gout)
        assert jct.produced_output_span(r, G, n, k, s, p, d) == (base, wloc, out_local, gout)


def _corner_grads(c, dtype):
    """Padded gradients of the 9 ranks of a 3x3 mesh, tile 4x4, halo 1: zero but for the
    four cells that meet in cell (0, 0) of the middle rank."""
    grads = {(i, j): torch.zeros(1, 1, 6, 6, dtype=dtype) for i in range(3) for j in range(3)}
    grads[(1, 1)][0, 0, 1, 1] = c["own"]
    grads[(1, 0)][0, 0, 1, 5] = c["left"]
    grads[(0, 1)][0, 0, 5, 1] = c["top"]
    grads[(0, 0)][0, 0, 5, 5] = c["diag"]
    return grads


@pytest.mark.parametrize("name", ["float32", "bfloat16"])
def test_fold_corner_oracle(name):
    c = CASES["fold_corner"][name]
    folded = oh.scatter_add_mesh(_corner_grads(c, DT[name]), (3, 3), (3, 3), (1, 1), (1, 1), (1, 1), (4, 4))
    got = folded[(1, 1)][0, 0, 0, 0].item()
    assert got == c["want"] and got != c["other_order"]


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["float32", "bfloat16"])
def test_fold_corner_kernels(name, dev):
    """The separate fold and the border fold (after a fused dgrad would have written the own
    cells) give the fixture's bits."""
    from jigsaw_amd.halo import HaloGeometry, halo_fold, halo_fold_border_, halo_pack

    c = CASES["fold_corner"][name]
    grads = {k: v.to(dev) for k, v in _corner_grads(c, DT[name]).items()}
    geom = HaloGeometry((4, 4), (1, 1), (1, 1))
    recv = {}
    for o in geom.offsets():
        nb = (1 + o[0], 1 + o[1])
        back = (-o[0], -o[1])
        recv[o] = halo_pack(grads[nb], geom, from_padded=True, present=[back])[back]
    gx = halo_fold(grads[(1, 1)], recv, geom)
    assert gx[0, 0, 0, 0].item() == c["want"]
    own = grads[(1, 1)][..., 1:5, 1:5].contiguous() + 0.0
    halo_fold_border_(own, recv, geom)
    assert own[0, 0, 0, 0].item() == c["want"]
    assert torch.equal(own, gx)


def _merge_inputs(case, device="cpu"):
    l1 = float("-inf") if case["l1"] == "-inf" else case["l1"]
    o1 = torch.full((1, 1, 1, 8), case["o1"], dtype=torch.float32, device=device)
    o2 = torch.full((1, 1, 1, 8), case["o2"], dtype=torch.float32, device=device)
    return o1, torch.full((1, 1, 1), l1, device=device), o2, torch.full((1, 1, 1), case["l2"], device=device)


def test_lse_merge_oracle():
    for case in CASES["lse_merge"]:
        for form in ("eager", "fused"):
            o, l = oa.merge_(*_merge_inputs(case), form=form)
            assert abs(o[0, 0, 0, 0].item() - case["o"]) < 1e-6 and abs(l.item() - case["l"]) < 1e-6


@pytest.mark.gpu
def test_lse_merge_kernel(dev):
    from jigsaw_amd import attention as ja

    for case in CASES["lse_merge"]:
        res = ja.fused_online_softmax_merge_(*_merge_inputs(case, dev), "bhsd")
        assert res is not None
        o, l = res
        assert abs(o[0, 0, 0, 0].item() - case["o"]) < 1e-6 and abs(l.item() - case["l"]) < 1e-6


def test_layernorm_two_shards_oracle():
    c = CASES["layernorm_two_shards"]
    xs = [torch.tensor([s], dtype=torch.float64) for s in c["shards"]]
    for x, m, v in zip(xs, c["partial_mean"], c["partial_var"]):
        pm, pv = ol.partial_stats(x)
        assert pm.item() == m and abs(pv.item() - v) < 1e-12
    ones = [torch.ones(4, dtype=torch.float64)] * 2
    ys, _, std = ol.forward(xs, ones, [None, None], 0.0)
    assert abs(std.item() ** 2 - c["var"]) < 1e-12
    assert torch.allclose(torch.cat(ys, -1)[0], torch.tensor(c["normalised"], dtype=torch.float64), rtol=1e-12)


@pytest.mark.gpu
def test_layernorm_two_shards_kernels(dev):
    from jigsaw_amd import layernorm as jl

    c = CASES["layernorm_two_shards"]

    class Other:
        """Channel group of two whose other member's contributions are the fixture's."""

        def __init__(self, mean, var):
            self.vals, self.calls = [mean, var], 0

        def size(self):
            return 2

        def all_reduce(self, t, op):
            assert op == "avg"
            t.add_(self.vals[self.calls]).div_(2)
            self.calls += 1

    for i in (0, 1):
        x = torch.tensor([c["shards"][i]], dtype=torch.float32, device=dev)
        m, v = jl.partial_stats(x)
        assert m.item() == c["partial_mean"][i] and abs(v.item() - c["partial_var"][i]) < 1e-6
        j = 1 - i
        # what the other shard adds to the variance all-reduce: var_j + (mean_j - mean)^2
        other = Other(c["partial_mean"][j], c["partial_var"][j] + (c["partial_mean"][j] - c["mean"]) ** 2)
        w = torch.ones(4, device=dev)
        y = jl._LayerNorm.apply(x, w, None, other, 0.0)[0]
        want = torch.tensor(c["normalised"][4 * i: 4 * i + 4], device=dev)
        assert torch.allclose(y[0], want, rtol=1e-5, atol=1e-6)
