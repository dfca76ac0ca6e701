"""HIP log-sum-exp merge against the oracle (GPU). fp32 tolerance 1e-6 abs/rel."""

import pytest
import torch

from jigsaw_amd.attention import fused_online_softmax_merge_
from oracle import attention as oa

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
@pytest.mark.parametrize("o2_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 8, 128, 64), (2, 3, 17, 16), (1, 2, 5, 7)])
def test_merge_matches_oracle(layout, o2_dtype, shape, dev):
    torch.manual_seed(0)
    b, h, n, d = shape
    oshape = (b, h, n, d) if layout == "bhsd" else (b, n, h, d)
    o1 = torch.randn(*oshape)
    o2 = torch.randn(*oshape).to(o2_dtype)
    l1, l2 = torch.randn(b, h, n) * 3, torch.randn(b, h, n) * 3
    l1[0, 0, 0] = float("-inf")
    want_o, want_l = oa.merge_(o1.clone(), l1, o2.float(), l2, layout=layout, form="fused")
    g1 = o1.to(dev)
    res = fused_online_softmax_merge_(g1, l1.to(dev), o2.to(dev), l2.to(dev), layout)
    assert res is not None and res[0] is g1
    torch.testing.assert_close(res[0].cpu(), want_o, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(res[1].cpu(), want_l, atol=1e-6, rtol=1e-6)


def test_merge_seed_state_is_exact(dev):
    torch.manual_seed(1)
    o2 = torch.randn(1, 8, 64, 64).bfloat16().to(dev)
    l2 = torch.randn(1, 8, 64).to(dev)
    o1 = torch.zeros(1, 8, 64, 64, device=dev)
    l1 = torch.full((1, 8, 64), float("-inf"), device=dev)
    o, l = fused_online_softmax_merge_(o1, l1, o2, l2, "bhsd")
    assert torch.equal(o, o2.float()) and torch.equal(l, l2)


def test_merge_declines_what_the_reference_declines(dev):
    o = torch.zeros(1, 2, 4, 8, device=dev)
    l = torch.zeros(1, 2, 4, device=dev)
    assert fused_online_softmax_merge_(o.cpu(), l.cpu(), o.cpu(), l.cpu(), "bhsd") is None
    assert fused_online_softmax_merge_(o, l, o, l, "sbhd") is None
    assert fused_online_softmax_merge_(o, l, o.transpose(1, 2), l, "bhsd") is None
    assert fused_online_softmax_merge_(o, l[0], o, l[0], "bhsd") is None
    assert fused_online_softmax_merge_(o.double(), l, o.double(), l, "bhsd") is None
