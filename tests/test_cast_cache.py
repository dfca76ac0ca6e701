"""The remembered parameter casts of jigsaw_amd.projection: off by default, and when on,
dropped by everything a tensor can show of a change (version counter, storage address, device, dtype)
and by invalidate_casts() for writes through ``.data``, which show nothing."""

import pytest
import torch

from jigsaw_amd import projection as jp


@pytest.fixture
def remembering():
    before = jp.remember_casts(True)
    yield
    jp.remember_casts(before)


def test_default_casts_anew_every_call():
    w = torch.nn.Parameter(torch.randn(4, 3))
    a = jp._cast_cached(w, torch.bfloat16)
    w.data.mul_(2.0)  # no version bump, same storage
    b = jp._cast_cached(w, torch.bfloat16)
    assert a is not b
    assert torch.equal(b, w.detach().to(torch.bfloat16))
    assert getattr(w, "_jg_casts", None) is None


def test_remembered_cast_follows_in_place_updates_and_new_storage(remembering):
    w = torch.nn.Parameter(torch.randn(4, 3))
    a = jp._cast_cached(w, torch.bfloat16)
    assert jp._cast_cached(w, torch.bfloat16) is a
    at = jp._cast_cached(w, torch.bfloat16, transposed=True)
    assert torch.equal(at, a.t())
    with torch.no_grad():
        w.add_(1.0)  # what an optimizer step does: bumps the version
    b = jp._cast_cached(w, torch.bfloat16)
    assert b is not a and torch.equal(b, w.detach().to(torch.bfloat16))
    w.data = torch.randn(4, 3)  # new storage, same version
    c = jp._cast_cached(w, torch.bfloat16)
    assert c is not b and torch.equal(c, w.detach().to(torch.bfloat16))


def test_data_write_needs_invalidate(remembering):
    lin = torch.nn.Linear(3, 4)
    a = jp._cast_cached(lin.weight, torch.bfloat16)
    lin.weight.data.normal_()  # invisible: same version, same address
    assert jp._cast_cached(lin.weight, torch.bfloat16) is a  # the documented limit of remembering
    jp.invalidate_casts(lin)
    b = jp._cast_cached(lin.weight, torch.bfloat16)
    assert b is not a and torch.equal(b, lin.weight.detach().to(torch.bfloat16))


def test_module_to_other_dtype_drops_the_cast(remembering):
    lin = torch.nn.Linear(3, 4)
    a = jp._cast_cached(lin.weight, torch.bfloat16)
    lin.double()
    b = jp._cast_cached(lin.weight, torch.bfloat16)
    assert b is not a and torch.equal(b, lin.weight.detach().to(torch.bfloat16))


@pytest.mark.gpu
def test_linear_follows_a_data_write_between_two_forwards():
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    lin = torch.nn.Linear(64, 64, device=dev)
    x = torch.randn(2, 128, 64, device=dev).bfloat16()

    def run():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            return jp.linear(x, lin.weight, lin.bias)

    run()
    lin.weight.data.mul_(-1.0)
    lin.bias.data.zero_()
    y = run()
    want = torch.nn.functional.linear(x.double(), lin.weight.detach().bfloat16().double())
    rel = ((y.double() - want).norm() / want.norm()).item()
    assert rel < 2e-2, rel  # bf16 bar; a stale weight gives rel ~ 2
