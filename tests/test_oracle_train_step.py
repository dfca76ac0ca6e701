"""The four-rank training step of the CPU-runnable configuration (oracle/train_step.py)
against the same model on the undivided image (the method of the reference's
tests/test_examples.py:172-217): losses and updated weights agree, and the replicas stay
identical (gradients are summed in-graph, parallel/_sync.py:33-46). CPU, gloo, world 4."""

import pytest
import torch

from oracle import train_step as ots


@pytest.mark.timeout(240)
def test_four_gloo_ranks_equal_the_undivided_model():
    steps, batch, size = 2, 2, 32
    got = ots.run_four_ranks(steps=steps, batch=batch, size=size, threads=1, timeout=200.0)
    assert sorted(got) == [0, 1, 2, 3]
    want_losses, want_params = ots.reference_step(steps, batch, size)
    for rank, (losses, sec, params) in got.items():
        assert sec > 0
        torch.testing.assert_close(torch.tensor(losses), torch.tensor(want_losses), atol=1e-5, rtol=1e-5)
        for p, w in zip(params, want_params):
            torch.testing.assert_close(p, w, atol=2e-5, rtol=1e-4)
    for p0, p3 in zip(got[0][2], got[3][2]):
        assert torch.equal(p0, p3), "replicas diverged"
