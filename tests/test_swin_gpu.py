"""One rank's Swin block on the GPU kernels against the block on the undivided grid
(the reference's method, tests/test_examples.py:219-271) (GPU).

Forward: every rank of a 2x2 mesh runs in this process, stage by stage; the slabs
the two rolls exchange are produced by the roll oracle from the other ranks' stage
outputs (pure copies, so exact). Backward: on a 1x1 mesh against autograd of the
oracle block (the roll's backward exchange is covered by test_roll_gpu).
Tolerance: 1e-4 of max|want| in fp32 (the reference's bound,
tests/test_examples.py:48-67); rel-L2 2e-2 in bf16.
"""

import pytest
import torch

from helpers import mesh_coords, rel_l2
from jigsaw_amd import swin as js
from jigsaw_amd.conv import TileGroup
from oracle import roll as orl
from oracle import swin as osw

pytestmark = pytest.mark.gpu

DIM, HEADS, WINDOW = 32, 2, 4


class Answers:
    """Stand-in for RollConfig.comm_halo_1d_fn: hands over precomputed slabs."""

    def __init__(self):
        self.queue = []

    def __call__(self, data, buffer, direction, *, group, async_op):
        buffer.copy_(self.queue.pop(0).to(buffer.device))
        return buffer, None


def _tiles(glob, mesh, n):
    return {c: glob[:, c[0] * n[0] : (c[0] + 1) * n[0], c[1] * n[1] : (c[1] + 1) * n[1]].contiguous() for c in mesh_coords(mesh)}


def _roll_all(blocks, comms, stage_in, mesh, shift, which):
    """Run the shift / unshift stage of every rank; exchange answers from the roll oracle."""
    if shift == 0:
        return {c: getattr(blocks[c], which)(t) for c, t in stage_in.items()}
    cpu = {c: t.detach().cpu() for c, t in stage_in.items()}
    local = {c: torch.roll(t, (shift, shift), (1, 2)) for c, t in cpu.items()}
    after_h = orl.distributed_roll_mesh({c: t.clone() for c, t in cpu.items()}, mesh, (shift, shift), (1, 2), [1])
    direction = 1 if shift > 0 else -1
    sl = slice(0, shift) if shift > 0 else slice(shift, None)
    out = {}
    for c in mesh_coords(mesh):
        src_h = ((c[0] - direction) % mesh[0], c[1])
        src_w = (c[0], (c[1] - direction) % mesh[1])
        comms[c].queue = [local[src_h][:, sl].contiguous(), after_h[src_w][:, :, sl].contiguous()]
        out[c] = getattr(blocks[c], which)(stage_in[c])
        assert not comms[c].queue
    return out


@pytest.mark.parametrize("shift", [0, 2])
def test_swin_block_forward_tiled_equals_undivided(shift, dev):
    torch.manual_seed(0)
    mesh, n = (2, 2), (8, 8)
    B = 2
    glob = torch.randn(B, n[0] * 2, n[1] * 2, DIM)
    ref_block = js.SwinBlock(DIM, HEADS, WINDOW, (n[0] * 2, n[1] * 2), shift=shift, device=dev)
    with torch.no_grad():
        ref_block.attn.bias_table.normal_(0, 0.5)
    params = {k: v.detach().double().cpu() for k, v in ref_block.state_dict().items()}
    want = osw.block(glob.double(), params, HEADS, WINDOW, shift)

    tiles = _tiles(glob, mesh, n)
    blocks, comms = {}, {}
    for c in mesh_coords(mesh):
        comms[c] = Answers()
        groups = (TileGroup(mesh[0], c[0]), TileGroup(mesh[1], c[1]))
        blocks[c] = js.SwinBlock(DIM, HEADS, WINDOW, n, groups, comms[c], shift=shift, device=dev)
        blocks[c].load_state_dict(ref_block.state_dict())
    with torch.no_grad():
        x = {c: t.to(dev) for c, t in tiles.items()}
        y = {c: blocks[c].pre_attention(x[c]) for c in x}
        y = _roll_all(blocks, comms, y, mesh, -shift, "shift")
        y = {c: blocks[c].attn(y[c]) for c in y}
        y = _roll_all(blocks, comms, y, mesh, shift, "unshift")
        out = {c: blocks[c].finish(x[c], y[c]) for c in x}
    want_tiles = _tiles(want, mesh, n)
    bound = 1e-4 * want.abs().max().item()
    for c in mesh_coords(mesh):
        err = (out[c].double().cpu() - want_tiles[c]).abs().max().item()
        assert err < bound, f"rank {c}: max err {err:.3e} >= {bound:.3e}"


@pytest.mark.parametrize("shift", [0, 2])
def test_swin_block_backward_matches_autograd(shift, dev):
    torch.manual_seed(1)
    n = (8, 12)
    x = torch.randn(2, *n, DIM)
    block = js.SwinBlock(DIM, HEADS, WINDOW, n, shift=shift, device=dev)
    with torch.no_grad():
        block.attn.bias_table.normal_(0, 0.5)
    params = {k: v.detach().double().cpu().requires_grad_() for k, v in block.state_dict().items()}
    xd = x.double().requires_grad_()
    want = osw.block(xd, params, HEADS, WINDOW, shift)
    g = torch.randn_like(want)
    want.backward(g)
    xg = x.to(dev).requires_grad_()
    out = block(xg)
    out.backward(g.float().to(dev))
    assert rel_l2(out, want.detach()) < 1e-5
    assert rel_l2(xg.grad, xd.grad) < 1e-4, f"dx {rel_l2(xg.grad, xd.grad):.3e}"
    for name, prm in block.named_parameters():
        assert rel_l2(prm.grad, params[name].grad) < 1e-4, f"{name}: {rel_l2(prm.grad, params[name].grad):.3e}"


def test_swin_block_bf16_config5_shape(dev):
    """Config 5 shape (reduced tile): dim 128, 4 heads, 8x8 windows, shift 4, bf16 tokens."""
    torch.manual_seed(2)
    n, dim, heads, window, shift = (64, 64), 128, 4, 8, 4
    x = torch.randn(1, *n, dim)
    block = js.SwinBlock(dim, heads, window, n, shift=shift, device=dev)
    params = {k: v.detach().double().cpu() for k, v in block.state_dict().items()}
    want = osw.block(x.double(), params, heads, window, shift)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = block(x.to(dev))
    assert rel_l2(out, want) < 2e-2


@pytest.mark.parametrize("shift,n", [(4, (256, 256)), (0, (64, 128)), (4, (64, 64))])
def test_swin_block_bf16_backward_config5(shift, n, dev):
    """Config 5's block (dim 128, 4 heads, 8x8 windows, shift 4, bf16 autocast, at its real
    256 x 256 tile) forward AND backward on the bf16 kernels the benchmark times, against
    autograd of the fp64 oracle block: rel-L2 2e-2 on the output, dx and every parameter
    gradient."""
    torch.manual_seed(3)
    dim, heads, window = 128, 4, 8
    x = torch.randn(1, *n, dim)
    block = js.SwinBlock(dim, heads, window, n, shift=shift, device=dev)
    with torch.no_grad():
        block.attn.bias_table.normal_(0, 0.5)
    params = {k: v.detach().double().cpu().requires_grad_() for k, v in block.state_dict().items()}
    xd = x.double().requires_grad_()
    want = osw.block(xd, params, heads, window, shift)
    g = torch.randn_like(want)
    want.backward(g)
    xg = x.to(dev).requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = block(xg)
    out.backward(g.to(out.dtype).to(dev))
    assert rel_l2(out, want.detach()) < 2e-2, f"out {rel_l2(out, want.detach()):.3e}"
    assert rel_l2(xg.grad, xd.grad) < 2e-2, f"dx {rel_l2(xg.grad, xd.grad):.3e}"
    for name, prm in block.named_parameters():
        err = rel_l2(prm.grad, params[name].grad)
        assert err < 2e-2, f"{name}: {err:.3e}"


@pytest.mark.parametrize("shift,n", [(4, (256, 256)), (0, (64, 128)), (4, (64, 64))])
def test_block_as_one_autograd_node_has_the_bits_of_its_parts(shift, n, dev):
    """bf16 tokens under bf16 autocast (what the benchmark times): the block runs as a single
    autograd function that calls the forward / backward of the functions it is made of. Output,
    dx and every parameter gradient equal those of the block composed of the separate functions
    bit for bit, and meet the oracle at the bf16 bar."""
    torch.manual_seed(5)
    dim, heads, window = 128, 4, 8
    one = js.SwinBlock(dim, heads, window, n, shift=shift, device=dev)
    parts = js.SwinBlock(dim, heads, window, n, shift=shift, device=dev, one_node=False)
    with torch.no_grad():
        one.attn.bias_table.normal_(0, 0.5)
    parts.load_state_dict(one.state_dict())
    x = torch.randn(1, *n, dim).bfloat16()
    g = torch.randn(1, *n, dim).bfloat16()
    results = []
    for block in (one, parts):
        xg = x.to(dev).requires_grad_()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block(xg)
        results.append((out, xg, block))
        out.backward(g.to(dev))
    assert "WholeBlock" in type(results[0][0].grad_fn).__name__ and "WholeBlock" not in type(results[1][0].grad_fn).__name__
    (o1, x1, b1), (o2, x2, b2) = results
    assert torch.equal(o1, o2) and torch.equal(x1.grad, x2.grad)
    for (name, p1), (_, p2) in zip(b1.named_parameters(), b2.named_parameters()):
        assert p1.grad is not None and torch.equal(p1.grad, p2.grad), name
    params = {k: v.detach().double().cpu().requires_grad_() for k, v in one.state_dict().items()}
    xd = x.double().requires_grad_()
    want = osw.block(xd, params, heads, window, shift)
    want.backward(g.double())
    assert rel_l2(o1, want.detach()) < 2e-2 and rel_l2(x1.grad, xd.grad) < 2e-2
    for name, prm in one.named_parameters():
        assert rel_l2(prm.grad, params[name].grad) < 2e-2, name


@pytest.mark.parametrize("shift", [0, 4])
def test_block_step_recorded_in_a_hip_graph_replays_the_eager_step(shift, dev):
    """``SwinBlock.captured_step``: forward + backward recorded once, replayed several times with eager
    work and synchronisations in between; every replay gives the eager step's output, input gradient
    and parameter gradients bit for bit, also after new values were copied into the input buffers and
    after a parameter changed in place."""
    torch.manual_seed(7)
    dim, heads, window, n = 128, 4, 8, (32, 48)
    block = js.SwinBlock(dim, heads, window, n, shift=shift, device=dev)
    with torch.no_grad():
        block.attn.bias_table.normal_(0, 0.5)

    def eager(x, g):
        for p in block.parameters():
            p.grad = None
        xg = x.clone().requires_grad_()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block(xg)
        out.backward(g)
        return out.detach(), xg.grad, {k: p.grad.clone() for k, p in block.named_parameters()}

    x = torch.randn(1, *n, dim, device=dev).bfloat16()
    g = torch.randn(1, *n, dim, device=dev).bfloat16()
    step = block.captured_step(x.clone(), g.clone())
    assert set(step.grads) == {k for k, _ in block.named_parameters()}
    for rep in range(4):
        if rep == 2:  # new values in the graph's input buffers
            x, g = torch.randn_like(x), torch.randn_like(g)
            step.x.copy_(x)
            step.grad_out.copy_(g)
        if rep == 3:  # parameters are read where they lie
            with torch.no_grad():
                for prm in block.parameters():
                    prm.mul_(1.25).add_(0.01)
        step.replay()
        torch.cuda.synchronize()
        y, gx, grads = eager(x, g)  # eager work between the replays, and the values to meet
        torch.cuda.synchronize()
        assert torch.equal(step.y, y) and torch.equal(step.grad_x, gx), rep
        for k, want in grads.items():
            assert step.grads[k].dtype == want.dtype and torch.equal(step.grads[k], want), (rep, k)
    with pytest.raises(NotImplementedError):
        block.captured_step(x.float(), g.float())


def test_one_node_block_with_frozen_parameters_and_a_second_backward(dev):
    """Frozen parameters and an input without a gradient get none from the one-node block, the others keep
    their bits; a second backward through the same graph says why it cannot run."""
    torch.manual_seed(5)
    n, dim = (16, 16), 128

    def comm(data, buffer, direction, *, group, async_op):
        return torch.zeros_like(buffer), None

    block = js.SwinBlock(dim, 4, 8, n, (TileGroup(1, 0), TileGroup(1, 0)), comm, shift=4, device=dev)
    x = torch.randn(2, *n, dim, device=dev).bfloat16().requires_grad_()
    gout = torch.randn(2, *n, dim, device=dev).bfloat16()

    def grads(freeze, x_grad):
        for name, p in block.named_parameters():
            p.requires_grad_(name not in freeze)
            p.grad = None
        xi = x.detach().requires_grad_(x_grad)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = block(xi)
        y.backward(gout, retain_graph=True)
        with pytest.raises(RuntimeError, match="second time"):
            y.backward(gout)
        return xi.grad, {k: p.grad for k, p in block.named_parameters()}

    gx_all, g_all = grads((), True)
    frozen = ("attn.qkv.weight", "norm2.bias", "mlp.0.weight", "attn.bias_table")
    gx_some, g_some = grads(frozen, False)
    assert gx_some is None and gx_all is not None
    for k, g in g_some.items():
        if k in frozen:
            assert g is None, k
        else:
            assert torch.equal(g, g_all[k]), k
