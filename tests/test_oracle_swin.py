"""Pins the Swin-block oracle (oracle/swin.py) on the CPU, each piece against a form
that does not share its formula:

* ``windows`` / ``unwindows``: explicit index loops, a hand-written 4x4 case, round trip;
* ``relative_position_index``: the double loop ``(dy + W - 1)(2W - 1) + (dx + W - 1)``;
* ``shift_mask_global``: a coordinate image rolled by ``-shift`` and cut into windows; a
  pair may attend iff the displacement between the two tokens is the same before and
  after the roll on both axes (i.e. neither axis crosses the image border);
* ``block``: a per-token restatement in which a shifted block is written without any roll
  or mask: token ``(y, x)`` attends the tokens of its window of the grid displaced by
  ``shift``, cut at the image border; softmax, LayerNorm and GELU written out by hand.
"""

import itertools
import math

import pytest
import torch

from oracle import swin as osw


def test_windows_hand_written_case():
    # 4x4 grid, windows of 2: rows of the result are the four 2x2 windows in row-major order
    x = torch.arange(16.0).view(1, 4, 4, 1)
    got = osw.windows(x, 2).view(4, 4)
    want = torch.tensor([[0, 1, 4, 5], [2, 3, 6, 7], [8, 9, 12, 13], [10, 11, 14, 15]], dtype=torch.float32)
    assert torch.equal(got, want)
    assert torch.equal(osw.unwindows(osw.windows(x, 2), 4, 4, 2), x)


@pytest.mark.parametrize("h,w,win", [(8, 12, 4), (6, 4, 2), (8, 8, 8)])
def test_windows_by_index_loops_and_round_trip(h, w, win):
    torch.manual_seed(0)
    x = torch.randn(2, h, w, 3)
    got = osw.windows(x, win)
    assert got.shape == (2, (h // win) * (w // win), win * win, 3)
    for b, y, xx in itertools.product(range(2), range(h), range(w)):
        nw = (y // win) * (w // win) + xx // win
        t = (y % win) * win + xx % win
        assert torch.equal(got[b, nw, t], x[b, y, xx])
    assert torch.equal(osw.unwindows(got, h, w, win), x)
    # and the other way round: unwindows of arbitrary window data, then windows
    z = torch.randn_like(got)
    assert torch.equal(osw.windows(osw.unwindows(z, h, w, win), win), z)


@pytest.mark.parametrize("win", [2, 3, 4, 8])
def test_relative_position_index_brute_force(win):
    got = osw.relative_position_index(win)
    n = win * win
    assert got.shape == (n, n)
    for a, b in itertools.product(range(n), repeat=2):
        dy, dx = a // win - b // win, a % win - b % win
        assert got[a, b].item() == (dy + win - 1) * (2 * win - 1) + (dx + win - 1)
    # every table row is addressed, the diagonal is the centre of the table
    assert sorted(set(got.view(-1).tolist())) == list(range((2 * win - 1) ** 2))
    assert set(got.diagonal().tolist()) == {((2 * win - 1) ** 2) // 2}


def _mask_from_rolled_coordinates(h, w, win, shift):
    """A pair of one window may attend iff the roll moved both tokens alike."""
    ys, xs = torch.meshgrid(torch.arange(h), torch.arange(w), indexing="ij")
    ys, xs = torch.roll(ys, (-shift, -shift), (0, 1)), torch.roll(xs, (-shift, -shift), (0, 1))
    out = torch.zeros((h // win) * (w // win), win * win, win * win, dtype=torch.float64)
    for wy, wx in itertools.product(range(h // win), range(w // win)):
        cells = [(wy * win + i, wx * win + j) for i in range(win) for j in range(win)]
        for a, (ay, ax) in enumerate(cells):
            for b, (by, bx) in enumerate(cells):
                moved_alike = (ys[ay, ax] - ys[by, bx] == ay - by) and (xs[ay, ax] - xs[by, bx] == ax - bx)
                if not moved_alike:
                    out[wy * (w // win) + wx, a, b] = float("-inf")
    return out


@pytest.mark.parametrize("h,w,win,shift", [(8, 8, 4, 2), (8, 12, 4, 1), (16, 8, 4, 3), (16, 16, 8, 4), (4, 4, 2, 1)])
def test_shift_mask_from_rolled_coordinate_image(h, w, win, shift):
    got = osw.shift_mask_global(h, w, win, shift)
    want = _mask_from_rolled_coordinates(h, w, win, shift)
    assert torch.equal(got, want)
    # only windows in the last window row / column contain a border
    nwx = w // win
    for nw in range(got.shape[0]):
        touches = (nw // nwx == h // win - 1) or (nw % nwx == nwx - 1)
        assert bool(torch.isinf(got[nw]).any()) == touches


def _gelu(v):
    return 0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0)))


def _layer_norm_rows(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def _block_per_token(x, p, heads, win, shift, eps):
    """The block with no roll and no mask: the windows of a shifted block are those of the
    grid displaced by ``shift`` (cyclically), and a token attends the tokens of its window
    that lie on its own side of the image border."""
    B, H, W, C = x.shape
    d = C // heads
    y = _layer_norm_rows(x, p["norm1.weight"], p["norm1.bias"], eps)
    qkv = y @ p["attn.qkv.weight"].T + p["attn.qkv.bias"]  # (B, H, W, 3C): features (three, head, d)
    att = torch.zeros_like(x)
    table = p["attn.bias_table"]
    for b, ty, tx in itertools.product(range(B), range(H), range(W)):
        # the window of (ty, tx): in displaced coordinates u = (t - shift) mod size the windows are aligned
        uy, ux = (ty - shift) % H, (tx - shift) % W
        members = []
        for i, j in itertools.product(range(win), repeat=2):
            vy, vx = (uy // win) * win + i, (ux // win) * win + j
            sy, sx = (vy + shift) % H, (vx + shift) % W
            # same side of the border: displaced and original coordinates differ by the same amount
            if (sy - ty == vy - uy) and (sx - tx == vx - ux):
                members.append((sy, sx, vy - uy, vx - ux))
        for hd in range(heads):
            q = qkv[b, ty, tx, hd * d : (hd + 1) * d]
            scores = []
            for sy, sx, dy, dx in members:
                k = qkv[b, sy, sx, C + hd * d : C + (hd + 1) * d]
                # bias entry for (query - key) displacement: query is at offset 0, key at (dy, dx)
                row = (-dy + win - 1) * (2 * win - 1) + (-dx + win - 1)
                scores.append(float(q @ k) / math.sqrt(d) + float(table[row, hd]))
            m = max(scores)
            e = [math.exp(s - m) for s in scores]
            z = sum(e)
            acc = torch.zeros(d, dtype=x.dtype)
            for wgt, (sy, sx, _, _) in zip(e, members):
                acc += (wgt / z) * qkv[b, sy, sx, 2 * C + hd * d : 2 * C + (hd + 1) * d]
            att[b, ty, tx, hd * d : (hd + 1) * d] = acc
    x = x + att @ p["attn.proj.weight"].T + p["attn.proj.bias"]
    z = _layer_norm_rows(x, p["norm2.weight"], p["norm2.bias"], eps)
    hid = z @ p["mlp.0.weight"].T + p["mlp.0.bias"]
    hid = hid.clone().apply_(_gelu)
    return x + hid @ p["mlp.2.weight"].T + p["mlp.2.bias"]


def _params(dim, heads, win, seed):
    g = torch.Generator().manual_seed(seed)

    def rn(*shape, scale=1.0):
        return torch.randn(*shape, generator=g, dtype=torch.float64) * scale

    return {
        "norm1.weight": 1 + 0.2 * rn(dim), "norm1.bias": 0.2 * rn(dim),
        "norm2.weight": 1 + 0.2 * rn(dim), "norm2.bias": 0.2 * rn(dim),
        "attn.qkv.weight": rn(3 * dim, dim, scale=dim**-0.5), "attn.qkv.bias": 0.1 * rn(3 * dim),
        "attn.proj.weight": rn(dim, dim, scale=dim**-0.5), "attn.proj.bias": 0.1 * rn(dim),
        "attn.bias_table": 0.5 * rn((2 * win - 1) ** 2, heads),
        "mlp.0.weight": rn(4 * dim, dim, scale=dim**-0.5), "mlp.0.bias": 0.1 * rn(4 * dim),
        "mlp.2.weight": rn(dim, 4 * dim, scale=(4 * dim) ** -0.5), "mlp.2.bias": 0.1 * rn(dim),
    }


@pytest.mark.parametrize("h,w,win,shift", [(8, 8, 4, 0), (8, 8, 4, 2), (8, 12, 4, 1), (4, 6, 2, 1)])
def test_block_against_per_token_restatement(h, w, win, shift):
    dim, heads = 8, 2
    p = _params(dim, heads, win, seed=h * 100 + w + shift)
    x = torch.randn(2, h, w, dim, dtype=torch.float64, generator=torch.Generator().manual_seed(7))
    got = osw.block(x, p, heads, win, shift)
    want = _block_per_token(x, p, heads, win, shift, 1e-5)
    torch.testing.assert_close(got, want, atol=1e-11, rtol=1e-9)


@pytest.mark.parametrize("H,W,win,shift", [(16, 16, 4, 2), (16, 24, 4, 1), (32, 32, 8, 4), (8, 8, 2, 1)])
def test_package_index_and_mask_on_1x1_and_2x2_tilings(H, W, win, shift):
    """The package's own index and mask builders (built from rolled global positions) agree
    with the pinned oracle: on the undivided grid, and tile by tile on a 2 x 2 tiling, where
    the mask depends on where the tile sits."""
    from jigsaw_amd import swin as js
    from jigsaw_amd.conv import TileGroup

    assert torch.equal(js.relative_position_index(win), osw.relative_position_index(win))
    full = osw.shift_mask_global(H, W, win, shift)
    one = js.shift_mask(H, W, win, shift, (TileGroup(1, 0), TileGroup(1, 0)))
    assert torch.equal(one.double(), full)
    h, w = H // 2, W // 2
    by_window = full.view(H // win, W // win, win * win, win * win)
    for r, c in itertools.product(range(2), repeat=2):
        got = js.shift_mask(h, w, win, shift, (TileGroup(2, r), TileGroup(2, c)))
        want = by_window[r * (h // win) : (r + 1) * (h // win), c * (w // win) : (c + 1) * (w // win)]
        assert torch.equal(got.double().view(want.shape), want), f"tile ({r}, {c})"
    # the side code the mask is built from: 0 everywhere except in the last window row / column of the grid
    side = js.border_sides(H, W, win, shift, (TileGroup(1, 0), TileGroup(1, 0))).view(H // win, W // win, -1)
    assert int(side[:-1, :-1].abs().sum()) == 0 and int(side[-1, -1].max()) == 3
