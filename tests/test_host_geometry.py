"""Host-side geometry of the halo exchange and of the dilation route, on the CPU.

Pins, without a GPU and without the kernels: the halo widths of every rank against a brute-force
enumeration of the cells a rank's outputs touch (also where the need spans drift against the
tiles and the widths change from rank to rank), that the two ends of every exchange agree on
the strip shapes, the raw spans of the transposed convolution, and the identity behind the
dilated route (the residues of the pixel index are undilated problems of their own).
"""

import itertools

import pytest
import torch
import torch.nn.functional as F

from jigsaw_amd import conv as jc
from jigsaw_amd import conv_transpose as jct
from jigsaw_amd.halo import HaloGeometry, halo_widths

from helpers import mesh_coords, neighbour


def touched_span(rank, G, n, k, s, p, d):
    """First and one-past-last input row touched by the outputs of `rank`, by enumeration."""
    extent = d * (k - 1) + 1
    gout = (G * n + 2 * p - extent) // s + 1
    if gout % G:
        return None
    ol = gout // G
    rows = [o * s - p + t * d for o in range(rank * ol, (rank + 1) * ol) for t in range(k)]
    return min(rows), max(rows) + 1, ol


def test_halo_widths_against_enumeration():
    accepted = rejected = drifting = 0
    for G, n, k, s, p, d in itertools.product([2, 3, 4], [4, 6, 8, 9], [1, 2, 3, 5], [1, 2, 3], [0, 1, 2], [1, 2]):
        if G * n + 2 * p < d * (k - 1) + 1:
            continue
        for rank in range(G):
            span = touched_span(rank, G, n, k, s, p, d)
            if span is None:
                with pytest.raises(NotImplementedError):
                    halo_widths(rank, G, n, k, s, p, d)
                continue
            lo, hi, ol = span
            lo_w, hi_w = rank * n - lo, hi - (rank + 1) * n
            if 0 <= lo_w <= n and 0 <= hi_w <= n:
                assert halo_widths(rank, G, n, k, s, p, d) == (lo_w, hi_w, ol)
                accepted += 1
                drifting += ol * s != n
            else:
                with pytest.raises(NotImplementedError):
                    halo_widths(rank, G, n, k, s, p, d)
                rejected += 1
    assert accepted > 500 and rejected > 50 and drifting > 100


MESH_CASES = [
    # mesh, local size, kernel, stride, padding, dilation
    ((2, 2), (8, 10), (3, 3), (1, 1), (0, 0), (1, 1)),
    ((4, 2), (6, 8), (5, 3), (1, 1), (0, 1), (1, 1)),
    ((2, 2), (8, 8), (6, 6), (2, 2), (0, 0), (1, 1)),
    ((3, 3), (4, 6), (3, 5), (2, 2), (1, 2), (1, 1)),
    ((2, 1, 2), (4, 5, 6), (3, 3, 5), (1, 1, 1), (0, 1, 1), (1, 1, 1)),
    ((2, 2, 2), (6, 5, 8), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("case", MESH_CASES)
def test_both_ends_of_an_exchange_agree_on_the_strip(case):
    """What a rank cuts for a neighbour (forward: by the neighbour's halo, backward: its own halo's
    gradient) has the shape the neighbour expects from that side."""
    mesh, n, k, s, p, d = case
    geoms = {c: HaloGeometry.for_conv(n, k, s, p, d, c, mesh) for c in mesh_coords(mesh)}
    pairs = 0
    for c, g in geoms.items():
        assert g.padded == tuple(
            (touched_span(c[a], mesh[a], n[a], k[a], s[a], p[a], d[a])[1] - touched_span(c[a], mesh[a], n[a], k[a], s[a], p[a], d[a])[0])
            if mesh[a] > 1 else n[a] for a in range(len(mesh)))
        for o in g.offsets():
            nb = neighbour(c, o, mesh)
            if nb is None:
                continue
            back = tuple(-v for v in o)
            assert g.strip_extent(o, "pack_fwd") == geoms[nb].strip_extent(back, "assemble"), (c, o)
            assert g.strip_extent(o, "pack_bwd") == geoms[nb].strip_extent(back, "fold"), (c, o)
            pairs += 1
    assert pairs > 0


def test_raw_spans_of_the_transposed_convolution_against_enumeration():
    """Input column i, tap j writes output column i * s - p + d * j."""
    accepted = drifting = 0
    for G, n, k, s, p, d in itertools.product([2, 3, 4], [3, 4, 6], [1, 2, 3, 4, 5], [1, 2, 3], [0, 1, 2], [1, 2]):
        extent = d * (k - 1) + 1
        gout = (G * n - 1) * s - 2 * p + extent
        if gout <= 0 or gout % G:
            continue
        ol = gout // G
        for rank in range(G):
            cols = [i * s - p + d * j for i in range(rank * n, (rank + 1) * n) for j in range(k)]
            left, right = rank * ol - min(cols), max(cols) + 1 - (rank + 1) * ol
            if 0 <= left <= ol and 0 <= right <= ol:
                assert jct.raw_span_widths(rank, G, n, k, s, p, d) == (left, right, ol)
                accepted += 1
                drifting += extent != s + 2 * p
            else:
                with pytest.raises(NotImplementedError):
                    jct.raw_span_widths(rank, G, n, k, s, p, d)
    assert accepted > 100 and drifting > 20


def test_transposed_neighbours_agree_on_the_overlap():
    n, k, s, p, d, mesh = (5, 7), (4, 4), (2, 2), (0, 0), (1, 1), (2, 2)
    geoms = {c: jct.transpose_geometry(n, k, s, p, d, c, mesh) for c in mesh_coords(mesh)}
    for c, g in geoms.items():
        for o in g.offsets():
            nb = neighbour(c, o, mesh)
            if nb is not None:
                back = tuple(-v for v in o)
                assert g.strip_extent(o, "pack_bwd") == geoms[nb].strip_extent(back, "fold")
                assert g.strip_extent(o, "pack_fwd") == geoms[nb].strip_extent(back, "assemble")


DILATED = [
    # in spatial, kernel, padding, dilation
    ((13, 17), (3, 3), (2, 3), (2, 3)),
    ((12, 16), (3, 3), (0, 0), (2, 2)),
    ((9, 10), (3, 1), (4, 0), (2, 5)),
    ((5, 9, 11), (3, 3, 3), (1, 2, 4), (1, 2, 2)),
    ((15, 18), (5, 3), (4, 2), (2, 2)),     # five taps: the residue images are undilated five-tap problems
    ((11, 12), (2, 4), (3, 0), (3, 2)),
]


@pytest.mark.parametrize("case", DILATED)
def test_residue_images_are_undilated_problems(case):
    """The route of the dilated convolution, with torch's CPU operators in place of the kernels:
    forward, input gradient and weight gradient of the residue images give those of the dilated layer."""
    insp, k, p, d = case
    ns = len(k)
    assert jc._dilated_ok(k, (1,) * ns, p, d)
    conv = {2: F.conv2d, 3: F.conv3d}[ns]
    torch.manual_seed(0)
    x = torch.randn(2, 3, *insp, dtype=torch.float64, requires_grad=True)
    w = torch.randn(4, 3, *k, dtype=torch.float64, requires_grad=True)
    y = conv(x, w, None, 1, p, d)
    g = torch.randn_like(y)
    y.backward(g)

    phases = jc._phase_counts(k, d)
    ext_in = tuple(-(-i // q) for i, q in zip(insp, phases))
    pad0 = tuple(pp // q for pp, q in zip(p, phases))
    xb = jc._to_phases(x.detach(), phases, ext_in).requires_grad_()
    wb = w.detach().clone().requires_grad_()
    yb = conv(xb, wb, None, 1, pad0, 1)
    assert torch.allclose(jc._from_phases(yb.detach(), phases, 2, y.shape[2:]), y.detach(), atol=1e-12)
    gb = jc._to_phases(g, phases, tuple(yb.shape[2:]))
    yb.backward(gb)
    assert torch.allclose(jc._from_phases(xb.grad, phases, 2, insp), x.grad, atol=1e-12)
    assert torch.allclose(wb.grad, w.grad, atol=1e-10)
    # and the two permutations are inverses of each other on the cells that exist
    assert torch.equal(jc._from_phases(jc._to_phases(x.detach(), phases, ext_in), phases, 2, insp), x.detach())


@pytest.mark.parametrize("insp,k,p,d", [((13, 17), (3, 3), (1, 3), (2, 2)), ((12, 15), (5, 3), (3, 1), (2, 3)), ((7, 9, 11), (3, 3, 3), (0, 1, 2), (1, 2, 4))])
def test_a_zero_rim_makes_the_padding_a_multiple_of_the_dilation(insp, k, p, d):
    """The route for paddings that are no multiple of the dilation, with torch's CPU operators in place of the kernels."""
    ns = len(k)
    extra = jc._prepad(k, (1,) * ns, p, d)
    assert extra is not None and all((pp - e) % dd == 0 for pp, e, dd in zip(p, extra, d))
    conv = {2: F.conv2d, 3: F.conv3d}[ns]
    torch.manual_seed(0)
    x = torch.randn(2, 3, *insp, dtype=torch.float64, requires_grad=True)
    w = torch.randn(4, 3, *k, dtype=torch.float64, requires_grad=True)
    y = conv(x, w, None, 1, p, d)
    g = torch.randn_like(y)
    y.backward(g)
    xr = jc._zero_rim(x.detach(), extra).requires_grad_()
    wr = w.detach().clone().requires_grad_()
    rest = tuple(pp - e for pp, e in zip(p, extra))
    yr = conv(xr, wr, None, 1, rest, d)
    assert yr.shape == y.shape and torch.allclose(yr, y.detach(), atol=1e-12)
    yr.backward(g)
    inner = (slice(None), slice(None)) + tuple(slice(e, e + v) for v, e in zip(insp, extra))
    assert torch.allclose(xr.grad[inner], x.grad, atol=1e-12) and torch.allclose(wr.grad, w.grad, atol=1e-10)


def test_the_dilated_route_takes_only_what_it_covers():
    assert not jc._dilated_ok((3, 3), (1, 1), (1, 1), (2, 2))      # padding not a multiple of the dilation
    assert not jc._dilated_ok((3, 3), (2, 1), (2, 2), (2, 2))      # strided: through the stride-1 route first
    assert jc._dilated_ok((5, 3), (1, 1), (4, 2), (2, 2))          # five taps: the residue images take the tap-block route
    assert not jc._dilated_ok((11, 11), (1, 1), (10, 10), (2, 2))  # ... where that route takes the undilated layer
    assert not jc._dilated_ok((3, 3), (1, 1), (1, 1), (1, 1))      # nothing dilated
    assert jc._dilated_ok((1, 3), (1, 1), (0, 4), (7, 2))          # a dilation on a one-tap axis means nothing
    assert jc._dense_stride_ok((3, 3), (2, 2), (2, 2), (2, 2)) and jc._dense_stride_ok((3, 3), (2, 2), (2, 2), (1, 1))
    # a padding that is no multiple of the dilation: the remainder is laid around the input as zeros
    assert jc._prepad((3, 3), (1, 1), (1, 1), (2, 2)) == (1, 1) and jc._prepad((3, 3), (1, 1), (3, 4), (2, 2)) == (1, 0)
    assert jc._prepad((3, 3), (1, 1), (2, 4), (2, 2)) is None and jc._prepad((3, 1), (1, 1), (1, 3), (1, 2)) is None
    assert jc._prepad((3, 3), (2, 1), (1, 1), (2, 2)) is None


@pytest.mark.parametrize("insp,k,p", [
    ((12, 13), (5, 5), (2, 2)), ((11, 14), (7, 4), (3, 0)), ((9, 10), (5, 3), (0, 1)), ((6, 9, 10), (5, 3, 4), (2, 1, 0)),
    ((10, 10), (9, 9), (4, 4)), ((12, 12), (2, 5), (0, 2)), ((9, 11), (2, 2), (1, 0)), ((8, 9), (2, 3), (0, 1)), ((6, 7, 8), (1, 2, 2), (0, 1, 1)),
])
def test_tap_blocks_are_channel_blocks_of_a_three_tap_layer(insp, k, p):
    """The route of kernels with more than three taps, with torch's CPU operators in place of the
    kernels: forward and weight gradient of the three-tap layer over the moved copies of the input,
    input gradient as the forward of the output gradient under the transposed, reversed kernel."""
    ns = len(k)
    assert jc._big_kernel_ok(k, (1,) * ns, (1,) * ns)
    conv = {2: F.conv2d, 3: F.conv3d}[ns]
    torch.manual_seed(0)
    x = torch.randn(2, 3, *insp, dtype=torch.float64, requires_grad=True)
    w = torch.randn(4, 3, *k, dtype=torch.float64, requires_grad=True)
    y = conv(x, w, None, 1, p)
    g = torch.randn_like(y)
    y.backward(g)
    moved = jc._moved_copies(x.detach(), k, p, tuple(y.shape[2:])).requires_grad_()
    w3 = jc._tap_block_weight(w.detach()).requires_grad_()
    y3 = conv(moved, w3, None, 1, 0)
    assert y3.shape == y.shape and torch.allclose(y3, y.detach(), atol=1e-10)
    y3.backward(g)
    assert torch.allclose(jc._from_tap_blocks(w3.grad, w.shape), w.grad, atol=1e-9)
    if all(pp <= kk - 1 for pp, kk in zip(p, k)):
        back = w.detach().transpose(0, 1).flip(*range(2, 2 + ns))
        gx = conv(g, back, None, 1, tuple(kk - 1 - pp for pp, kk in zip(p, k)))
        assert gx.shape == x.shape and torch.allclose(gx, x.grad, atol=1e-9)


def test_the_tap_block_route_takes_only_what_it_covers():
    assert not jc._big_kernel_ok((3, 3), (1, 1), (1, 1))          # three taps: the kernels as they are
    assert not jc._big_kernel_ok((1, 3), (1, 1), (1, 1)) and jc._big_kernel_ok((2, 2), (1, 1), (1, 1))  # two taps: a block with a zero tap in front
    assert not jc._big_kernel_ok((5, 5), (2, 2), (1, 1))          # strided: through the stride-1 route first
    assert jc._dense_stride_ok((5, 5), (2, 2), (1, 1), (2, 2)) and not jc._dense_stride_ok((4, 4), (4, 4), (1, 1), (0, 0))
    assert not jc._big_kernel_ok((5, 5), (1, 1), (2, 1))          # dilated
    assert not jc._big_kernel_ok((11, 11), (1, 1), (1, 1))        # 16 blocks: too many copies of the input
    assert not jc._big_kernel_ok((5,), (1,), (1,))                # one axis: the direct kernels


def test_head_sizes_the_attention_host_pads_to():
    """fp32 without a bias goes to the head sizes of its matrix-core kernels, everything else to those
    of the one-thread-per-row kernels; a head size beyond the largest is passed on for the library to refuse."""
    from jigsaw_amd import attention as ja

    for d, want in ((1, 32), (8, 32), (32, 32), (33, 64), (64, 64), (72, 128), (96, 128), (128, 128), (129, 129)):
        assert ja._kernel_head_size(d, torch.float32, False) == want
    for d, want in ((1, 8), (8, 8), (9, 16), (33, 64), (72, 96), (96, 96), (100, 128), (129, 129)):
        assert ja._kernel_head_size(d, torch.float32, True) == want
        assert ja._kernel_head_size(d, torch.bfloat16, False) == want
        assert ja._kernel_head_size(d) == want


def test_general_span_plan_against_enumeration():
    """``spans_fit_the_strips`` and ``span_overlap`` (the host side of the axis-by-axis exchange) from first
    principles: output block r touches input rows ``o * s - p + d * t``; the rows of that range a peer owns are
    what it sends, and what one rank expects from a peer is what the peer cuts for it."""
    from jigsaw_amd.halo import needed_input_span, span_overlap, spans_fit_the_strips

    seen_general = seen_fit = 0
    for G, n, k, s, p, d in itertools.product((2, 3, 4), (2, 3, 5, 9), (1, 3, 5, 7), (1, 2), (0, 1, 3), (1, 2)):
        extent = d * (k - 1) + 1
        if G * n + 2 * p < extent:
            continue
        gout = (G * n + 2 * p - extent) // s + 1
        if gout % G:
            with pytest.raises(NotImplementedError):
                spans_fit_the_strips((n,), (k,), (s,), (p,), (d,), (G,))
            continue
        ol = gout // G
        fits = True
        for r in range(G):
            touched = sorted({o * s - p + d * t for o in range(r * ol, (r + 1) * ol) for t in range(k)})
            lo, hi, need, out_local = needed_input_span(r, G, n, k, s, p, d)
            assert (lo, hi - 1, out_local) == (touched[0], touched[-1], ol) and need == hi - lo
            own = range(r * n, (r + 1) * n)
            fits &= lo <= own[0] and hi >= own[-1] + 1 and own[0] - lo <= n and hi - (own[-1] + 1) <= n
            for peer in range(G):
                r0, cnt = span_overlap(lo, hi, peer, n, G)
                rows = [g for g in range(lo, hi) if peer * n <= g < (peer + 1) * n]
                assert cnt == len(rows) and (cnt == 0 or r0 == rows[0])
        assert spans_fit_the_strips((n,), (k,), (s,), (p,), (d,), (G,)) == fits
        seen_general += not fits
        seen_fit += fits
    assert seen_general > 20 and seen_fit > 20
