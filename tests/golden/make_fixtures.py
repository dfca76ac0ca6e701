"""Writes the known-answer fixtures of this directory. Run: python tests/golden/make_fixtures.py

The reference holds no golden vectors for these operators (its tests compare with serial
torch operators on seeded data) and cannot be imported by this interpreter, so the vectors
here are derived independently of both the oracle and the kernels: integer brute force for
the span tables, exact rational / double arithmetic with explicit rounding for the
floating-point cases. Nothing in this script imports the package, the oracle or torch.
"""

import json
import math
import struct
from fractions import Fraction
from pathlib import Path

HERE = Path(__file__).parent


def f32(v: float) -> float:
    return struct.unpack("<f", struct.pack("<f", v))[0]


def bf16_bits(v: float) -> int:
    """Round-to-nearest-even to bfloat16; the 16-bit pattern."""
    (b,) = struct.unpack("<I", struct.pack("<f", v))
    b += 0x7FFF + ((b >> 16) & 1)
    return (b >> 16) & 0xFFFF


def bf16(v: float) -> float:
    return struct.unpack("<f", struct.pack("<I", bf16_bits(v) << 16))[0]


def spans() -> dict:
    """For every (G, n, k, s, p, d): which input rows does rank r's output block read
    (convolution), which output columns do rank r's inputs write (transposed convolution)?"""
    conv, convt = [], []
    for G in (1, 2, 3):
        for n in (4, 6):
            for k in (1, 2, 3, 5):
                for s in (1, 2):
                    for p in (0, 1, 2):
                        for d in (1, 2):
                            ext = d * (k - 1) + 1
                            gin = G * n
                            gout = (gin + 2 * p - ext) // s + 1
                            if gout > 0 and gout % G == 0:
                                ol = gout // G
                                for r in range(G):
                                    rows = [o * s - p + d * j for o in range(r * ol, (r + 1) * ol) for j in range(k)]
                                    conv.append([G, n, k, s, p, d, r, min(rows), max(rows) + 1, ol])
                            tout = (gin - 1) * s - 2 * p + ext
                            if tout > 0 and tout % G == 0:
                                for r in range(G):
                                    cols = [i * s - p + d * j for i in range(r * n, (r + 1) * n) for j in range(k)]
                                    convt.append([G, n, k, s, p, d, r, min(cols), max(cols) + 1 - min(cols), tout // G, tout])
    return {"conv_need_span": conv, "convt_raw_span": convt}


def fold_corner() -> dict:
    """Corner cell (0, 0) of the interior rank of a 3x3 mesh, halo width 1: the four terms
    are its own padded cell, the left neighbour's, the top neighbour's and the diagonal's.
    The reference folds W first, then H, each axis as ((0 + lower) + own) + upper with every
    add rounded to the storage type: (0 + (0 + diag + top)) + (0 + left + own)."""
    out = {}
    for name, rnd, tiny in (("float32", f32, 2.0**-24), ("bfloat16", bf16, 2.0**-8)):
        own, left, top, diag = 1.0, tiny, tiny, tiny
        w_top = rnd(rnd(rnd(0.0 + diag) + top))          # W fold of the halo row above: diag is its lower-W term
        w_own = rnd(rnd(rnd(0.0 + left) + own))          # W fold of the own row
        want = rnd(rnd(rnd(0.0 + w_top) + w_own))        # H fold
        naive = rnd(rnd(rnd(own + left) + top) + diag)   # a different association, for contrast
        out[name] = {"own": own, "left": left, "top": top, "diag": diag, "want": want, "other_order": naive}
        assert want != naive
    return out


def lse_merge() -> list:
    """(o1, l1) merged with (o2, l2): w = sigmoid(l2 - l1), o = o1 + w (o2 - o1),
    l = log(exp(l1) + exp(l2)); in double."""
    cases = []
    for o1, l1, o2, l2 in [(0.5, 0.0, -1.5, 0.0), (2.0, 3.0, -4.0, 1.0), (1.25, -7.5, 0.75, 2.5), (0.0, float("-inf"), 3.0, 0.25)]:
        if l1 == float("-inf"):
            w, l = 1.0, l2
        else:
            w = 1.0 / (1.0 + math.exp(l1 - l2))
            l = max(l1, l2) + math.log1p(math.exp(-abs(l1 - l2)))
        cases.append({"o1": o1, "l1": "-inf" if l1 == float("-inf") else l1, "o2": o2, "l2": l2, "o": o1 + w * (o2 - o1) if l1 != float("-inf") else o2, "l": l})
    return cases


def layernorm_two_shards() -> dict:
    """Row [1, 2, 3, 4 | 6, 8, 10, 12] split in two shards of four: partial mean / biased
    variance per shard, the combination, and the normalised row (eps = 0), exactly."""
    a, b = [Fraction(v) for v in (1, 2, 3, 4)], [Fraction(v) for v in (6, 8, 10, 12)]
    mean = lambda v: sum(v) / len(v)  # noqa: E731
    var = lambda v: sum((t - mean(v)) ** 2 for t in v) / len(v)  # noqa: E731
    m = (mean(a) + mean(b)) / 2
    v = (var(a) + (mean(a) - m) ** 2 + var(b) + (mean(b) - m) ** 2) / 2
    assert m == mean(a + b) and v == var(a + b)
    return {
        "shards": [[float(t) for t in a], [float(t) for t in b]],
        "partial_mean": [float(mean(a)), float(mean(b))],
        "partial_var": [float(var(a)), float(var(b))],
        "mean": float(m),
        "var": float(v),
        "normalised": [float(t - m) / math.sqrt(float(v)) for t in a + b],
    }


def main() -> None:
    (HERE / "spans.json").write_text(json.dumps(spans()))
    (HERE / "float_cases.json").write_text(json.dumps({"fold_corner": fold_corner(), "lse_merge": lse_merge(), "layernorm_two_shards": layernorm_two_shards()}, indent=1))


if __name__ == "__main__":
    main()
