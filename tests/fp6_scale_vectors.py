"""Constructed inputs and an independent evaluation of the FP6 scale rule of the reference's harness
(gen_fp6_weight, test.py:19-27: s = max|w| / 28 per column, w / s, zero below 0.0625, clamp to +-28, then the
truncating cast of weight_quant.cpp:27-96), written with numpy binary16 / binary32 arithmetic and the e3m2 value grid
instead of the torch lines that the oracle and the shipped packer share.  Used by the CPU pin and by the GPU packer's test."""
import numpy as np

GRID = np.array([0, .0625, .125, .1875, .25, .3125, .375, .4375, .5, .625, .75, .875, 1, 1.25, 1.5, 1.75, 2, 2.5, 3, 3.5,
                 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28], dtype=np.float64)      # the 32 magnitudes of e3m2, bias 3


def expected(w, harness=False):
    """(scales fp16 [n] in natural column order, dequantised weight fp16 [k, n]) for w fp16 [k, n].
    harness=True: what the reference's harness computes for a square w.  Its quantiser reads the flat [k, n] buffer as
    [n, k] without transposing (pybind.cpp:52-57) and its dequantiser multiplies row r of that buffer by scale r
    (weight_prepacking.cpp:212, test.py:32-38), so the code of w[r, c] / s[c] comes back as value * s[r] at [c, r]."""
    w = np.asarray(w, dtype=np.float16)
    amax = np.abs(w).max(axis=0)
    s = (amax.astype(np.float32) * np.float32(1.0 / 28.0)).astype(np.float16)          # one binary32 product, rounded once
    with np.errstate(divide="ignore", invalid="ignore"):
        x = (w.astype(np.float32) / s.astype(np.float32)[None, :]).astype(np.float16)  # one binary32 quotient, rounded once
    x = np.where(np.abs(x) < np.float16(0.0625), np.float16(0), x)
    x = np.clip(x, np.float16(-28), np.float16(28))
    mag = np.abs(x.astype(np.float64))
    v = GRID[np.searchsorted(GRID, mag, side="right") - 1] * np.sign(x.astype(np.float64))   # largest grid value <= |x|
    if harness:
        assert w.shape[0] == w.shape[1]
        return s, np.ascontiguousarray((v.astype(np.float32) * s.astype(np.float32)[:, None]).astype(np.float16).T)
    ref = (v.astype(np.float32) * s.astype(np.float32)[None, :]).astype(np.float16)   # exact product, rounded once
    return s, ref


def over_range_maximum():
    """A binary16 column maximum whose quotient by its own rounded scale rounds to more than 28: only the clamp keeps
    such an entry inside the cast's range."""
    for bits in range(0x2000, 0x5000):
        a = np.uint16(bits).view(np.float16)
        s = (np.float32(a) * np.float32(1.0 / 28.0)).astype(np.float16)
        if s > 0 and (np.float32(a) / np.float32(s)).astype(np.float16) > np.float16(28):
            return a
    raise AssertionError("no such maximum")


def vectors(k=256, n=256, seed=3):
    """fp16 [k, n]: column 0 has max 28 (scale exactly 1) and holds every positive grid value, the values just below
    and just above each, and values just below 0.0625; column 1 has max 14 (scale 0.5), column 2 max 1.75 (scale
    0.0625); column 3 a maximum whose own quotient rounds above 28; the rest are random columns."""
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
    g = GRID[1:].astype(np.float16)
    below = (g.view(np.uint16) - 1).view(np.float16)
    above = (g.view(np.uint16) + 1).view(np.float16)
    col = np.concatenate([g, below, above[:-1], -g, -below, np.array([0.0, -0.0, 0.06244, 0.03, 1e-4], dtype=np.float16)])
    assert col.size <= k and np.abs(col).max() == 28
    for c, top in ((0, 28.0), (1, 14.0), (2, 1.75)):
        w[:, c] = 0
        w[: col.size, c] = (col.astype(np.float32) * np.float32(top / 28.0)).astype(np.float16)   # exact: a power of two
    a = over_range_maximum()
    w[:, 3] = (rng.normal(0, 0.3, k).astype(np.float32) * np.float32(a) / 2).astype(np.float16).clip(-a, a)
    w[0, 3], w[1, 3] = a, -a
    return w
