"""The division-free k-slice and tile arithmetic of the GEMM kernels (gemm_common.h: SliceRule / slice_begin,
FastDiv / fast_div; fp6m_gemm.hip: make_rule / make_div), restated here to check the properties the kernels rely on:

* the slices of a rule tile [0, units) exactly, in order, with lengths q or q + 1 and the longer ones last;
* for the lock-step kernel: a slice with work can run the longest step count of its workgroup from its own begin
  without leaving [0, units), and a slice without work can run it from 0;
* the multiply-high quotient equals n // d for every divisor below 65536 and dividends below 65536.

The GPU tests exercise the compiled arithmetic itself (forced splits, single k units, ragged shapes).
"""
import numpy as np


def make_rule(units, nslices):
    return units // nslices, nslices - units % nslices             # q, first_long


def slice_begin(rule, i):
    q, first_long = rule
    return i * q + max(0, i - first_long)


def test_slices_tile_the_k_range():
    for units in list(range(1, 70)) + [224, 448, 1000]:
        for nslices in list(range(1, 40)) + [64, 128, 333]:
            rule = make_rule(units, nslices)
            b = [slice_begin(rule, i) for i in range(nslices + 1)]
            assert b[0] == 0 and b[-1] == units
            lens = np.diff(b)
            assert set(lens.tolist()) <= {rule[0], rule[0] + 1}
            assert (np.diff(lens) >= 0).all(), "longer slices must come last"


def test_lock_step_workgroups_stay_inside_k():
    for wk in (1, 2):
        for units in range(1, 40):
            for ks in range(1, 12):
                nslices = ks * wk
                rule = make_rule(units, nslices)
                for part in range(ks):
                    longest = rule[0] + (1 if part * wk + wk - 1 >= rule[1] else 0)
                    lens = [slice_begin(rule, part * wk + j + 1) - slice_begin(rule, part * wk + j) for j in range(wk)]
                    assert longest == max(lens)
                    for j in range(wk):
                        begin = slice_begin(rule, part * wk + j) if lens[j] else 0
                        assert begin + longest <= units


def test_multiply_high_quotient_is_exact():
    n = np.concatenate([np.arange(0, 2048), np.arange(65536 - 2048, 65536),
                        np.random.default_rng(0).integers(0, 65536, 4096)]).astype(np.uint64)
    for d in range(2, 65536, 7):
        magic = np.uint64((2 ** 32 + d - 1) // d)
        assert np.array_equal((n * magic) >> np.uint64(32), n // np.uint64(d)), d
    for d in (2, 3, 5, 255, 256, 257, 448, 32767, 32768, 65535):                    # and exhaustively for a few
        alln = np.arange(65536, dtype=np.uint64)
        magic = np.uint64((2 ** 32 + d - 1) // d)
        assert np.array_equal((alln * magic) >> np.uint64(32), alln // np.uint64(d)), d


# ---------------------------------------------------------------- equal shares of the m <= 16 kernel (gemm_sk.h)

def share(j, q, r):
    """Units of workgroup j: the first r workgroups hold q + 1."""
    begin = j * q + min(j, r)
    return begin, begin + q + (1 if j < r else 0)


def owner(x, q, r):
    head = r * (q + 1)
    return x // (q + 1) if x < head else r + (x - head) // q


def test_equal_shares_cover_every_unit_once_and_owner_inverts_them():
    rng = np.random.default_rng(0)
    cases = [(30, 32, 256), (446, 64, 512), (2, 32, 6), (94, 32, 500), (446, 224, 384), (1, 5, 3), (7, 1, 7), (3, 9, 2)]
    cases += [(int(rng.integers(1, 60)), int(rng.integers(1, 40)), 0) for _ in range(200)]
    for tiles, units, wgs in cases:
        total = tiles * units
        if wgs == 0:
            wgs = int(rng.integers(1, total + 1))
        wgs = min(wgs, total)
        q, r = divmod(total, wgs)
        covered = np.zeros(total, dtype=np.int32)
        touching = np.zeros(tiles, dtype=np.int32)
        for j in range(wgs):
            b, e = share(j, q, r)
            assert e - b in (q, q + 1) and e > b
            covered[b:e] += 1
            assert all(owner(x, q, r) == j for x in (b, e - 1))
            for t in range(b // units, (e - 1) // units + 1):        # the segments the kernel walks
                touching[t] += 1
        assert (covered == 1).all()
        for t in range(tiles):                                      # what the kernel takes as a tile's number of parts
            parts = owner((t + 1) * units - 1, q, r) - owner(t * units, q, r) + 1
            assert parts == touching[t], (tiles, units, wgs, t)


def test_forty_bit_reciprocal_division_is_exact_in_its_range():
    rng = np.random.default_rng(1)
    ds = np.unique(np.concatenate([np.arange(1, 300), rng.integers(1, 65536, 2000), [65535]])).astype(np.uint64)
    ns = np.unique(np.concatenate([np.arange(0, 2000), rng.integers(0, 1 << 24, 4000), [(1 << 24) - 1]])).astype(np.uint64)
    for d in ds.tolist():
        magic = ((1 << 40) + d - 1) // d
        assert magic < (1 << 41)
        got = (ns * np.uint64(magic)) >> np.uint64(40)              # n < 2^24, magic < 2^41: no overflow of 64 bits
        assert (got == ns // np.uint64(d)).all(), d


# ---- placement of the workgroups that share a tile on one XCD (gemm_common.h: xcd_place; fp6m_gemm.hip: the grid and
# the multiply-high constants of the m <= 16 launch).  A workgroup knows the XCD it runs on from the hardware; the only
# thing assumed about the dispatch is that workgroups 8i .. 8i+7 run on eight different XCDs, in any order.

def xcd_grid(tiles6, tiles4, ks6, ks4):
    most = 0
    for x in range(8):
        c6 = (tiles6 + 7 - x) >> 3
        g0 = (x - tiles6) & 7
        c4 = (tiles4 + 7 - g0) >> 3
        most = max(most, c6 * ks6 + c4 * ks4)
    per = (tiles4 >> 3, tiles6 >> 3)
    xmagic = [[((2 ** 32 + (per[r] + h) - 1) // (per[r] + h)) if per[r] + h >= 2 else 0 for h in range(2)] for r in range(2)]
    return 8 * most, xmagic


def xcd_place(b, x, tiles6, tiles4, ks6, ks4, xmagic):
    i = b >> 3
    c6 = (tiles6 + 7 - x) >> 3
    g0 = (x - tiles6) & 7
    c4 = (tiles4 + 7 - g0) >> 3
    w6 = c6 * ks6
    fp6 = i < w6
    li = i if fp6 else i - w6
    c = c6 if fp6 else c4
    lo = (tiles6 if fp6 else tiles4) >> 3
    magic = xmagic[1 if fp6 else 0][0 if c == lo else 1]
    part = li if c <= 1 else (li * magic) >> 32
    j = li - part * c
    group = (x if fp6 else g0) + 8 * j
    valid = c > 0 and part < (ks6 if fp6 else ks4)
    return valid, fp6, group, part, x


def test_xcd_placement_covers_every_tile_part_once_on_one_xcd():
    cases = [(t6, t4, k6, k4) for t6 in (0, 1, 2, 3, 4, 7, 8, 9, 17) for t4 in (0, 1, 5, 8, 30, 62, 78, 94, 170, 447)
             for (k6, k4) in ((1, 1), (2, 1), (4, 2), (16, 8), (6, 3), (5, 7), (1, 4))]
    for tiles6, tiles4, ks6, ks4 in cases:
        if tiles6 + tiles4 == 0:
            continue
        grid, xmagic = xcd_grid(tiles6, tiles4, ks6, ks4)
        seen = {}
        rng = np.random.default_rng(tiles6 * 1000 + tiles4)
        # XCD of every workgroup: a rotation per dispatch (what the hardware does) or any permutation per group of eight
        xcd_of = np.concatenate([rng.permutation(8) if tiles4 % 2 else (np.arange(8) + tiles6) % 8 for _ in range(grid // 8)])
        for b in range(grid):
            valid, fp6, group, part, x = xcd_place(b, int(xcd_of[b]), tiles6, tiles4, ks6, ks4, xmagic)
            if not valid:
                continue
            assert 0 <= group < (tiles6 if fp6 else tiles4) and 0 <= part < (ks6 if fp6 else ks4)
            key = (fp6, group, part)
            assert key not in seen, (tiles6, tiles4, ks6, ks4, b)
            seen[key] = x
        assert len(seen) == tiles6 * ks6 + tiles4 * ks4, (tiles6, tiles4, ks6, ks4)
        for (fp6, group, part), x in seen.items():                                   # all parts of a tile on one XCD
            assert x == seen[(fp6, group, 0)]
        assert grid <= 8 * (-(-(tiles6 * ks6 + tiles4 * ks4) // 8) + max(ks6, ks4) * 2)   # little padding
