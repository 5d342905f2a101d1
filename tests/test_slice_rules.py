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


# ---- the decode kernel's generation-major wave order and its chunk sub-lists (gemm_sk.h: sk_generation_order, the
# sub-list selection at the top of sk_wave; fp6m_gemm.hip: the chunk lengths by generation)

def xcd_contiguous_id(b, total):
    q, r, x = total >> 3, total & 7, b & 7
    return x * q + min(x, r) + (b >> 3)


def sk_generation_order(b, total, gen_waves):
    if gen_waves == 0 or total <= gen_waves:
        return xcd_contiguous_id(b, total)
    per = gen_waves >> 3
    x, i = b & 7, b >> 3
    g = (i >= per) + (i >= 2 * per) + (i >= 3 * per)
    rest = total - g * gen_waves
    if rest >= gen_waves:
        return g * gen_waves + x * per + (i - g * per)
    return g * gen_waves + xcd_contiguous_id(((i - g * per) << 3) | x, rest)


def test_generation_major_order_is_a_permutation_that_keeps_generations_apart():
    for gen_waves in (0, 64, 1024):
        for total in (1, 7, 8, 63, 64, 65, 100, 128, 129, 200, 1023, 1024, 1025, 1800, 2047, 2048, 2049, 2784, 2816, 4096):
            if gen_waves and total > 4 * gen_waves:
                continue                                                 # (the host plans at most four generations)
            order = [sk_generation_order(b, total, gen_waves) for b in range(total)]
            assert sorted(order) == list(range(total)), (gen_waves, total)
            if gen_waves and total > gen_waves:
                for b, pos in enumerate(order):                           # workgroup b is of generation (b / 8) / (gen / 8)
                    assert pos // gen_waves == (b >> 3) // (gen_waves >> 3), (gen_waves, total, b)


def test_chunk_sub_lists_cover_every_tile_once():
    """Chunk j of the INT4 region -> (tile, first unit, units) through the three sub-lists, as the top of sk_wave does."""
    for units in (32, 64, 86, 224):
        for (ta, tb, tc), (qa, qb, qc) in [((252, 170, 26), (16, 11, 10)), ((5, 0, 0), (7, 7, 7)), ((3, 4, 5), (9, 5, 2)),
                                           ((0, 6, 1), (8, 3, 3))]:
            cpt = [-(-units // q) for q in (qa, qb, qc)]
            chunks = [ta * cpt[0], tb * cpt[1], tc * cpt[2]]
            covered = {}
            for j in range(sum(chunks)):
                if j >= chunks[0] + chunks[1]:
                    jj, tile0, q, c = j - chunks[0] - chunks[1], ta + tb, qc, cpt[2]
                elif j >= chunks[0]:
                    jj, tile0, q, c = j - chunks[0], ta, qb, cpt[1]
                else:
                    jj, tile0, q, c = j, 0, qa, cpt[0]
                if j < chunks[0]:
                    tile = (jj * (((1 << 40) + c - 1) // c)) >> 40           # 40-bit reciprocal (also serves drawn chunks)
                else:
                    tile = jj if c <= 1 else (jj * (((1 << 32) + c - 1) // c)) >> 32   # 32-bit multiply-high
                assert tile == jj // c
                kb = (jj - tile * c) * q
                length = min(q, units - kb)
                assert length > 0
                for u in range(kb, kb + length):
                    key = (tile0 + tile, u)
                    assert key not in covered
                    covered[key] = j
            assert len(covered) == (ta + tb + tc) * units


# ---- k slices by wave with the second wave of every SIMD given less (gemm_common.h: WaveRule / wave_rule_begin;
# fp6m_gemm.hip: make_wave_rule)

def make_wave_rule(units, ks, wk, young_pct):
    ks = max(ks, 1)
    per_part = units // ks
    lo = ly = per_part // wk
    if wk == 8 and per_part >= 16 and 0 < young_pct < 100:
        lo = (per_part * 100 + 2 * (100 + young_pct)) // (4 * (100 + young_pct))
        if 4 * lo > per_part:
            lo = per_part // 4
        ly = min((per_part - 4 * lo) // 4, lo)
    rem = units - ks * (4 * lo + (wk - 4) * ly)
    eo = min(rem, 4 * ks)
    return lo, ly, eo, rem - eo


def wave_rule_begin(rule, wk, part, wave):
    lo, ly, eo, ey = rule
    no, ny = 4, wk - 4
    eo_here = min(max(eo - no * part, 0), no)
    ey_here = min(max(ey - ny * part, 0), ny)
    base = part * (no * lo + ny * ly) + min(eo, no * part) + min(ey, ny * part)
    if wave < no:
        return base + wave * lo + min(wave, eo_here)
    y = wave - no
    return base + no * lo + eo_here + y * ly + min(y, ey_here)


def test_wave_slices_tile_the_k_range_and_favour_the_older_waves():
    for wk in (4, 8):
        for units in list(range(1, 70)) + [86, 128, 172, 224, 448]:
            for ks in (1, 2, 3, 4, 5, 7, 8, 16):
                if ks * wk > units and units > 8:
                    continue                                              # (the host keeps a unit for every wave)
                for pct in (100, 85, 70, 50):
                    rule = make_wave_rule(units, ks, wk, pct)
                    assert min(rule) >= 0 and rule[3] <= (wk - 4) * ks and rule[2] <= 4 * ks, (units, ks, wk, pct, rule)
                    pos = 0
                    for part in range(ks):
                        lens = []
                        for w in range(wk):
                            b, e = wave_rule_begin(rule, wk, part, w), wave_rule_begin(rule, wk, part, w + 1)
                            assert b == pos and e >= b, (units, ks, wk, pct, part, w)
                            pos = e
                            lens.append(e - b)
                        assert wave_rule_begin(rule, wk, part, wk) == (wave_rule_begin(rule, wk, part + 1, 0))
                        if wk == 8:
                            assert min(lens[:4]) >= max(lens[4:]), (units, ks, pct, lens)       # older waves never get less
                            if pct < 100 and units // ks >= 16:
                                assert sum(lens[4:]) <= sum(lens[:4])
                        assert max(lens[:4]) - min(lens[:4]) <= 1 and max(lens[4:] or [0]) - min(lens[4:] or [0]) <= 1
                    assert pos == units, (units, ks, wk, pct, rule)


# ---- two classes of INT4 tiles in the m <= 16 kernel (gemm_m16_kernel's index arithmetic)

def m16_place(b, groups6, ks6, groups4, ks4, groups4b, ks4b):
    """workgroup b -> (fp6, tile inside its region, part, parts, slot of its partial tile)"""
    wgs6 = groups6 * ks6
    fp6 = b < wgs6
    local = b if fp6 else b - wgs6
    wgs4 = groups4 * ks4
    later = (not fp6) and local >= wgs4
    if later:
        local -= wgs4
    groups = groups6 if fp6 else (groups4b if later else groups4)
    part = local // groups
    group = local - part * groups + (groups4 if later else 0)
    ks = ks6 if fp6 else (ks4b if later else ks4)
    if fp6:
        slot = group * ks6 + part
    elif later:
        slot = groups6 * ks6 + groups4 * ks4 + (group - groups4) * ks4b + part
    else:
        slot = groups6 * ks6 + group * ks4 + part
    return fp6, group, part, ks, slot


def test_two_classes_cover_every_tile_part_once():
    rng = np.random.default_rng(11)
    cases = [(2, 2, 252, 1, 22, 11), (0, 0, 24, 1, 8, 3), (2, 4, 4, 2, 6, 2), (1, 1, 1, 1, 1, 1), (2, 2, 10, 1, 0, 1)]
    cases += [tuple(int(v) for v in (rng.integers(0, 4), rng.integers(1, 9), rng.integers(1, 300), rng.integers(1, 6),
                                     rng.integers(0, 120), rng.integers(1, 14))) for _ in range(60)]
    for groups6, ks6, groups4, ks4, groups4b, ks4b in cases:
        if groups6 == 0:
            ks6 = 0
        wgs = groups6 * ks6 + groups4 * ks4 + groups4b * ks4b
        seen, slots = set(), set()
        for b in range(wgs):
            fp6, group, part, ks, slot = m16_place(b, groups6, ks6, groups4, ks4, groups4b, ks4b)
            assert 0 <= part < ks and 0 <= group < (groups6 if fp6 else groups4 + groups4b)
            assert ks == (ks6 if fp6 else (ks4 if group < groups4 else ks4b))
            assert (fp6, group, part) not in seen and slot not in slots and 0 <= slot < wgs
            seen.add((fp6, group, part))
            slots.add(slot)
        assert len(seen) == wgs
