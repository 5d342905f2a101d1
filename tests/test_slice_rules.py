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
