"""
Pins for the CPU oracle.  The reference holds no golden vectors and cannot be
compiled or imported in this image, so every oracle function is checked against
something that does not share its code: the number format's closed form, a
bit-string construction, or the reference GPU kernel's own read/decode rules
(tests/kernel_rules.py).  A dropped term, a swapped index or a transposed
operand in the oracle fails at least one of these.
"""
import numpy as np
import pytest

import kernel_rules as kr


# --------------------------------------------------------------------------- binary16 helpers

def test_half_to_float_all_patterns(oracle):
    L = oracle.lib()
    pats = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = pats.view(np.float16).astype(np.float32)
    got = np.array([L.orc_half_to_float(int(p)) for p in pats], dtype=np.float32)
    ok = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert ok.all()


def test_float_to_half_matches_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    # random bit patterns, values straddling every rounding boundary of every binary16, and the edges
    f = rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    h = np.arange(0, 0x7c00, 7, dtype=np.uint16).view(np.float16).astype(np.float32)
    nxt = (np.arange(0, 0x7c00, 7, dtype=np.uint16) + 1).view(np.float16).astype(np.float32)
    mid = (h.astype(np.float64) + nxt.astype(np.float64)) / 2
    around = np.concatenate([mid, np.nextafter(mid.astype(np.float32), np.float32(np.inf)),
                             np.nextafter(mid.astype(np.float32), np.float32(-np.inf))]).astype(np.float32)
    edge = np.array([0, -0.0, 65504, 65519.99, 65520, 1e9, 2 ** -24, 2 ** -25, 2 ** -25 * 1.0001, 2 ** -26,
                     np.inf, -np.inf], dtype=np.float32)
    vals = np.concatenate([f, around, -around, edge])
    vals = vals[~np.isnan(vals)]
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_float_to_half(float(v)) for v in vals], dtype=np.uint16)
    assert (got == want).all()


# --------------------------------------------------------------------------- FP6 cast (Q1/Q2)

def test_fp6_grid_is_the_closed_form():
    assert np.array_equal(kr.fp6_value(np.arange(32)), kr.FP6_GRID)
    assert np.array_equal(kr.fp6_value(np.arange(32, 64)), -kr.FP6_GRID)


def test_fp6_cast_exhaustive(oracle):
    """All 65,536 binary16 inputs: in range -> truncation toward zero onto the e3m2 grid, sign kept;
    out of range -> error (weight_quant.cpp:48-53)."""
    grid = kr.fp6_value(np.arange(32))
    zero3 = [0, 0, 0]
    for p in range(65536):
        v = float(np.uint16(p).view(np.float16))
        mag = abs(v)
        bad = (mag != mag) or (mag != 0 and mag < 0.0625) or mag > 28
        if bad:
            with pytest.raises(oracle.OracleError):
                oracle.fp6_cast4([p] + zero3)
            continue
        out = oracle.fp6_cast4([p] + zero3)
        code = int(out[0]) >> 2
        want = int(np.searchsorted(grid, mag, side="right") - 1) | ((p >> 15) << 5)
        assert code == want, (hex(p), v, code, want)


def test_fp6_cast_byte_packing(oracle):
    """Four codes are laid down MSB first as one 24-bit string (weight_quant.cpp:93-95)."""
    rng = np.random.default_rng(1)
    for _ in range(200):
        codes = rng.integers(0, 64, 4)
        vals = kr.fp6_value(codes).astype(np.float16)
        # -0.0 must keep its sign: build bit patterns by hand
        bits = vals.view(np.uint16) | np.where((codes >> 5) == 1, 0x8000, 0).astype(np.uint16)
        out = oracle.fp6_cast4(bits)
        s = "".join(format(int(c), "06b") for c in codes)
        want = [int(s[0:8], 2), int(s[8:16], 2), int(s[16:24], 2)]
        assert list(out) == want


def test_fp6_quantize_rows_and_flat_view(oracle):
    """Row quantiser = per-row cast; the torch-level wrapper reads the *flat* buffer as [IC, OC]
    (pybind.cpp:52-57 passes the storage of the transposed view)."""
    rng = np.random.default_rng(2)
    codes = rng.integers(0, 64, (256, 512)).astype(np.uint8)
    w = kr.fp6_value(codes).astype(np.float16)
    w.view(np.uint16)[(codes >> 5) == 1] |= 0x8000
    q = oracle.fp6_quantize(w)                       # OC=256, IC=512 -> [512, 256*3/16]
    assert q.shape == (512, 48) and q.dtype == np.int32
    flat_codes = codes.reshape(-1).reshape(512, 256)  # NOT a transpose
    assert np.array_equal(q.view(np.uint8).reshape(512, -1), kr.pack_fp6_rows(flat_codes))
    with pytest.raises(oracle.OracleError):
        oracle.fp6_quantize(w[:, :128].copy())        # not a multiple of 256
    w[3, 5] = 29.0
    with pytest.raises(oracle.OracleError):
        oracle.fp6_quantize(w)


# --------------------------------------------------------------------------- FP6 prepack (P)

@pytest.mark.parametrize("rows,cols", [(64, 64), (128, 64), (64, 192), (256, 256), (256, 512), (512, 256)])
def test_fp6_prepack_decodes_with_kernel_rules(oracle, rows, cols):
    """rows = output channels n, cols = input channels k.  Pack, then read the buffer the way the
    reference kernel does: every weight must come back at its (k, n)."""
    rng = np.random.default_rng(rows * 1000 + cols)
    codes = rng.integers(0, 64, (rows, cols)).astype(np.uint8)      # [n][k]
    packed = oracle.fp6_prepack_bytes(kr.pack_fp6_rows(codes), rows, cols)
    got = kr.decode_fp6(packed.view(np.int32), cols, rows)           # [k][n] float16
    want = kr.fp6_value(codes).T.astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16) | ((codes.T >> 5).astype(np.uint16) << 15))


def test_fp6_prepack_is_a_bit_permutation(oracle):
    rows, cols = 64, 128
    nbytes = rows * cols * 6 // 8
    rng = np.random.default_rng(3)
    x = rng.integers(0, 256, nbytes, dtype=np.uint8)
    y = rng.integers(0, 256, nbytes, dtype=np.uint8)
    px, py, pxy = (oracle.fp6_prepack_bytes(v, rows, cols) for v in (x, y, x ^ y))
    assert np.array_equal(px ^ py, pxy)                               # linear over GF(2)
    assert np.unpackbits(px).sum() == np.unpackbits(x).sum()          # popcount kept
    seen = set()
    for bit in rng.choice(nbytes * 8, 300, replace=False):           # one bit in -> one bit out, all distinct
        one = np.zeros(nbytes, dtype=np.uint8)
        one[bit // 8] = 0x80 >> (bit % 8)
        out = np.flatnonzero(np.unpackbits(oracle.fp6_prepack_bytes(one, rows, cols)))
        assert out.size == 1 and int(out[0]) not in seen
        seen.add(int(out[0]))


def test_fp6_prepack_shapes(oracle):
    q = np.zeros((256, 48), dtype=np.int32)                           # OC=256, IC=256
    assert oracle.fp6_prepack(q).shape == (24, 512)                   # [IC*3/32, OC*2]
    with pytest.raises(oracle.OracleError):
        oracle.fp6_prepack(np.zeros((128, 48), dtype=np.int32))
    with pytest.raises(oracle.OracleError):
        oracle.fp6_prepack_bytes(np.zeros(32 * 64 * 6 // 8, dtype=np.uint8), 32, 64)


# --------------------------------------------------------------------------- FP6 dequant (DQ)

def test_fp6_dequant_table_times_scale(oracle):
    rng = np.random.default_rng(4)
    rows, cols = 64, 128
    codes = rng.integers(0, 64, (rows, cols)).astype(np.uint8)
    codes[0, :64] = np.arange(64)
    scale = np.abs(rng.normal(0.01, 0.01, rows)).astype(np.float16) + np.float16(1e-4)
    scale[:4] = [1.0, 2.0 ** -14, 0.333, 60.0]
    got = oracle.fp6_dequant(kr.pack_fp6_rows(codes).reshape(rows, -1).view(np.int32), scale)
    want = (kr.fp6_value(codes).astype(np.float16) * scale[:, None]).astype(np.float16)   # one binary16 rounding
    assert np.array_equal(np.abs(got).view(np.uint16), np.abs(want).view(np.uint16))
    neg = (codes >> 5) == 1
    assert np.array_equal(np.signbit(got), neg)


# --------------------------------------------------------------------------- INT4 packer + scale order (I4/SP)

def test_marlin_perm_is_a_bijection(oracle):
    perm, sp = oracle.marlin_perms()
    assert sorted(perm.tolist()) == list(range(1024))
    assert sorted(sp.tolist()) == list(range(32))


@pytest.mark.parametrize("k,n", [(16, 64), (32, 128), (64, 256), (128, 192)])
def test_int4_pack_decodes_with_kernel_rules(oracle, k, n):
    rng = np.random.default_rng(k + n)
    codes = rng.integers(0, 16, (k, n)).astype(np.uint8)
    packed = oracle.int4_pack(codes)
    assert packed.shape == (k // 16, n * 2) and packed.dtype == np.int32
    got = kr.decode_int4(packed, k, n)
    assert np.array_equal(got, codes.astype(np.float16) - np.float16(8))


def test_scale_permutation_matches_kernel_epilogue(oracle):
    _, sp = oracle.marlin_perms()
    for col in range(32):
        assert sp[kr.scale_slot(col)] == col
    s = np.arange(96, dtype=np.float16)
    ps = oracle.permute_scales(s)
    for col in range(96):
        assert ps[32 * (col // 32) + kr.scale_slot(col % 32)] == s[col]


def test_int4_quantize_closed_form(oracle):
    """Symmetric 4-bit: s = max|w| * 2/15, code = clamp(round(w/s) + 8, 0, 15), w_ref = (code-8)*s,
    and the codes are a fixed point of re-quantising w_ref (test.py:98-101)."""
    rng = np.random.default_rng(5)
    w = rng.normal(0, 0.02, (256, 64)).astype(np.float16)
    for gs in (-1, 128):
        codes, s, ref = oracle.int4_quantize(w, gs)
        g = 256 if gs == -1 else gs
        assert s.shape == (256 // g, 64)
        amax = np.abs(w.reshape(256 // g, g, 64)).max(axis=1)
        assert np.allclose(s.astype(np.float64), amax.astype(np.float64) * 2 / 15, rtol=2e-3)   # (bit for bit: next test)
        srep = np.repeat(s, g, axis=0)
        assert np.array_equal(ref, ((codes.astype(np.float16) - np.float16(8)) * srep).astype(np.float16))
        assert codes.min() >= 0 and codes.max() <= 15
        assert np.abs(ref.astype(np.float64) - w.astype(np.float64)).max() <= srep.astype(np.float64).max() * 0.51 + 1e-6
        # the column maximum maps to +/-7.5 -> code 0/1 or 15/16 clamp: extremes are reached
        assert codes.max() == 15 or codes.min() <= 1


def test_int4_scale_and_codes_against_numpy_binary16(oracle):
    """The harness computes in torch CPU half arithmetic (test.py:88-92): every operation takes binary16 operands, is
    carried out in binary32 and rounded back to binary16.  The same steps in numpy, each rounding written out, must
    give the scale and the codes bit for bit: s = fp16(fp32(amax) * fp32(2/15)), code = clamp(rint(fp16(fp32(w) /
    fp32(s))) + 8, 0, 15)."""
    rng = np.random.default_rng(9)
    w = rng.normal(0, 0.02, (256, 96)).astype(np.float16)
    w[5, 3] = np.float16(0.3)                                            # an outlier: most of its column rounds to code 8
    for gs in (-1, 128):
        codes, s, ref = oracle.int4_quantize(w, gs)
        g = 256 if gs == -1 else gs
        amax = np.abs(w).reshape(256 // g, g, 96).max(axis=1)
        s_np = (amax.astype(np.float32) * np.float32(2 / 15)).astype(np.float16)
        assert np.array_equal(s.view(np.uint16), s_np.view(np.uint16))
        srep = np.repeat(s_np, g, axis=0)
        ratio = (w.astype(np.float32) / srep.astype(np.float32)).astype(np.float16)
        want = np.clip(np.rint(ratio.astype(np.float32)).astype(np.int32) + 8, 0, 15)
        assert np.array_equal(codes.astype(np.int32), want)
        ref_np = ((want - 8).astype(np.float16).astype(np.float32) * srep.astype(np.float32)).astype(np.float16)
        assert np.array_equal(ref.view(np.uint16), ref_np.view(np.uint16))


def test_int4_rounding_ties(oracle):
    """Constructed ties: with max|w| = 15/128 the scale is exactly 2^-6, so w = t * 2^-6 sits exactly half way between
    two codes for t = +-0.5 ... +-7.5.  torch.round (test.py:90) rounds half to even, and the clamp (test.py:92) cuts
    +8 to code 15: the expected codes below are written out by hand."""
    import torch
    import fp6_marlin
    ties = [0.5, 1.5, 2.5, 3.5, 4.5, 5.5, 6.5, 7.5]
    even = [0, 2, 2, 4, 4, 6, 6, 8]                                      # nearest even integer of each tie
    expect = {}
    for t, e in zip(ties, even):
        expect[t] = min(e + 8, 15)
        expect[-t] = max(-e + 8, 0)
    col = [t for t in ties] + [-t for t in ties]
    k = 128
    w = np.zeros((k, 64), dtype=np.float16)
    for c in range(64):
        w[: len(col), c] = (np.array(col, dtype=np.float64) / 64).astype(np.float16)     # t * 2^-6: exact in binary16
    assert np.abs(w).max() == np.float16(15 / 128)
    for gs in (-1, 128):
        codes, s, ref = oracle.int4_quantize(w, gs)
        assert (s == np.float16(2 ** -6)).all()
        for r, t in enumerate(col):
            assert (codes[r] == expect[t]).all(), (t, codes[r, 0], expect[t])
        assert (codes[len(col):] == 8).all()
        c2, s2, r2 = fp6_marlin.int4_quantize(torch.from_numpy(w), gs)  # the shipped host routine agrees on the ties
        assert np.array_equal(c2.numpy(), codes) and np.array_equal(s2.numpy(), s) and np.array_equal(r2.numpy(), ref)


# --------------------------------------------------------------------------- FP6 scale rule of the harness

def test_fp6_scale_rule_of_the_harness(oracle):
    """gen_fp6_weight's scale, threshold and clamp (test.py:19-27) against an evaluation that shares none of its
    lines (tests/fp6_scale_vectors.py): columns whose maxima are 28, 14 and 1.75 must get the scales 1, 0.5 and
    0.0625 exactly (a divisor other than 28 fails here); every e3m2 value and its binary16 neighbours must land on
    the right side of the truncation; entries below 0.0625 must come out as zero and an entry whose quotient rounds
    above 28 as +-28 (a dropped threshold or clamp makes the cast refuse them); random columns bit for bit."""
    import torch
    import fp6_marlin
    import fp6_scale_vectors as fv
    w = fv.vectors()
    k, n = w.shape
    s_want, ref_true = fv.expected(w)
    assert s_want[0] == 1.0 and s_want[1] == 0.5 and s_want[2] == 0.0625
    a = fv.over_range_maximum()
    assert ref_true[0, 3] == np.float16(np.float32(28) * np.float32(s_want[3])) and ref_true[1, 3] == -ref_true[0, 3]
    assert (ref_true[:, 0][np.abs(w[:, 0]) < 0.0625] == 0).all()
    # the harness itself (square w): codes of w / s, read back through its untransposed quantiser and dequantiser
    _, ref_want = fv.expected(w, harness=True)
    ref, packed, s_perm = oracle.gen_fp6_weight(w)
    s_nat = np.array([s_perm[32 * (c // 32) + kr.scale_slot(c % 32)] for c in range(n)], dtype=np.float16)
    assert np.array_equal(s_nat.view(np.uint16), s_want.view(np.uint16))
    assert np.array_equal(ref.astype(np.float32), ref_want.astype(np.float32))        # (+0 and -0 compare equal)
    # the shipped host packer (the rule's torch lines live there a second time) on the same vectors: the harness's
    # layout bit for bit, and the true transpose (what Layer.pack uses) against the plain evaluation
    B, s2, r2 = fp6_marlin.pack_mixed_weight(torch.from_numpy(w), n, -1)
    assert np.array_equal(B.numpy(), packed.reshape(-1)) and np.array_equal(s2.numpy(), s_perm)
    assert np.array_equal(r2.numpy().astype(np.float32), ref_want.astype(np.float32))
    B, s2, r2 = fp6_marlin.pack_mixed_weight(torch.from_numpy(w), n, -1, harness_layout=False)
    assert np.array_equal(s2.numpy(), s_perm)
    assert np.array_equal(r2.numpy().astype(np.float32), ref_true.astype(np.float32))
    assert np.array_equal((kr.decode_fp6(B.numpy(), k, n) * s_nat[None, :]).astype(np.float16).astype(np.float32),
                          ref_true.astype(np.float32))


# --------------------------------------------------------------------------- wire format (MX)

def test_mixed_wire_format(oracle):
    rng = np.random.default_rng(6)
    k, n, qc = 256, 512, 256
    w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
    ref, b, s = oracle.gen_mixed_weight(w, qc)
    n4 = n - qc
    assert b.dtype == np.int32 and b.size == k // 16 * 2 * n4 + k * 3 // 32 * 2 * qc    # test.py:146
    assert s.shape == (n,) and ref.shape == (k, n)
    # INT4 region decodes to (w_ref / s) exactly, FP6 region to w_ref = fp16(value * s)
    i4 = kr.decode_int4(b[: k // 16 * 2 * n4], k, n4)
    s_nat = np.empty(n, dtype=np.float16)
    for col in range(n):
        s_nat[col] = s[32 * (col // 32) + kr.scale_slot(col % 32)]
    assert np.array_equal((i4 * s_nat[None, :n4]).astype(np.float16), ref[:, :n4])
    f6 = kr.decode_fp6(b[k // 16 * 2 * n4:], k, qc)
    assert np.array_equal((f6 * s_nat[None, n4:]).astype(np.float16), ref[:, n4:])
    # all-INT4 and all-FP6 degenerate cases (test.py:125-128)
    _, b_all4, _ = oracle.gen_mixed_weight(w, -1)
    assert b_all4.size == k // 16 * 2 * n
    _, b_all6, _ = oracle.gen_mixed_weight(w[:, :256].copy(), 256)
    assert b_all6.size == k * 3 // 32 * 2 * 256


def test_row_mix_wire_format(oracle):
    """The row-mixed operands (no reference counterpart): the INT4 words of the first rows and the FP6 planes of the
    last rows decode, with the kernel's decode rules, to the check weight the function returns; sizes and scale
    layout are those the GEMM entry documents."""
    rng = np.random.default_rng(8)
    k, n, qr = 384, 256, 128
    k4 = k - qr
    w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
    ref, b, s = oracle.gen_row_mix_weight(w, qr)
    words4 = k4 * n // 8
    assert b.dtype == np.int32 and b.size == words4 + qr * n * 3 // 16
    assert s.size == (k4 // 128) * n + n and ref.shape == (k, n)
    i4 = kr.decode_int4(b[:words4], k4, n)                               # nibble - 8
    s4 = s[: (k4 // 128) * n].reshape(k4 // 128, n)                      # natural column order, one row per group
    assert np.array_equal((i4 * np.repeat(s4, 128, axis=0)).astype(np.float16), ref[:k4])
    f6 = kr.decode_fp6(b[words4:], qr, n)
    s6 = s[(k4 // 128) * n:]
    s6_nat = np.array([s6[32 * (c // 32) + kr.scale_slot(c % 32)] for c in range(n)], dtype=np.float16)
    assert np.array_equal((f6 * s6_nat[None, :]).astype(np.float16), ref[k4:])
    # the shipped packer builds the same buffers from the same two routines (FP6 part in the harness layout)
    import torch
    import fp6_marlin
    wt = torch.from_numpy(w)
    b4, s4p, r4 = fp6_marlin.pack_mixed_weight(wt[:k4].contiguous(), -1, 128)
    b6, s6p, r6 = fp6_marlin.pack_mixed_weight(wt[k4:].contiguous(), n, -1, harness_layout=True)
    assert np.array_equal(torch.cat([b4, b6]).numpy(), b) and np.array_equal(torch.cat([s4p, s6p]).numpy(), s)
    assert np.array_equal(torch.cat([r4, r6], 0).numpy(), ref)
