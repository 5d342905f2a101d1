"""
Lane-level simulation, on the CPU, of how the gfx950 kernel routes packed words to MFMA operands
(fp6-marlin_amd/csrc/gemm_m16.h): linear 16-byte loads -> swizzled wave-private LDS slab -> permuted
reads -> in-register dequant -> v_mfma_f32_16x16x32_f16 with the weights as the 16-row operand.

The MFMA is modelled from its documented operand layout: lane L supplies row/column L % 16 and the
eight k-slots 8*(L / 16) .. +7; the result D[r][c] sits in lane c + 16*(r / 4), register r % 4.
If the index algebra of the kernel were wrong (owner/lane transposition, swizzle, k-slot order of the
activations, column of an accumulator), this test fails without needing a GPU.
"""
import numpy as np
import pytest

import kernel_rules as kr


def simulate_tile(words4, words2, a_tile, fp6):
    """words4: uint32 [2 kblocks][256] (1 KiB per k-block: 2 groups x 32 owners x 4 tiles)
    words2: uint32 [2][128] or None; a_tile: float [16 rows][32 k].  Returns D [128 columns][16 rows]."""
    lane = np.arange(64)
    i, c = lane >> 4, lane & 15
    sigma, l = c >> 3, c & 7
    owner = 32 * sigma + 4 * l + i
    wr4 = lane ^ ((lane >> 4) & 3)
    rd4 = owner ^ ((owner >> 4) & 3)
    wr2 = lane ^ ((lane >> 5) << 1)
    rd2 = owner ^ ((owner >> 5) << 1)

    q = np.zeros((2, 64, 4), dtype=np.uint32)
    t2 = np.zeros((2, 64, 2), dtype=np.uint32)
    for kb in range(2):
        slab = np.zeros((64, 4), dtype=np.uint32)
        slab[wr4] = words4[kb].reshape(64, 4)          # lane L stores its linear granule at wr4[L]
        q[kb] = slab[rd4]
        if fp6:
            slab2 = np.zeros((64, 2), dtype=np.uint32)
            slab2[wr2] = words2[kb].reshape(64, 2)
            t2[kb] = slab2[rd2]

    # activation operand: lane (m = L%16, i = L/16), slot 2d+e <- A[m][8d + 2i + e]
    aop = np.zeros((64, 8), dtype=np.float64)
    for d in range(4):
        for e in range(2):
            aop[:, 2 * d + e] = a_tile[c, 8 * d + 2 * i + e]

    out = np.zeros((128, 16), dtype=np.float64)
    for j in range(4):
        if fp6:
            r = [kr.dequant_8fp6(t2[kb][:, j >> 1] << np.uint32(4 * (j & 1)), q[kb][:, j]) for kb in range(2)]
        else:
            r = [kr.dequant_8int4(q[kb][:, j]) for kb in range(2)]
        for half in range(2):
            # join(r0[2h], r0[2h+1], r1[2h], r1[2h+1]) -> eight k-slots
            wop = np.concatenate([r[0][:, 4 * half:4 * half + 4], r[1][:, 4 * half:4 * half + 4]], axis=1).astype(np.float64)
            d = np.zeros((16, 16))
            for g in range(4):
                d += wop[16 * g:16 * g + 16] @ aop[16 * g:16 * g + 16].T     # D[row slot][m]
            # result register file: lane (m, qq) holds slots 4qq..4qq+3 -> columns 64*(qq>>1) + 16j + 8h + 4*(qq&1) + r
            for slot in range(16):
                qq, reg = slot >> 2, slot & 3
                out[64 * (qq >> 1) + 16 * j + 8 * half + 4 * (qq & 1) + reg] = d[slot]
    return out


@pytest.mark.parametrize("fp6", [False, True])
def test_wave_tile_matches_dequantise_then_matmul(oracle, fp6):
    rng = np.random.default_rng(11 + fp6)
    k, n = 32, 128
    a = rng.normal(0, 1, (16, k)).astype(np.float16).astype(np.float64)
    if fp6:
        kk = 64                                                 # the prepacker needs k % 64 == 0; use its first 32 rows
        codes = rng.integers(0, 64, (n, kk)).astype(np.uint8)
        packed = oracle.fp6_prepack_bytes(kr.pack_fp6_rows(codes), n, kk).view(np.uint32)
        n2 = kk * n * 2 // 32
        words2 = packed[:n2].reshape(4, 128)[:2]
        words4 = packed[n2:].reshape(4, 256)[:2]
        w = kr.fp6_value(codes).T[:k]                           # [k][n]
    else:
        codes = rng.integers(0, 16, (k, n)).astype(np.uint8)
        words4 = oracle.int4_pack(codes).view(np.uint32).reshape(2, 256)
        words2 = None
        w = codes.astype(np.float64) - 8
    got = simulate_tile(words4, words2, a, fp6)
    want = (a @ w).T                                             # [n][m]
    assert np.allclose(got, want, rtol=0, atol=1e-9)


def test_swizzles_are_bijections_and_bank_conflict_free():
    lane = np.arange(64)
    owner = 32 * ((lane & 15) >> 3) + 4 * (lane & 7) + (lane >> 4)
    for idx in (lane ^ ((lane >> 4) & 3), owner ^ ((owner >> 4) & 3)):
        assert sorted(idx.tolist()) == list(range(64))
        for grp in range(4):                                      # 16 lanes x 16 B must cover 16 distinct bank quads
            assert len(set((idx[16 * grp:16 * grp + 16] % 16).tolist())) == 16
    for idx in (lane ^ ((lane >> 5) << 1), owner ^ ((owner >> 5) << 1)):
        assert sorted(idx.tolist()) == list(range(64))
        for grp in range(2):                                      # 32 lanes x 8 B must cover 32 distinct bank pairs
            assert len(set((idx[32 * grp:32 * grp + 32] % 32).tolist())) == 32
