"""The gfx950 word order of the packed weight (fp6m_repack_gfx950 / fp6_marlin.repack_gfx950).

CPU part: the C routine and the tensor-permute mirror agree, both are lossless, and a brute-force walk over
(tile, k-block, lane) places every granule where the layout's definition says: lane 16 i + 8 sigma + l of tile t holds
the reference granule of 64-column group 2 t + sigma, fragment owner 4 l + i (weight_prepacking.cpp:142-150,
test.py:62-72 give the owner's (k, n) elements; the MFMA operand order is the kernel's).

GPU part: the GEMM on the repacked words equals the GEMM on the reference words bit for bit, for all three kernels,
both mixes, group and column scales.
"""

import numpy as np
import pytest
import torch


def random_words(k, n, qc, qr, seed=0):
    qcc = 0 if qc == -1 else qc
    words = ((k - qr) * n // 8 + qr * n * 3 // 16) if qr else (k * (n - qcc) // 8 + k * qcc * 3 // 16)
    g = torch.Generator().manual_seed(seed)
    return torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), generator=g, dtype=torch.int64).to(torch.int32)


CASES = [(256, 512, 128, 0), (128, 256, -1, 0), (64, 256, 256, 0), (384, 256, -1, 128), (48, 384, 256, 0)]


@pytest.mark.parametrize("k,n,qc,qr", CASES)
def test_both_converters_agree_and_invert(k, n, qc, qr):
    import fp6_marlin
    B = random_words(k, n, qc, qr)
    a = fp6_marlin.repack_gfx950(B, k, n, qc, qr)
    b = fp6_marlin.repack_gfx950_host(B, k, n, qc, qr)
    assert torch.equal(a, b)
    assert not torch.equal(a, B)
    assert torch.equal(torch.sort(a.view(-1))[0], torch.sort(B.view(-1))[0])       # same words, another order
    assert torch.equal(fp6_marlin.repack_gfx950(a, k, n, qc, qr, to_gfx950=False), B)
    assert torch.equal(fp6_marlin.repack_gfx950_host(a, k, n, qc, qr, to_gfx950=False), B)


def test_granule_placement_by_brute_force():
    import fp6_marlin
    k, n, qc = 64, 384, 128
    n4 = n - qc
    B = random_words(k, n, qc, 0, seed=1).numpy().view(np.uint32)
    nat = fp6_marlin.repack_gfx950_host(torch.from_numpy(B.view(np.int32)), k, n, qc).numpy().view(np.uint32)
    words4, words2 = k * n4 // 8, k * qc // 16
    for off, cols, words in ((0, n4, 4), (words4, qc, 2), (words4 + words2, qc, 4)):
        kblocks, tiles = k // 16, cols // 128
        for t in range(tiles):
            for kb in range(kblocks):
                for lane in range(64):
                    i, sigma, l = lane >> 4, (lane >> 3) & 1, lane & 7
                    ref = off + ((kb * (cols // 64) + 2 * t + sigma) * 32 + 4 * l + i) * words
                    got = off + ((t * kblocks + kb) * 64 + lane) * words
                    assert np.array_equal(nat[got:got + words], B[ref:ref + words]), (off, t, kb, lane)


def test_converter_shape_errors():
    import fp6_marlin
    with pytest.raises(ValueError):
        fp6_marlin.repack_gfx950(random_words(64, 256, 64, 0), 64, 256, 64)          # 64-column FP6 region: no whole tile
    with pytest.raises(ValueError):
        fp6_marlin.repack_gfx950(torch.zeros(10, dtype=torch.int32), 64, 256, -1)
    with pytest.raises(ValueError):
        fp6_marlin.repack_gfx950_host(torch.zeros(64 * 256 // 8, dtype=torch.float32), 64, 256)


# ------------------------------------------------------------------------------------------------ GPU

def gpu_case(oracle, m, k, n, qc, gs, env=None):
    import fp6_marlin
    dev = torch.device("cuda:0")
    print(f"case gfx950 layout m={m} k={k} n={n} qc={qc} gs={gs} env={env}", flush=True)
    rng = np.random.default_rng(k + n + m)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
    ref, b, s = oracle.gen_mixed_weight(w, qc, gs, strict=False)
    B, sd = torch.from_numpy(b).to(dev), torch.from_numpy(s).to(dev)
    Bn = fp6_marlin.repack_gfx950(B, k, n, qc)                                          # on the GPU
    assert torch.equal(Bn.cpu(), fp6_marlin.repack_gfx950_host(B.cpu(), k, n, qc))
    A = torch.randn((m, k), generator=torch.Generator().manual_seed(m)).half().to(dev)
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev)
    with fp6_marlin.cabi.tuning(**{name[5:].lower(): value for name, value in (env or {}).items()}):
        want = torch.full((m, n), float("nan"), dtype=torch.half, device=dev)
        fp6_marlin.cabi.mul(A, B, want, sd, ws, qc, -1, -1, -1, 16, gs)
        got = torch.full((m, n), float("nan"), dtype=torch.half, device=dev)
        fp6_marlin.mul_fused(A, Bn, got, sd, ws, qc, gs, layout="gfx950")
        torch.cuda.synchronize()
    assert int(ws.abs().sum()) == 0
    assert torch.equal(got, want)
    assert oracle.rel_err(got.cpu().numpy(), oracle.matmul_ref(A.cpu().numpy(), ref)) <= 1e-3


@pytest.mark.gpu
def test_gemm_on_gfx950_layout_is_bit_identical():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from oracle import fp6m_oracle as oracle
    for m in (1, 4, 16, 32, 64, 200):
        gpu_case(oracle, m, 1024, 768, 256, 128)
        gpu_case(oracle, m, 512, 512, 256, -1)
    gpu_case(oracle, 16, 2048, 512, 512, -1)                                           # all FP6
    gpu_case(oracle, 16, 2048, 512, -1, 128)                                           # all INT4
    gpu_case(oracle, 300, 1024, 1024, 256, 128, {"FP6M_MB": 8})                        # 128-row tiles, forced
    gpu_case(oracle, 300, 1024, 1024, 256, 128, {"FP6M_MB": 4})


@pytest.mark.gpu
def test_row_mix_on_gfx950_layout_is_bit_identical():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fp6_marlin
    from oracle import fp6m_oracle as oracle
    dev = torch.device("cuda:0")
    k, n, qr = 1024 + 256, 512, 256
    w = np.random.default_rng(4).normal(0, 0.02, (k, n)).astype(np.float16)
    ref, b, s = oracle.gen_row_mix_weight(w, qr)
    B, sd = torch.from_numpy(b).to(dev), torch.from_numpy(s).to(dev)
    Bn = fp6_marlin.repack_gfx950(B, k, n, quant_rows=qr)
    assert torch.equal(fp6_marlin.repack_gfx950(Bn, k, n, quant_rows=qr, to_gfx950=False), B)
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev)
    for m in (1, 16, 48, 130):
        print(f"case gfx950 layout rows m={m}", flush=True)
        A = torch.randn((m, k), generator=torch.Generator().manual_seed(m)).half().to(dev)
        want = torch.empty((m, n), dtype=torch.half, device=dev)
        got = torch.empty((m, n), dtype=torch.half, device=dev)
        fp6_marlin.mul_rows(A, B, want, sd, ws, qr)
        fp6_marlin.mul_rows(A, Bn, got, sd, ws, qr, layout="gfx950")
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert oracle.rel_err(got.cpu().numpy(), oracle.matmul_ref(A.cpu().numpy(), ref)) <= 1e-3
