"""fp6m_mul_static, the entry point that allocates nothing (partial tiles in a static device array), through the C
ABI: bit-identical to fp6m_mul on two calls in a row, the second on a smaller problem, with a workspace that no other
entry point has seen and the device's free memory unchanged across the calls; and a clear refusal when a split needs
more scratch than the array holds."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def operands(m, k, n, qc, gs, seed):
    g = torch.Generator().manual_seed(seed)
    n4 = n - qc
    B = torch.randint(-2 ** 31, 2 ** 31 - 1, (k * n4 // 8 + k * qc * 3 // 16,), generator=g, dtype=torch.int64).to(torch.int32)
    s = (torch.rand((k // gs) * n4 + qc, generator=g) * 0.01 + 0.001).half()
    A = torch.randn((m, k), generator=g).half()
    return A.cuda(), B.cuda(), s.cuda()


def call(fn, A, B, C, s, ws, m, n, k, qc, gs):
    return fn(A.data_ptr(), B.data_ptr(), C.data_ptr(), s.data_ptr(), m, n, k, ws.data_ptr(), 0,
              torch.cuda.current_stream().cuda_stream, -1, -1, -1, 16, qc, gs)


def test_static_scratch_entry_matches_mul_on_consecutive_calls():
    from fp6_marlin import cabi
    L = cabi.lib
    assert L.fp6m_init(0) == cabi.OK
    qc, gs = 256, 128
    # every problem splits k across workgroups, so partial tiles go through the scratch; sizes shrink from call
    # to call (the array keeps the previous call's contents), across all three kernels
    # (the 256-row case on 13824 x 5120 is one where the dispatcher's rule for 128-row tiles with a k split must
    # look at this entry point's smaller scratch: with the region's 16 MiB in mind it picked a split of 15.75 MiB)
    probs = [(16, 8192, 4096), (1, 4096, 4096), (1, 2048, 512), (128, 8192, 2048), (256, 13824, 5120), (40, 4096, 1024),
             (24, 2048, 512)]
    for i, (m, k, n) in enumerate(probs):
        print(f"case static m={m} k={k} n={n}", flush=True)
        A, B, s = operands(m, k, n, qc, gs, 50 + i)
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda")
        ws_static = torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda")   # never passed to any other entry point
        want = torch.full((m, n), float("nan"), dtype=torch.half, device="cuda")
        assert call(L.fp6m_mul, A, B, want, s, ws, m, n, k, qc, gs) == cabi.OK
        torch.cuda.synchronize()
        gots = [torch.full((m, n), float("nan"), dtype=torch.half, device="cuda") for _ in range(2)]
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for rep in range(2):
            assert call(L.fp6m_mul_static, A, B, gots[rep], s, ws_static, m, n, k, qc, gs) == cabi.OK
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "fp6m_mul_static allocated device memory"
        for rep in range(2):
            assert torch.isfinite(gots[rep]).all()
            if (m, k, n) == (256, 13824, 5120):
                # the two entry points tile this one differently (128-row tiles with a k split of three need 15.75 MiB
                # of partial tiles: the region has them, the array does not), so the fp32 sums are taken in another
                # order: equal to within fp16 rounding of sums of this size, and the two static calls equal bit for bit
                assert torch.allclose(gots[rep].float(), want.float(), rtol=2e-3, atol=2e-3), rep
                assert float((gots[rep] != want).float().mean()) < 0.05
                assert torch.equal(gots[rep], gots[0])
            else:
                assert torch.equal(gots[rep], want), (m, k, n, rep)
        assert int(ws_static.abs().sum()) == 0
        cabi.release_workspace(ws)


def test_static_scratch_entry_refuses_what_does_not_fit():
    from fp6_marlin import cabi
    L = cabi.lib
    m, k, n, qc, gs = 64, 8192, 8192, 256, 128
    A, B, s = operands(m, k, n, qc, gs, 60)
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device="cuda")
    C = torch.zeros((m, n), dtype=torch.half, device="cuda")
    with cabi.tuning(ksplit=8):                                          # 66 tile slots x 8 parts x 32 KiB > 12 MiB
        assert call(L.fp6m_mul_static, A, B, C, s, ws, m, n, k, qc, gs) == cabi.ERR_SCRATCH
        assert call(L.fp6m_mul, A, B, C, s, ws, m, n, k, qc, gs) == cabi.OK      # the region-backed entry shrinks the split
    assert "fp6m_mul has room" in cabi.strerror(cabi.ERR_SCRATCH)
    assert call(L.fp6m_mul_static, A, B, C, s, ws, m, n, k, qc, gs) == cabi.OK    # the dispatcher's own split fits
    torch.cuda.synchronize()
    assert int(ws.abs().sum()) == 0
