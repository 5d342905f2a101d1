"""GPU tests of `mul_rows` (C ABI fp6m_mul_rows): INT4 rows and FP6 rows of the same columns accumulated into one
output tile.  The reference has no such kernel; the operands come from the oracle's composition of the reference
harness's two weight generators, and what pins the result:

* one-hot rows of A return rows of the dequantised weight bit for bit, from both segments (layout, scale order and
  the hand-over between the segments);
* the oracle's fp32 product within the GEMM tolerance (mean |d| / mean |ref| <= 1e-3) over m = 1 .. 300, forced
  k splits, segments of very different length;
* the two-launch formulation the reference would need (column-mix `mul` on the two row ranges, added in fp32)
  within the same tolerance.
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def oracle():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from oracle import fp6m_oracle
    return fp6m_oracle


def dev():
    return torch.device("cuda:0")


_cache = {}


def operands(oracle, k, n, qr, seed=0):
    key = (k, n, qr, seed)
    if key not in _cache:
        rng = np.random.default_rng(seed + 17 * k + n)
        w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
        ref, b, s = oracle.gen_row_mix_weight(w, qr)
        _cache[key] = (ref, torch.from_numpy(b).to(dev()), torch.from_numpy(s).to(dev()))
    return _cache[key]


def run(oracle, m, k, n, qr, ksplit=None, seed=0, **kw):
    import fp6_marlin
    print(f"case rows m={m} k={k} n={n} quant_rows={qr} ksplit={ksplit}", flush=True)
    ref, B, s = operands(oracle, k, n, qr, seed)
    A = torch.randn((m, k), generator=torch.Generator().manual_seed(m + seed)).half()
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
    outs = []
    with fp6_marlin.cabi.tuning(ksplit=ksplit):
        for _ in range(2):
            C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
            fp6_marlin.mul_rows(A.to(dev()), B, C, s, ws, qr, **kw)
            torch.cuda.synchronize()
            outs.append(C)
    assert int(ws.abs().sum()) == 0
    assert torch.equal(outs[0], outs[1]), "two identical calls differ"
    c = outs[0].cpu().numpy()
    assert np.isfinite(c).all()
    err = oracle.rel_err(c, oracle.matmul_ref(A.numpy(), ref))
    assert err <= TOL, err
    return A, outs[0]


def test_row_mix_against_oracle(oracle):
    for m in (1, 3, 16, 17, 32, 64, 100, 300):
        run(oracle, m, 1024, 512, 256)
    for k, qr in ((512, 256), (2048 + 64, 64), (1024 + 448, 448), (128 + 1024, 1024)):
        for m in (1, 16, 40):
            run(oracle, m, k, 256, qr)
    run(oracle, 16, 4096 + 256, 1024, 256)


def test_row_mix_forced_splits(oracle):
    for m in (2, 16, 48):
        for ks in (1, 2, 3, 8):
            run(oracle, m, 2048, 384, 256, ksplit=ks)


def test_row_mix_one_hot_rows_are_exact(oracle):
    import fp6_marlin
    k, n, qr = 640, 256, 128
    ref, B, s = operands(oracle, k, n, qr, seed=3)
    rows = [0, 1, 127, 128, 300, 511, 512, 513, 600, 639]              # the last five lie in the FP6 segment
    for m_pad in (len(rows), 40):
        A = torch.zeros((m_pad, k), dtype=torch.half)
        for i, r in enumerate(rows):
            A[i, r] = 1.0
        C = torch.full((m_pad, n), float("nan"), dtype=torch.half, device=dev())
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        fp6_marlin.mul_rows(A.to(dev()), B, C, s, ws, qr)
        torch.cuda.synchronize()
        got = C.cpu().numpy()[:len(rows)]
        assert np.array_equal(got.view(np.uint16) & 0x7fff != 0, ref[rows].view(np.uint16) & 0x7fff != 0)
        assert np.array_equal(got.astype(np.float32), ref[rows].astype(np.float32))


def test_row_mix_equals_two_column_mix_calls(oracle):
    """What the reference would do: one launch per row range (all INT4 / all FP6) and an addition."""
    import fp6_marlin
    k, n, qr = 1024, 512, 256
    k4 = k - qr
    for m in (1, 16, 70):
        A, C = run(oracle, m, k, n, qr)
        ref, B, s = operands(oracle, k, n, qr)
        words4, ns4 = k4 * n // 8, (k4 // 128) * n
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        c4 = torch.empty((m, n), dtype=torch.half, device=dev())
        c6 = torch.empty((m, n), dtype=torch.half, device=dev())
        fp6_marlin.cabi.mul(A[:, :k4].contiguous().to(dev()), B[:words4].contiguous(), c4, s[:ns4].contiguous(), ws, -1, -1, -1,
                            -1, 16, 128)
        fp6_marlin.cabi.mul(A[:, k4:].contiguous().to(dev()), B[words4:].contiguous(), c6, s[ns4:].contiguous(), ws, n, -1, -1,
                            -1, 16, -1)
        torch.cuda.synchronize()
        two = (c4.float() + c6.float()).cpu().numpy()
        assert oracle.rel_err(C.cpu().numpy(), two) <= TOL


def test_row_mix_with_gather_and_epilogue(oracle):
    import fp6_marlin
    k, n, qr = 1024, 512, 256
    ref, B, s = operands(oracle, k, n, qr)
    g = torch.Generator().manual_seed(9)
    for m in (1, 16, 90):
        A = torch.randn((m, k), generator=g).half()
        # the FP6 rows multiply 256 scattered input channels, the INT4 rows the others in order
        picked = torch.randperm(k, generator=g)[:qr].sort().values
        rest = torch.tensor(sorted(set(range(k)) - set(picked.tolist())))
        a_cols = torch.cat([rest, picked]).to(torch.int32)
        c_cols = torch.randperm(n, generator=g).to(torch.int32)
        bias = torch.randn(n, generator=g).half()
        C = torch.full((m, n), float("nan"), dtype=torch.half, device=dev())
        ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
        fp6_marlin.mul_rows(A.to(dev()), B, C, s, ws, qr, a_cols=a_cols.to(dev()), c_cols=c_cols.to(dev()), bias=bias.to(dev()))
        torch.cuda.synchronize()
        prod = oracle.matmul_ref(A[:, a_cols.long()].numpy(), ref)
        want = np.empty_like(prod)
        want[:, c_cols.numpy()] = prod
        want += bias.float().numpy()
        assert oracle.rel_err(C.cpu().numpy(), want) <= TOL


def test_row_mix_packer_and_errors(oracle):
    import fp6_marlin
    k, n, qr = 768, 256, 256
    w = (torch.randn((k, n), generator=torch.Generator().manual_seed(2)) * 0.02).half()
    B, s, w_ref = fp6_marlin.pack_row_mix_weight(w, qr)
    Bd, sd, w_ref_d = fp6_marlin.pack_row_mix_weight(w.to(dev()), qr)           # packed on the GPU: same bits
    assert torch.equal(B, Bd.cpu()) and torch.equal(s, sd.cpu()) and torch.equal(w_ref, w_ref_d.cpu())
    assert ((w_ref.float() - w.float()).abs().mean() / w.float().abs().mean()).item() < 0.2      # INT4 and e3m2 quantisation error
    A = torch.randn((5, k), generator=torch.Generator().manual_seed(3)).half()
    C = torch.empty((5, n), dtype=torch.half, device=dev())
    ws = torch.zeros(n // 128 * 16, dtype=torch.int32, device=dev())
    fp6_marlin.mul_rows(A.to(dev()), Bd, C, sd, ws, qr)
    torch.cuda.synchronize()
    assert oracle.rel_err(C.cpu().numpy(), oracle.matmul_ref(A.numpy(), w_ref.numpy())) <= TOL
    with pytest.raises(RuntimeError):
        fp6_marlin.mul_rows(A.to(dev()), Bd, C, sd, ws, 0)
    with pytest.raises(RuntimeError):
        fp6_marlin.mul_rows(A.to(dev()), Bd, C, sd, ws, k)
    with pytest.raises(RuntimeError, match="not compatible"):
        fp6_marlin.mul_rows(A.to(dev()), Bd, C, sd, ws, 192)                      # 768 - 192 is no multiple of 128
    with pytest.raises(ValueError):
        fp6_marlin.pack_row_mix_weight(w, 100)


def test_layer_with_fp6_input_features(oracle):
    """`Layer(quant_rows=..., fp6_in_channels=...)`: chosen input features in FP6, gathered inside the call; the check
    weight comes back in the linear layer's own order; both word orders agree bit for bit; checkpoints carry the mix."""
    import fp6_marlin
    torch.manual_seed(4)
    k, n, qr = 768, 512, 256
    lin = torch.nn.Linear(k, n, bias=True).half()
    picked = torch.randperm(k)[:qr]
    x = torch.randn((5, k), dtype=torch.half)
    outs = []
    for layout in ("reference", "gfx950"):
        layer = fp6_marlin.Layer(k, n, groupsize=128, quant_rows=qr, fp6_in_channels=picked, bias=True, layout=layout)
        w_ref = layer.pack(lin)
        err = (w_ref.float() - lin.weight.data.t().float()).abs().mean(1) / lin.weight.data.t().float().abs().mean(1)
        assert err.max() < 0.3                                         # row order restored (a wrong order gives ~1.4)
        layer = layer.to(dev())
        y = layer(x.to(dev())).cpu()
        y_ref = x.float() @ w_ref.float() + lin.bias.data.float()
        assert oracle.rel_err(y.numpy(), y_ref.numpy()) <= TOL
        outs.append(y)
        clone = fp6_marlin.Layer(k, n, groupsize=128, quant_rows=qr, fp6_in_channels=picked, bias=True, layout=layout)
        clone.load_state_dict(layer.state_dict())
        assert torch.equal(clone.to(dev())(x.to(dev())).cpu(), y)
        with pytest.raises(RuntimeError, match="does not match"):
            fp6_marlin.Layer(k, n, groupsize=128, quant_cols=256, bias=True, layout=layout).load_state_dict(layer.state_dict(), strict=False)
    assert torch.equal(outs[0], outs[1])
    with pytest.raises(ValueError):
        fp6_marlin.Layer(k, n, groupsize=-1, quant_rows=qr)
