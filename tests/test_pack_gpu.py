"""On-GPU weight preparation against the host path (which tests/test_cpu_routines.py pins to the oracle bit for
bit): packed words, scales and the dequantised check weight must be identical."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def same_bits(a, b):
    return torch.equal(a.cpu().contiguous().view(torch.int16), b.cpu().contiguous().view(torch.int16))


def same_values(a, b):
    # the host INT4 check weight writes +0 where the GPU kernel writes the product's sign: compare as numbers
    return np.array_equal(a.cpu().numpy().astype(np.float32), b.cpu().numpy().astype(np.float32))


@pytest.mark.parametrize("k,n,qc,gs", [(256, 512, 256, 128), (256, 512, 256, -1), (512, 768, 128, 128), (256, 256, 256, -1),
                                       (256, 512, -1, 128), (1024, 1024, 512, -1), (128, 192, 64, 128)])
@pytest.mark.parametrize("harness", [True, False])
def test_device_pack_matches_host_pack(k, n, qc, gs, harness):
    import fp6_marlin
    g = torch.Generator().manual_seed(k * 7 + n + (qc if qc > 0 else 0))
    w = (torch.randn((k, n), generator=g) * 0.02).half()
    w[3, 5] = 0.0
    n4 = n - max(qc, 0)
    if n4 > 7:
        w[:, 7] = 0.0                                                 # an all-zero INT4 column: scale 0, codes 8
    if qc > 0 and not harness:
        w[:, n4 + 3] = 0.0                                            # an all-zero FP6 column: its scale becomes 1
    Bh, sh, rh = fp6_marlin.pack_mixed_weight(w, qc, gs, harness_layout=harness)
    Bd, sd, rd = fp6_marlin.pack_mixed_weight(w.to(dev()), qc, gs, harness_layout=harness)
    assert Bd.is_cuda and sd.is_cuda and rd.is_cuda
    assert torch.equal(Bd.cpu(), Bh)
    assert same_bits(sd, sh)
    assert same_values(rd, rh)


def test_every_fp6_code_and_range_errors():
    """A column whose largest magnitude is 28 has scale 1, so its entries are cast as they are: feed every
    binary16 pattern inside [0.0625, 28] (and both zeros) through the GPU cast and compare with the host's."""
    import fp6_marlin
    allh = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    mag = allh.float().abs()
    ok = allh[((mag >= 0.0625) & (mag <= 28.0)) | (mag == 0)]
    k, qc = 256, 128
    reps = (k * qc + ok.numel() - 1) // ok.numel()
    w6 = ok.repeat(reps)[: k * qc].reshape(k, qc).clone()
    w6[0, :] = 28.0                                                   # every column: max 28 -> scale 1
    w = torch.cat([torch.randn(k, 128).half() * 0.02, w6], dim=1).contiguous()
    for harness in (True, False):
        Bh, sh, rh = fp6_marlin.pack_mixed_weight(w, qc, -1, harness_layout=harness)
        Bd, sd, rd = fp6_marlin.pack_mixed_weight(w.to(dev()), qc, -1, harness_layout=harness)
        assert torch.equal(Bd.cpu(), Bh) and same_bits(sd, sh) and same_values(rd, rh)
    bad = w.clone()
    bad[5, 130] = float("nan")
    with pytest.raises(ValueError):
        fp6_marlin.pack_mixed_weight(bad.to(dev()), qc, -1)
    with pytest.raises(ValueError):                                   # shape rule: quant_cols % 64
        fp6_marlin.pack_mixed_weight(w.to(dev()), 96, -1)


def test_fp6_scale_rule_vectors_through_the_gpu_packer():
    """The constructed columns of tests/fp6_scale_vectors.py (exact scales 1, 0.5, 0.0625; values around every e3m2
    grid point; entries below the 0.0625 threshold; a quotient that rounds above 28) through the on-GPU packer: scales
    and check weight against the independent numpy evaluation, words against the host packer."""
    import fp6_marlin
    import fp6_scale_vectors as fv
    import kernel_rules as kr
    w = fv.vectors()
    k, n = w.shape
    s_want, ref_want = fv.expected(w)
    # (the harness layout reads the flat [k, n] buffer as [n, k] without transposing; with k == n that is the transpose)
    wt = torch.from_numpy(np.ascontiguousarray(w.T))
    Bd, sd, rd = fp6_marlin.pack_mixed_weight(wt.to(dev()), n, -1, harness_layout=True)
    Bh, sh, rh = fp6_marlin.pack_mixed_weight(wt, n, -1, harness_layout=True)
    assert torch.equal(Bd.cpu(), Bh) and same_bits(sd, sh) and same_values(rd, rh)
    Bd, sd, rd = fp6_marlin.pack_mixed_weight(torch.from_numpy(w).to(dev()), n, -1, harness_layout=False)
    s_perm = sd.cpu().numpy()
    s_nat = np.array([s_perm[32 * (c // 32) + kr.scale_slot(c % 32)] for c in range(n)], dtype=np.float16)
    assert np.array_equal(s_nat.view(np.uint16), s_want.view(np.uint16))
    assert np.array_equal(rd.cpu().numpy().astype(np.float32), ref_want.astype(np.float32))


def test_layer_pack_on_gpu_matches_cpu_and_runs():
    import fp6_marlin
    torch.manual_seed(3)
    lin = torch.nn.Linear(512, 768, bias=False).half()
    a = fp6_marlin.Layer(512, 768, groupsize=128, quant_cols=256)
    ref_cpu = a.pack(lin)
    b = fp6_marlin.Layer(512, 768, groupsize=128, quant_cols=256).to(dev())
    ref_gpu = b.pack(lin.to(dev()))
    assert torch.equal(b.B.cpu(), a.B) and same_bits(b.s, a.s) and same_values(ref_gpu, ref_cpu)
    x = torch.randn((4, 512), dtype=torch.half, device=dev())
    y = b(x)
    y_ref = x.float() @ ref_gpu.float()
    assert ((y.float() - y_ref).abs().mean() / y_ref.abs().mean()).item() <= 1e-3
