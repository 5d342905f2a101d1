"""Shipped host routines (libfp6m.so through fp6_marlin) against the oracle: bit-exact, no GPU needed."""
import numpy as np
import pytest
import torch

import fp6_marlin
import kernel_rules as kr


def _fake_quantised(rng, shape):
    codes = rng.integers(0, 64, shape).astype(np.uint8)
    w = kr.fp6_value(codes).astype(np.float16)
    w.view(np.uint16)[(codes >> 5) == 1] |= 0x8000
    return w


def test_fp6_cast_all_patterns_match_oracle(oracle):
    """Every binary16 pattern, one per 4-group so an out-of-range one is isolated."""
    L = fp6_marlin.cabi.lib
    import ctypes
    src = np.zeros(4, dtype=np.uint16)
    dst = np.zeros(3, dtype=np.uint8)
    for p in range(65536):
        src[0] = p
        rc = L.fp6m_fp6_quantize(src.ctypes.data, dst.ctypes.data, 1, 4)
        try:
            want = oracle.fp6_cast4(src)
            assert rc == 0 and np.array_equal(dst, want), hex(p)
        except oracle.OracleError:
            assert rc == fp6_marlin.cabi.ERR_RANGE, hex(p)


@pytest.mark.parametrize("oc,ic", [(256, 256), (256, 512), (512, 256)])
def test_quantize_prepack_dequantize_match_oracle(oracle, oc, ic):
    rng = np.random.default_rng(oc + ic)
    w = _fake_quantised(rng, (oc, ic))
    q = fp6_marlin.quantize(torch.from_numpy(w))
    q_ref = oracle.fp6_quantize(w)
    assert q.dtype == torch.int32 and tuple(q.shape) == (ic, oc * 3 // 16)
    assert np.array_equal(q.numpy(), q_ref)
    p = fp6_marlin.prepacking(q)
    assert tuple(p.shape) == (oc * 3 // 32, ic * 2)      # here q is [ic rows, ...]: OC' = ic, IC' = oc
    assert np.array_equal(p.numpy(), oracle.fp6_prepack(q_ref))
    s = np.abs(rng.normal(0.02, 0.01, ic)).astype(np.float16) + np.float16(1e-3)
    d = fp6_marlin.dequantize(q, torch.from_numpy(s))
    assert np.array_equal(d.numpy().view(np.uint16), oracle.fp6_dequant(q_ref, s).view(np.uint16))


def test_prepack_random_bytes_match_oracle(oracle):
    """Arbitrary bit patterns, K != N, and the raw C routine at its 64-granularity."""
    rng = np.random.default_rng(7)
    L = fp6_marlin.cabi.lib
    for oc, ic in [(64, 64), (64, 192), (192, 64), (256, 768)]:
        raw = rng.integers(0, 256, oc * ic * 6 // 8, dtype=np.uint8)
        out = np.zeros_like(raw)
        assert L.fp6m_fp6_prepack(out.ctypes.data, raw.ctypes.data, oc, ic) == 0
        assert np.array_equal(out, oracle.fp6_prepack_bytes(raw, oc, ic))
    assert L.fp6m_fp6_prepack(out.ctypes.data, raw.ctypes.data, 32, 64) == fp6_marlin.cabi.ERR_SHAPE


def test_fp6_errors_are_exceptions():
    w = torch.zeros((256, 256), dtype=torch.float16)
    w[5, 7] = 30.0
    with pytest.raises(ValueError):
        fp6_marlin.quantize(w)
    w[5, 7] = 0.03
    with pytest.raises(ValueError):
        fp6_marlin.quantize(w)
    with pytest.raises(ValueError):
        fp6_marlin.quantize(torch.zeros((256, 256), dtype=torch.float32))
    with pytest.raises(ValueError):
        fp6_marlin.quantize(torch.zeros((128, 256), dtype=torch.float16))
    with pytest.raises(ValueError):
        fp6_marlin.prepacking(torch.zeros((128, 48), dtype=torch.int32))


@pytest.mark.parametrize("gs", [-1, 128])
def test_int4_quantize_and_pack_match_oracle(oracle, gs):
    rng = np.random.default_rng(9)
    w = rng.normal(0, 0.02, (512, 192)).astype(np.float16)
    w[:, 5] = 0                                             # an all-zero column must not produce NaN codes
    codes, scales, ref = fp6_marlin.int4_quantize(torch.from_numpy(w), gs)
    ok = np.ones(192, dtype=bool)
    ok[5] = False
    c_ref, s_ref, r_ref = oracle.int4_quantize(w[:, ok], gs)
    assert np.array_equal(codes.numpy()[:, ok], c_ref)
    assert np.array_equal(scales.numpy()[:, ok].view(np.uint16), s_ref.view(np.uint16))
    assert np.array_equal(ref.numpy()[:, ok].view(np.uint16), r_ref.view(np.uint16))
    assert (codes.numpy()[:, 5] == 8).all() and (ref.numpy()[:, 5] == 0).all()
    packed = fp6_marlin.int4_pack(codes)
    assert np.array_equal(packed.numpy(), oracle.int4_pack(codes.numpy()))


def test_permute_scales_matches_oracle(oracle):
    s = torch.arange(3 * 128, dtype=torch.float16).reshape(3, 128)
    assert np.array_equal(fp6_marlin.permute_scales(s).numpy(), oracle.permute_scales(s.numpy()))


@pytest.mark.parametrize("qc,gs", [(-1, -1), (256, -1), (512, -1), (256, 128), (-1, 128)])
def test_mixed_weight_wire_format_and_unpack(oracle, qc, gs):
    rng = np.random.default_rng(13)
    k, n = 256, 512
    w = rng.normal(0, 0.02, (k, n)).astype(np.float16)
    B, s, ref = fp6_marlin.pack_mixed_weight(torch.from_numpy(w), qc, gs)
    r_ref, b_ref, s_ref = oracle.gen_mixed_weight(w, qc, gs)
    assert np.array_equal(B.numpy(), b_ref)
    assert np.array_equal(s.numpy().view(np.uint16), s_ref.view(np.uint16))
    assert np.array_equal(ref.numpy().view(np.uint16), r_ref.view(np.uint16))
    back = fp6_marlin.unpack_to_fp16(B, s, k, n, qc, gs)
    # -0.0 vs +0.0: a zero INT4 weight times a scale is +0, compare as values
    assert np.array_equal(back.numpy().astype(np.float32), r_ref.astype(np.float32))


def test_layer_pack_is_a_real_transpose(oracle):
    """Layer.pack quantises W^T column for column (unlike the harness's flat reinterpretation)."""
    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 512, bias=False).half()
    layer = fp6_marlin.Layer(256, 512, groupsize=128, quant_cols=256)
    w_ref = layer.pack(lin)
    w = lin.weight.data.t().float()
    err = (w_ref.float() - w).abs().mean() / w.abs().mean()
    assert err < 0.12                                         # 4-bit / 6-bit quantisation noise, not a reshuffle
    err6 = (w_ref[:, 256:].float() - w[:, 256:]).abs().mean() / w[:, 256:].abs().mean()
    assert err6 < 0.12                                        # truncating e3m2: about half an ulp of 2 mantissa bits
    back = fp6_marlin.unpack_to_fp16(layer.B, layer.s, 256, 512, 256, 128)
    assert np.array_equal(back.numpy().astype(np.float32), w_ref.numpy().astype(np.float32))


def test_results_do_not_depend_on_thread_count(oracle, monkeypatch):
    rng = np.random.default_rng(17)
    w = _fake_quantised(rng, (256, 256))
    outs = []
    for nt in ("1", "5"):
        monkeypatch.setenv("FP6M_NUM_THREADS", nt)
        q = fp6_marlin.quantize(torch.from_numpy(w))
        outs.append((q.numpy().copy(), fp6_marlin.prepacking(q).numpy().copy()))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
