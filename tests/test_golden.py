"""Committed fixtures (tests/golden/, written by make_golden.py from the pinned oracle) against the oracle
and against the shipped host routines: bit-exact."""
import os

import numpy as np
import torch

import fp6_marlin

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(G, name), allow_pickle=False)


def test_fp6_cast_fixture(oracle):
    want = load("fp6_cast_all_patterns.npz")["codes"]
    L = fp6_marlin.cabi.lib
    src = np.zeros(4, dtype=np.uint16)
    dst = np.zeros(3, dtype=np.uint8)
    got = np.full(65536, 255, dtype=np.uint8)
    for p in range(65536):
        src[0] = p
        if L.fp6m_fp6_quantize(src.ctypes.data, dst.ctypes.data, 1, 4) == 0:
            got[p] = dst[0] >> 2
    assert np.array_equal(got, want)
    assert (want != 255).sum() == 2 * (1 + (np.float16(28).view(np.uint16) - np.float16(0.0625).view(np.uint16) + 1))
    for p in (0x0000, 0x8000, 0x2C00, 0x4F00, 0xCF00, 0x3C00, 0x3555):   # spot checks through the oracle too
        assert oracle.fp6_cast4([p, 0, 0, 0])[0] >> 2 == want[p]


def test_fp6_pipeline_fixture(oracle):
    f = load("fp6_pipeline_256x256.npz")
    w = torch.from_numpy(f["w"].view(np.float16).copy())
    q = fp6_marlin.quantize(w)
    assert np.array_equal(q.numpy(), f["q"]) and np.array_equal(oracle.fp6_quantize(w.numpy()), f["q"])
    assert np.array_equal(fp6_marlin.prepacking(q).numpy(), f["packed"])
    assert np.array_equal(oracle.fp6_prepack(f["q"]), f["packed"])
    s = torch.from_numpy(f["scale"].view(np.float16).copy())
    assert np.array_equal(fp6_marlin.dequantize(q, s).numpy().view(np.uint16), f["deq"])
    assert np.array_equal(oracle.fp6_dequant(f["q"], s.numpy()).view(np.uint16), f["deq"])


def test_prepack_bytes_fixtures(oracle):
    L = fp6_marlin.cabi.lib
    for oc, ic in ((64, 192), (128, 64)):
        f = load(f"fp6_prepack_bytes_{oc}x{ic}.npz")
        raw = np.ascontiguousarray(f["raw"])
        out = np.zeros_like(raw)
        assert L.fp6m_fp6_prepack(out.ctypes.data, raw.ctypes.data, oc, ic) == 0
        assert np.array_equal(out, f["packed"])
        assert np.array_equal(oracle.fp6_prepack_bytes(raw, oc, ic), f["packed"])


def test_int4_fixtures(oracle):
    for gs in (-1, 128):
        f = load(f"int4_256x64_g{gs}.npz")
        w = torch.from_numpy(f["w"].view(np.float16).copy())
        codes, scales, ref = fp6_marlin.int4_quantize(w, gs)
        assert np.array_equal(codes.numpy(), f["codes"])
        assert np.array_equal(scales.numpy().view(np.uint16), f["scales"])
        assert np.array_equal(ref.numpy().view(np.uint16), f["ref"])
        assert np.array_equal(fp6_marlin.int4_pack(codes).numpy(), f["packed"])
        assert np.array_equal(fp6_marlin.permute_scales(scales).numpy().view(np.uint16), f["scales_perm"])
        assert np.array_equal(oracle.int4_pack(f["codes"]), f["packed"])
