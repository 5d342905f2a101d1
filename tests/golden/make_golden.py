"""Writes tests/golden/*.npz.  Run from the repository root:  python tests/golden/make_golden.py

The reference ships no golden vectors and neither its Python package nor its C++ can be run in this image,
so these vectors come from the CPU oracle (oracle/), *after* its pins in tests/test_oracle_pins.py pass.
They freeze the bit-exact contract (quantise / prepack / dequantise / INT4 pack) against regressions of
both the oracle and the shipped code.  Small on purpose (< 400 KiB together).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
from oracle import fp6m_oracle as oracle  # noqa: E402
import kernel_rules as kr  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def main():
    rng = np.random.default_rng(20240601)

    # 1. FP6 cast of every binary16 pattern: code (0..63) or 255 where the reference throws
    codes = np.full(65536, 255, dtype=np.uint8)
    for p in range(65536):
        try:
            codes[p] = oracle.fp6_cast4([p, 0, 0, 0])[0] >> 2
        except oracle.OracleError:
            pass
    np.savez_compressed(os.path.join(OUT, "fp6_cast_all_patterns.npz"), codes=codes)

    # 2. quantise -> prepack -> dequantise on a seeded fake-quantised 256 x 256 weight
    c = rng.integers(0, 64, (256, 256)).astype(np.uint8)
    w = kr.fp6_value(c).astype(np.float16)
    w.view(np.uint16)[(c >> 5) == 1] |= 0x8000
    q = oracle.fp6_quantize(w)
    scale = (np.abs(rng.normal(0.01, 0.005, 256)) + 1e-3).astype(np.float16)
    np.savez_compressed(os.path.join(OUT, "fp6_pipeline_256x256.npz"), w=w.view(np.uint16), q=q,
                        packed=oracle.fp6_prepack(q), scale=scale.view(np.uint16),
                        deq=oracle.fp6_dequant(q, scale).view(np.uint16))

    # 3. prepack of raw bytes, K != N, at the C routine's 64 granularity
    for oc, ic in ((64, 192), (128, 64)):
        raw = rng.integers(0, 256, oc * ic * 6 // 8, dtype=np.uint8)
        np.savez_compressed(os.path.join(OUT, f"fp6_prepack_bytes_{oc}x{ic}.npz"), raw=raw,
                            packed=oracle.fp6_prepack_bytes(raw, oc, ic))

    # 4. INT4 quantise + pack + scale permutation, per column and per group of 128
    w4 = rng.normal(0, 0.02, (256, 64)).astype(np.float16)
    for gs in (-1, 128):
        codes4, s4, ref4 = oracle.int4_quantize(w4, gs)
        np.savez_compressed(os.path.join(OUT, f"int4_256x64_g{gs}.npz"), w=w4.view(np.uint16), codes=codes4,
                            scales=s4.view(np.uint16), ref=ref4.view(np.uint16), packed=oracle.int4_pack(codes4),
                            scales_perm=oracle.permute_scales(s4).view(np.uint16))

    print("wrote", sorted(f for f in os.listdir(OUT) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
