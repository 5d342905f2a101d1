"""
TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

Python face of the CPU oracle: ctypes bindings for ``fp6m_oracle.c`` plus a
numpy/torch-CPU restatement of the pieces of the reference that only exist in
its Python test harness.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the shipped
package never does.

What each function follows (paths relative to the reference checkout):

=====================  ======================================================
``fp6_quantize``       ``fp6_marlin/pybind.cpp:42-59`` over ``weight_quant.cpp:106-124``
``fp6_prepack``        ``fp6_marlin/pybind.cpp:18-31`` over ``weight_prepacking.cpp:123-177``
``fp6_dequant``        ``fp6_marlin/pybind.cpp:70-87`` over ``weight_prepacking.cpp:180-217``
``marlin_perms``       ``test.py:60-83``   (get_perms)
``int4_quantize``      ``test.py:85-101``  (scale, round, clamp, fake-quantised reference)
``int4_pack``          ``test.py:106-113`` (tile, permute, eight nibbles per word)
``permute_scales``     ``test.py:49-53, 102-105``
``gen_fp6_weight``     ``test.py:13-58``
``gen_int4_weight``    ``test.py:85-121``
``gen_mixed_weight``   ``test.py:123-152`` (the wire format of ``B`` and ``s``)
``matmul_ref``         ``test.py:165-167`` (dequantise-then-matmul), fp32 here
``gen_row_mix_weight`` no counterpart: ``gen_int4_weight`` on the first rows,
                       ``gen_fp6_weight`` on the last ones (same columns)
=====================  ======================================================

Pinning of the ctypes-bound functions is described at the top of
``fp6m_oracle.c``.  The INT4 packer and the scale permutation are pinned in
``tests/test_oracle_pins.py`` by decoding the packed words with the reference
kernel's own rules (``fp6_marlin_cuda_kernel.cu:249-286, 441-450, 548-600``
and the PTX ``mma.m16n8k16`` fragment maps).  ``int4_quantize`` with
``group_size=128`` has no counterpart in the reference (its kernel is
per-channel only, ``fp6_marlin_cuda_kernel.cu:447-448``): it is the same
formula applied per 128-row group, and is **parity unpinned** against the
reference by construction; it is checked against its closed form only.
``gen_row_mix_weight`` is likewise **parity unpinned** against the reference
(which mixes along columns only, ``fp6_marlin_cuda_kernel.cu:308-337``): it
concatenates the outputs of two pinned generators, and
``tests/test_oracle_pins.py`` checks that its packed words decode, with the
kernel's decode rules, to the check weight it returns.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfp6m_oracle.so")
_lib = None


def build(force=False):
    """Compile the C restatement with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        u16p, u8p = ctypes.POINTER(ctypes.c_uint16), ctypes.POINTER(ctypes.c_uint8)
        L.orc_half_to_float.restype = ctypes.c_float
        L.orc_half_to_float.argtypes = [ctypes.c_uint16]
        L.orc_float_to_half.restype = ctypes.c_uint16
        L.orc_float_to_half.argtypes = [ctypes.c_float]
        L.orc_fp6_cast4.argtypes = [u16p, u8p]
        L.orc_fp6_quantize.argtypes = [u16p, u8p, ctypes.c_size_t, ctypes.c_size_t]
        L.orc_fp6_prepack.argtypes = [u8p, u8p, ctypes.c_size_t, ctypes.c_size_t]
        L.orc_fp6_dequant.argtypes = [u16p, u8p, ctypes.c_size_t, ctypes.c_size_t, u16p]
        _lib = L
    return _lib


class OracleError(ValueError):
    pass


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _check(rc):
    if rc == 1:
        raise OracleError("Input value out of range for FP6.")
    if rc:
        raise OracleError("shape not supported")


# --------------------------------------------------------------------------- FP6 (C restatement)

def fp6_cast4(h4):
    """Four binary16 bit patterns -> three bytes (weight_quant.cpp:27-96)."""
    src = np.ascontiguousarray(h4, dtype=np.uint16)
    dst = np.zeros(3, dtype=np.uint8)
    _check(lib().orc_fp6_cast4(_p(src, ctypes.c_uint16), _p(dst, ctypes.c_uint8)))
    return dst


def fp6_quantize_flat(w_bits, rows, cols):
    """rows x cols binary16 bit patterns (flat) -> rows x cols*3/4 bytes."""
    src = np.ascontiguousarray(w_bits, dtype=np.uint16).reshape(-1)
    assert src.size == rows * cols
    dst = np.zeros((rows, cols * 6 // 8), dtype=np.uint8)
    _check(lib().orc_fp6_quantize(_p(src, ctypes.c_uint16), _p(dst, ctypes.c_uint8), rows, cols))
    return dst


def fp6_quantize(w, strict=True):
    """pybind.cpp:42-59.  `w`: float16 [OC, IC]; returns int32 [IC, OC*3/16].

    The reference labels its result "transposed" but hands the *untransposed*
    storage to the row quantiser (pybind.cpp:52-57): the flat buffer is read as
    IC rows of OC values.  Restated as is.
    """
    w = np.ascontiguousarray(w)
    assert w.dtype == np.float16 and w.ndim == 2
    oc, ic = w.shape
    if strict and (oc % 256 or ic % 256):  # pybind.cpp:50 (strict=False: only what the C routines need)
        raise OracleError("shape not supported")
    q = fp6_quantize_flat(w.view(np.uint16), ic, oc)
    return q.view(np.int32).reshape(ic, oc * 3 // 16)


def fp6_prepack_bytes(in6, rows, cols):
    src = np.ascontiguousarray(in6, dtype=np.uint8).reshape(-1)
    assert src.size == rows * cols * 6 // 8
    dst = np.zeros(rows * cols * 6 // 8, dtype=np.uint8)
    _check(lib().orc_fp6_prepack(_p(dst, ctypes.c_uint8), _p(src, ctypes.c_uint8), rows, cols))
    return dst


def fp6_prepack(q, strict=True):
    """pybind.cpp:18-31.  `q`: int32 [OC, IC*3/16] -> int32 [IC*3/32, OC*2]."""
    q = np.ascontiguousarray(q)
    assert q.dtype == np.int32 and q.ndim == 2
    oc = q.shape[0]
    if q.shape[1] % 3:
        raise OracleError("shape not supported")
    ic = q.shape[1] * 16 // 3
    if strict and (oc % 256 or ic % 256):  # pybind.cpp:24
        raise OracleError("shape not supported")
    out = fp6_prepack_bytes(q.view(np.uint8), oc, ic)
    return out.view(np.int32).reshape(ic * 3 // 32, oc * 2)


def fp6_dequant(q, scale):
    """pybind.cpp:70-87.  int32 [OC, IC*3/16] + float16 [OC] -> float16 [OC, IC]."""
    q = np.ascontiguousarray(q)
    scale = np.ascontiguousarray(scale, dtype=np.float16)
    oc = q.shape[0]
    ic = q.shape[1] // 3 * 16
    assert scale.shape == (oc,)
    out = np.zeros((oc, ic), dtype=np.uint16)
    _check(lib().orc_fp6_dequant(_p(out, ctypes.c_uint16), _p(q.view(np.uint8).reshape(-1), ctypes.c_uint8),
                                 oc, ic, _p(scale.view(np.uint16), ctypes.c_uint16)))
    return out.view(np.float16)


# --------------------------------------------------------------------------- harness-resident pieces

def marlin_perms():
    """test.py:60-83: the 1024-long weight permutation and the 32-long scale permutation."""
    perm = []
    for lane in range(32):                                   # :62
        col = lane // 4                                      # :64
        one = []
        for block in (0, 1):                                 # :65
            for row in (2 * (lane % 4), 2 * (lane % 4) + 1, 2 * (lane % 4 + 4), 2 * (lane % 4 + 4) + 1):
                one.append(16 * row + col + 8 * block)       # :72
        for j in range(4):                                   # :73-74
            perm.extend(p + 256 * j for p in one)
    perm = np.array(perm).reshape(-1, 8)[:, [0, 2, 4, 6, 1, 3, 5, 7]].ravel()  # :76-78
    scale_perm = [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]  # :80-82
    return perm, np.array(scale_perm)


def permute_scales(s):
    """test.py:49-53 / 102-105: per group of 32 columns, apply the scale permutation."""
    _, sp = marlin_perms()
    n = s.shape[-1]
    return s.reshape(-1, 32)[:, sp].reshape(s.shape[:-1] + (n,))


def int4_quantize(w, group_size=-1):
    """test.py:85-101 with torch CPU half arithmetic, per column (group_size=-1)
    or per (group_size rows, column).  Returns (codes uint8 (k,n) in 0..15,
    scales float16 (groups, n), w_ref float16 (k,n))."""
    w = torch.as_tensor(np.ascontiguousarray(w)).clone()
    assert w.dtype == torch.half
    k, n = w.shape
    g = k if group_size == -1 else group_size
    assert k % g == 0
    maxq = 2 ** 4 - 1
    wg = w.reshape(k // g, g, n)
    s = torch.max(torch.abs(wg), 1, keepdim=True)[0]         # :88
    s *= 2 / maxq                                            # :89
    q = torch.round(wg / s).int()                            # :90
    q += (maxq + 1) // 2                                     # :91
    q = torch.clamp(q, 0, maxq)                              # :92
    ref = (q - (maxq + 1) // 2).half() * s                   # :98
    q = torch.round(ref / s).int()                           # :99
    q += (maxq + 1) // 2                                     # :100
    q = torch.clamp(q, 0, maxq)                              # :101
    return (q.reshape(k, n).numpy().astype(np.uint8), s.reshape(k // g, n).numpy(),
            ref.reshape(k, n).numpy())


def int4_pack(codes):
    """test.py:106-113.  codes (k,n) in 0..15 -> int32 [k/16, n*2]."""
    perm, _ = marlin_perms()
    k, n = codes.shape
    w = codes.astype(np.uint32).reshape(k // 16, 16, n // 16, 16)   # :106
    w = w.transpose(0, 2, 1, 3).reshape(k // 16, n * 16)            # :107-108
    w = w.reshape(-1, perm.size)[:, perm].reshape(w.shape)          # :109
    q = np.zeros((w.shape[0], w.shape[1] // 8), dtype=np.uint32)    # :111
    for i in range(8):
        q |= w[:, i::8] << np.uint32(4 * i)                         # :112-113
    return q.view(np.int32)


def gen_int4_weight(w, group_size=-1):
    """test.py:85-121.  Returns (w_ref (k,n) f16, B int32 [k/16, n*2], s f16).

    `s` is (n,) in the reference's permuted order for group_size=-1; for
    group_size=128 it is (k/128, n) in natural column order (no reference)."""
    codes, s, ref = int4_quantize(w, group_size)
    s = permute_scales(s)[0] if group_size == -1 else s
    return ref, int4_pack(codes), np.ascontiguousarray(s)


def gen_fp6_weight(w, strict=True):
    """test.py:13-58.  w (k,n) f16 -> (w_ref (k,n) f16, B int32 [k*3/32, n*2], s (n,) f16 permuted)."""
    w = torch.as_tensor(np.ascontiguousarray(w)).clone()
    k, n = w.shape
    s = torch.max(torch.abs(w), 0, keepdim=True)[0]          # :19
    s *= 1.0 / 28.0                                          # :20
    s = s.reshape(-1, n).contiguous().squeeze(0)             # :21-22
    w = w / s                                                # :24
    w = torch.where(torch.abs(w) < 0.0625, torch.zeros_like(w), w)  # :26
    w = torch.clamp(w, -28.0, 28.0)                          # :27
    q = fp6_quantize(w.numpy(), strict)                      # :32  int32 [n, k*3/16]
    w_ref = fp6_dequant(q, s.numpy()).T                      # :37-38
    packed = fp6_prepack(q, strict)                          # :43
    return np.ascontiguousarray(w_ref), packed, permute_scales(s.numpy())


def gen_mixed_weight(w, quant_cols=-1, group_size=-1, strict=True):
    """test.py:123-152.  w (k,n) f16.  Returns (w_ref (k,n) f16, B int32 1-D, s f16 1-D).

    B = INT4 words of columns [0, n-qc)  ||  FP6 2-bit words  ||  FP6 4-bit words
    s = INT4 scales || FP6 scales        (test.py:139, 143-147).
    strict=False drops the multiple-of-256 asserts of the Python wrappers (pybind.cpp:24,50) and keeps
    the multiple-of-64 ones of the C routines, for FP6 regions of 128 columns."""
    k, n = w.shape
    if quant_cols == -1:
        ref, b, s = gen_int4_weight(w, group_size)
        return ref, b.reshape(-1), s.reshape(-1)
    if quant_cols == n:
        ref, b, s = gen_fp6_weight(w, strict)
        return ref, b.reshape(-1), s.reshape(-1)
    assert quant_cols % 64 == 0                               # :129
    w1, w2 = w[:, : n - quant_cols], w[:, n - quant_cols:]    # :130
    r1, b1, s1 = gen_int4_weight(np.ascontiguousarray(w1), group_size)
    r2, b2, s2 = gen_fp6_weight(np.ascontiguousarray(w2), strict)
    return (np.ascontiguousarray(np.concatenate([r1, r2], axis=1)),
            np.concatenate([b1.reshape(-1), b2.reshape(-1)]),
            np.concatenate([s1.reshape(-1), s2.reshape(-1)]))


def gen_row_mix_weight(w, quant_rows):
    """Operands of the row-mixed GEMM (no counterpart in the reference; a composition of its harness routines):
    rows [0, k - quant_rows) through gen_int4_weight with 128-row groups (test.py:85-121), the last quant_rows
    rows through gen_fp6_weight (test.py:13-58), both over all n columns.
    B = INT4 words || FP6 words, s = INT4 group scales || FP6 scales, w_ref = the two check weights stacked."""
    k, n = w.shape
    k4 = k - quant_rows
    assert 0 < k4 < k and k4 % 128 == 0 and quant_rows % 64 == 0 and n % 128 == 0
    r1, b1, s1 = gen_int4_weight(np.ascontiguousarray(w[:k4]), 128)
    r2, b2, s2 = gen_fp6_weight(np.ascontiguousarray(w[k4:]), False)
    return (np.ascontiguousarray(np.concatenate([r1, r2], axis=0)),
            np.concatenate([b1.reshape(-1), b2.reshape(-1)]),
            np.concatenate([s1.reshape(-1), s2.reshape(-1)]))


def matmul_ref(a, w_ref):
    """test.py:165-167 in fp32 (fp16 inputs are exact in fp32; fp64 accumulate)."""
    return (np.asarray(a, dtype=np.float64) @ np.asarray(w_ref, dtype=np.float64)).astype(np.float32)


def rel_err(c, c_ref):
    """test.py:181: mean|C - C_ref| / mean|C_ref|."""
    c = np.asarray(c, dtype=np.float64)
    c_ref = np.asarray(c_ref, dtype=np.float64)
    return float(np.mean(np.abs(c - c_ref)) / np.mean(np.abs(c_ref)))
