"""
How the *reference GPU kernel* reads and decodes a packed weight buffer,
restated in numpy.  It is the independent witness used to pin the packers:
packing is right exactly when these rules recover every (k, n) weight.

Sources (paths relative to the reference checkout, fp6_marlin/fp6_marlin_cuda_kernel.cu):

* word addressing: a 16-row k-block is one row of `16*n/32` 16-byte vectors
  (:421); inside a 64-column group, lane t of the warp owns vector `32*g + t`
  (:441-445, :555), and its four 32-bit words are tiles j = 0..3 (:575-585).
  The 2-bit plane uses 8-byte vectors with the same indexing (:484, :559), one
  word per two tiles, shifted left by 4 for the odd tile (:579-583).
* INT4 bit rules: dequant_8int4 (:249-286).
* FP6 bit rules: dequant_8fp6 (:195-237) and mult_bias (:137-147).
* which (k, n) a register holds: registers 0,1 feed the mma for columns
  16j + l, registers 2,3 the mma for columns 16j + 8 + l (:588-597); inside an
  `mma.m16n8k16` B fragment (PTX ISA, "Matrix Fragments for mma.m16n8k16"),
  lane t = 4l + i holds rows k = 2i, 2i+1 in register 0 and k = 2i+8, 2i+9 in
  register 1, column l.
* scale order: s_sh_rd (:450), the two 16-byte scale loads (:798-799) and the
  epilogue's use of s_frag[j / 2][2 * (j % 2) + half] (:731-734) on the
  m16n8 C fragment (columns 2i, 2i+1 of the 8).
"""
import numpy as np


def fragment_coords():
    """(k_local, n_local) of element x = 0..7 held by lane t for tile j: arrays [32, 4, 8]."""
    t = np.arange(32)[:, None, None]
    j = np.arange(4)[None, :, None]
    x = np.arange(8)[None, None, :]
    l, i = t // 4, t % 4
    k = 2 * i + (x % 2) + 8 * ((x % 4) // 2)
    n = 16 * j + l + 8 * (x // 4)
    return np.broadcast_to(k, (32, 4, 8)).copy(), np.broadcast_to(n, (32, 4, 8)).copy()


def _halves(u32):
    """uint32 array -> float16 array with a trailing axis of 2: (low half, high half)."""
    u32 = np.ascontiguousarray(u32, dtype=np.uint32)
    return u32.view(np.uint16).reshape(u32.shape + (2,)).view(np.float16)


def dequant_8int4(q):
    """:249-286.  uint32 [...] -> float16 [..., 8] in register order (reg0.lo, reg0.hi, reg1.lo, ...)."""
    q = np.asarray(q, dtype=np.uint32)
    LO, HI, EX = np.uint32(0x000F000F), np.uint32(0x00F000F0), np.uint32(0x64006400)
    out = []
    for sh in (0, 8):
        v = q >> np.uint32(sh)
        lo = _halves((v & LO) | EX) - np.float16(1032.0)                                # hsub2
        hi = (_halves((v & HI) | EX).astype(np.float32) * np.float32(0.0625) + np.float32(-72.0)).astype(np.float16)  # hfma2
        out += [lo, hi]
    return np.concatenate(out, axis=-1)


def dequant_8fp6(q2, q4):
    """:195-237.  uint32 q2 (already shifted for the tile), q4 -> float16 [..., 8] in register order."""
    q2 = np.asarray(q2, dtype=np.uint32)
    q4 = np.asarray(q4, dtype=np.uint32)
    out = []
    for _ in range(2):
        p = (q2 & np.uint32(0xC0C0C0C0)) | ((q4 & np.uint32(0xF0F0F0F0)) >> np.uint32(2))
        for _ in range(2):
            o = (p & np.uint32(0x80008000)) | ((p & np.uint32(0x7C007C00)) >> np.uint32(2))
            out.append((_halves(o).astype(np.float32) * np.float32(4096.0)).astype(np.float16))  # mult_bias
            p = p << np.uint32(8)
        q2 = q2 << np.uint32(2)
        q4 = q4 << np.uint32(4)
    return np.concatenate(out, axis=-1)


def _scatter(vals, kdim, ndim):
    """vals [K/16, n/64, 32, 4, 8] -> [K, n] using the fragment map."""
    kl, nl = fragment_coords()
    out = np.zeros((kdim, ndim), dtype=vals.dtype)
    shape = (kdim // 16, ndim // 64, 32, 4, 8)
    kb = np.arange(kdim // 16)[:, None, None, None, None]
    g = np.arange(ndim // 64)[None, :, None, None, None]
    kk = np.broadcast_to(16 * kb + kl[None, None], shape).reshape(-1)
    nn = np.broadcast_to(64 * g + nl[None, None], shape).reshape(-1)
    out[kk, nn] = vals.reshape(-1)
    hits = np.zeros((kdim, ndim), dtype=np.int32)
    np.add.at(hits, (kk, nn), 1)
    assert (hits == 1).all(), "fragment map is not a bijection"
    return out


def decode_int4(words, kdim, ndim):
    """Packed INT4 words (int32 [K/16, n*2] or flat) -> float16 [K, n] of (nibble - 8)."""
    w = np.ascontiguousarray(words).view(np.uint32).reshape(kdim // 16, ndim // 64, 32, 4)
    return _scatter(dequant_8int4(w), kdim, ndim)


def decode_fp6(words, kdim, ndim):
    """Packed FP6 words (int32 [K*3/32, n*2] or flat: 2-bit plane then 4-bit plane) -> float16 [K, n]."""
    flat = np.ascontiguousarray(words).view(np.uint32).reshape(-1)
    n2 = kdim * ndim * 2 // 32
    w2 = flat[:n2].reshape(kdim // 16, ndim // 64, 32, 2)
    w4 = flat[n2:].reshape(kdim // 16, ndim // 64, 32, 4)
    j = np.arange(4)
    q2 = w2[..., j // 2] << (np.uint32(4) * (j % 2).astype(np.uint32))
    return _scatter(dequant_8fp6(q2, w4), kdim, ndim)


def scale_slot(col):
    """Stored position, inside its group of 32, of the scale the epilogue applies to column `col` (0..31)."""
    i, d = (col % 8) // 2, col % 2
    half, jj = (col // 8) % 2, col // 16
    return 8 * i + 4 * jj + 2 * half + d


FP6_GRID = np.array([0, .0625, .125, .1875, .25, .3125, .375, .4375, .5, .625, .75, .875, 1, 1.25, 1.5, 1.75,
                     2, 2.5, 3, 3.5, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28], dtype=np.float64)


def fp6_value(code):
    """e3m2 (bias 3, no inf/NaN) from its closed form: code = s eee mm."""
    code = np.asarray(code, dtype=np.int64)
    s, e, m = code >> 5, (code >> 2) & 7, code & 3
    mag = np.where(e == 0, m / 4.0 * 2.0 ** -2, (1 + m / 4.0) * 2.0 ** (e - 3.0))
    return np.where(s == 1, -mag, mag)


def unpack_fp6_rows(q_bytes, rows, cols):
    """Row-packed 6-bit codes (MSB first, weight_quant.cpp:93-95) -> uint8 [rows, cols]."""
    b = np.ascontiguousarray(q_bytes, dtype=np.uint8).reshape(rows, cols * 6 // 8)
    bits = np.unpackbits(b, axis=1).reshape(rows, cols, 6)
    return (bits * (1 << np.arange(5, -1, -1))).sum(axis=2).astype(np.uint8)


def pack_fp6_rows(codes):
    """uint8 [rows, cols] codes -> row-packed bytes [rows, cols*6/8] (bit-string construction)."""
    codes = np.asarray(codes, dtype=np.uint8)
    bits = ((codes[..., None] >> np.arange(5, -1, -1)) & 1).astype(np.uint8)
    return np.packbits(bits.reshape(codes.shape[0], -1), axis=1)
