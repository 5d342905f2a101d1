"""ctypes binding of the C ABI declared in include/fp6m.h (libfp6m.so, built by fp6-marlin_amd/build.py).

Nothing here computes anything: every function checks shapes/dtypes, hands raw pointers to the shared
library and maps its return code to the exception the reference raises for the same condition
(std::invalid_argument -> ValueError for the CPU helpers, AT_ERROR -> RuntimeError for `mul`).
There is no Python fallback: if the library is missing, importing this module fails.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfp6m.so")

OK, ERR_PROB_SHAPE, ERR_KERN_SHAPE, ERR_RANGE, ERR_SHAPE, ERR_ARG, ERR_HIP, ERR_NO_GPU_CODE, ERR_SCRATCH = range(9)

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `python fp6-marlin_amd/build.py` "
        "(hipcc --offload-arch=gfx950); there is no fallback implementation")

lib = ctypes.CDLL(LIB_PATH)

_vp, _sz, _int = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
lib.fp6m_strerror.restype = ctypes.c_char_p
lib.fp6m_strerror.argtypes = [_int]
lib.fp6m_last_hip_error.restype = _int
lib.fp6m_abi_version.restype = _int
lib.fp6m_workspace_elems.restype = _sz
lib.fp6m_pack_mixed_device.restype = _int
lib.fp6m_pack_mixed_device.argtypes = [_vp, _int, _int, _int, _int, _int, _vp, _vp, _vp, _int, _vp]
lib.fp6m_workspace_elems.argtypes = [_int, _int]
lib.fp6m_init.argtypes = [_int]
lib.fp6m_tuning_set.argtypes = [ctypes.c_char_p, _int]
lib.fp6m_tuning_set.restype = _int
lib.fp6m_init_workspace.argtypes = [_int, _vp, _int]
lib.fp6m_init_workspace.restype = _int
lib.fp6m_release_workspace.argtypes = [_int, _vp]
lib.fp6m_release_workspace.restype = _int
lib.fp6m_mul.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _vp, _int, _vp, _int, _int, _int, _int, _int, _int]
lib.fp6m_mul_static.argtypes = lib.fp6m_mul.argtypes
lib.fp6m_mul_static.restype = _int
lib.fp6m_mul_fused.argtypes = [_vp, _int, _vp, _vp, _vp, _int, _int, _int, _vp, _int, _vp, _int, _int, _int, _int, _vp, _vp,
                               _vp, _vp, _int]
lib.fp6m_repack_gfx950.argtypes = [_vp, _vp, _sz, _sz, _int, _int, _int]
lib.fp6m_mul_rows.argtypes = [_vp, _int, _vp, _vp, _vp, _int, _int, _int, _vp, _int, _vp, _int, _int, _int, _vp, _vp, _vp, _vp,
                              _int]
lib.fp6m_fp6_quantize.argtypes = [_vp, _vp, _sz, _sz]
lib.fp6m_fp6_prepack.argtypes = [_vp, _vp, _sz, _sz]
lib.fp6m_fp6_dequant.argtypes = [_vp, _vp, _sz, _sz, _vp]
lib.fp6m_int4_quantize.argtypes = [_vp, _sz, _sz, _int, _vp, _vp, _vp]
lib.fp6m_int4_pack.argtypes = [_vp, _vp, _sz, _sz]
lib.fp6m_permute_scales.argtypes = [_vp, _vp, _sz]
lib.fp6m_unpack_to_fp16.argtypes = [_vp, _vp, _vp, _sz, _sz, _int, _int]
for _f in (lib.fp6m_init, lib.fp6m_mul, lib.fp6m_mul_fused, lib.fp6m_mul_rows, lib.fp6m_repack_gfx950, lib.fp6m_fp6_quantize, lib.fp6m_fp6_prepack, lib.fp6m_fp6_dequant,
           lib.fp6m_int4_quantize, lib.fp6m_int4_pack, lib.fp6m_permute_scales, lib.fp6m_unpack_to_fp16):
    _f.restype = _int


class tuning:
    """Context manager around fp6m_tuning_set: `with tuning(ksplit=3, wk=8): ...` overrides the dispatcher's choices
    inside the block (tests and tuning runs only; process-wide, not thread-safe)."""

    def __init__(self, **knobs):
        self.knobs = {k: v for k, v in knobs.items() if v is not None}

    def __enter__(self):
        for name, value in self.knobs.items():
            if lib.fp6m_tuning_set(name.encode(), int(value)) != OK:
                lib.fp6m_tuning_set(None, 0)
                raise ValueError(f"unknown tuning knob {name!r}")
        return self

    def __exit__(self, *exc):
        lib.fp6m_tuning_set(None, 0)
        return False


def strerror(code):
    return lib.fp6m_strerror(code).decode()


def _raise_cpu(code):
    if code != OK:
        raise ValueError(strerror(code))


def _cpu(t, dtype, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} should be of type {dtype}.")
    if t.device.type != "cpu":
        raise ValueError(f"{name} must be a CPU tensor")
    return t.contiguous()


# ------------------------------------------------------------------------------------------ host routines

def fp6_quantize(w, strict=True):
    """float16 [OC, IC] -> int32 [IC, OC*3/16].  The flat row-major buffer is quantised as IC rows of OC
    values and *labelled* transposed, exactly as fp6_marlin/pybind.cpp:42-59 does."""
    w = _cpu(w, torch.float16, "Input tensor")
    mult = 256 if strict else 64        # the reference's wrapper asserts 256 (pybind.cpp:50), its C routine needs less
    if w.dim() != 2 or w.shape[0] % mult or w.shape[1] % mult:
        raise ValueError(f"quantize expects a 2-D tensor with both dimensions multiples of {mult}")
    oc, ic = w.shape
    out = torch.empty((ic, oc // 16 * 3), dtype=torch.int32)
    _raise_cpu(lib.fp6m_fp6_quantize(w.data_ptr(), out.data_ptr(), ic, oc))
    return out


def fp6_prepack(q, strict=True):
    """int32 [OC, IC*3/16] -> int32 [IC*3/32, OC*2] (2-bit plane then 4-bit plane), fp6_marlin/pybind.cpp:18-31."""
    q = _cpu(q, torch.int32, "fp6 tensor")
    if q.dim() != 2 or q.shape[1] % 3:
        raise ValueError("prepacking expects int32 [OC, IC*3/16]")
    oc, ic = q.shape[0], q.shape[1] * 16 // 3
    mult = 256 if strict else 64        # pybind.cpp:24 asserts 256, weight_prepacking.cpp:124-125 asserts 64
    if oc % mult or ic % mult:
        raise ValueError(f"prepacking expects OC and IC to be multiples of {mult}")
    out = torch.empty((ic // 32 * 3, oc * 2), dtype=torch.int32)
    _raise_cpu(lib.fp6m_fp6_prepack(out.data_ptr(), q.data_ptr(), oc, ic))
    return out


def fp6_dequant(q, scale):
    """int32 [OC, IC*3/16], float16 [OC] -> float16 [OC, IC], fp6_marlin/pybind.cpp:70-87."""
    q = _cpu(q, torch.int32, "fp6 tensor")
    scale = _cpu(scale, torch.float16, "scales")
    if q.dim() != 2 or q.shape[1] % 3 or scale.numel() != q.shape[0]:
        raise ValueError("dequantize expects int32 [OC, IC*3/16] and float16 [OC]")
    oc, ic = q.shape[0], q.shape[1] // 3 * 16
    out = torch.empty((oc, ic), dtype=torch.float16)
    _raise_cpu(lib.fp6m_fp6_dequant(out.data_ptr(), q.data_ptr(), oc, ic, scale.data_ptr()))
    return out


def int4_quantize(w, group_size=-1):
    """float16 [k, n] -> (codes uint8 [k, n], scales float16 [k/group, n], w_ref float16 [k, n]); test.py:85-101."""
    w = _cpu(w, torch.float16, "weight")
    k, n = w.shape
    g = k if group_size == -1 else group_size
    if g <= 0 or k % g:
        raise ValueError("group_size must be -1 or divide k")
    codes = torch.empty((k, n), dtype=torch.uint8)
    scales = torch.empty((k // g, n), dtype=torch.float16)
    ref = torch.empty((k, n), dtype=torch.float16)
    _raise_cpu(lib.fp6m_int4_quantize(w.data_ptr(), k, n, group_size, codes.data_ptr(), scales.data_ptr(), ref.data_ptr()))
    return codes, scales, ref


def int4_pack(codes):
    """uint8 [k, n] in 0..15 -> int32 [k/16, n*2]; test.py:106-113."""
    codes = _cpu(codes, torch.uint8, "codes")
    k, n = codes.shape
    out = torch.empty((k // 16, n * 2), dtype=torch.int32)
    _raise_cpu(lib.fp6m_int4_pack(codes.data_ptr(), out.data_ptr(), k, n))
    return out


def permute_scales(s):
    """float16 [..., n] -> same shape with the reference's 32-column scale permutation; test.py:80-83."""
    s = _cpu(s, torch.float16, "scales")
    out = torch.empty_like(s)
    rows = s.numel() // s.shape[-1] if s.numel() else 0
    for r in range(rows):
        off = r * s.shape[-1] * 2
        _raise_cpu(lib.fp6m_permute_scales(s.data_ptr() + off, out.data_ptr() + off, s.shape[-1]))
    return out


def unpack_to_fp16(B, s, k, n, quant_cols=-1, group_size=-1):
    """Packed B / s (CPU tensors) -> dequantised float16 [k, n]."""
    B = _cpu(B, torch.int32, "B")
    s = _cpu(s, torch.float16, "s")
    out = torch.empty((k, n), dtype=torch.float16)
    _raise_cpu(lib.fp6m_unpack_to_fp16(B.data_ptr(), s.data_ptr(), out.data_ptr(), k, n, quant_cols, group_size))
    return out


def pack_mixed_weight_device(w, quant_cols=-1, group_size=-1, harness_layout=True, want_ref=True):
    """Quantise and pack a CUDA float16 weight [k, n] on the GPU; same outputs, bit for bit, as the host path
    (`layer.pack_mixed_weight`).  Returns (B int32 1-D, s float16 1-D, w_ref float16 [k, n] or None), all on
    w's device."""
    if not isinstance(w, torch.Tensor) or not w.is_cuda or w.dtype != torch.float16 or w.dim() != 2:
        raise ValueError("w must be a 2-D CUDA float16 tensor")
    w = w.contiguous()
    k, n = w.shape
    qc = 0 if quant_cols in (-1, 0) else int(quant_cols)
    n4 = n - qc
    words = k * n4 // 8 + k * qc * 3 // 16
    nscale = (n4 if group_size == -1 else (k // group_size if group_size > 0 else 0) * n4) + qc
    B = torch.empty(words, dtype=torch.int32, device=w.device)
    s = torch.empty(nscale, dtype=torch.float16, device=w.device)
    ref = torch.empty((k, n), dtype=torch.float16, device=w.device) if want_ref else None
    with torch.cuda.device(w.device):
        code = lib.fp6m_pack_mixed_device(w.data_ptr(), k, n, qc, int(group_size), int(bool(harness_layout)), B.data_ptr(),
                                          s.data_ptr(), ref.data_ptr() if want_ref else None, w.device.index,
                                          torch.cuda.current_stream().cuda_stream)
    if code == ERR_HIP:
        raise RuntimeError(f"fp6m_pack_mixed_device: {strerror(code)} (hip error {lib.fp6m_last_hip_error()})")
    _raise_cpu(code)
    return B, s, ref


# ------------------------------------------------------------------------------------------ the GEMM

def workspace_elems(n, max_par=16):
    return int(lib.fp6m_workspace_elems(n, max_par))


def init(device=0):
    """Look up the device's properties now rather than in the first GEMM call.  Allocates nothing."""
    code = lib.fp6m_init(int(device))
    if code != OK:
        raise RuntimeError(f"fp6m_init: {strerror(code)} (hip error {lib.fp6m_last_hip_error()})")


def init_workspace(workspace, gather=False):
    """Allocate the partial-sum region that belongs to `workspace` (a CUDA tensor) now (and, with `gather`, the
    buffer that `a_cols` gathers pass through) instead of on its first call: do it before HIP-graph capture or any
    other section that must not allocate.  Returns the workspace."""
    code = lib.fp6m_init_workspace(workspace.device.index, workspace.data_ptr(), int(bool(gather)))
    if code != OK:
        raise RuntimeError(f"fp6m_init_workspace: {strerror(code)} (hip error {lib.fp6m_last_hip_error()})")
    return workspace


def release_workspace(workspace=None, device=0):
    """Wait for the device and free the region of `workspace` (call before the tensor is freed), or every region of
    `device` when no workspace is given."""
    if workspace is not None:
        code = lib.fp6m_release_workspace(workspace.device.index, workspace.data_ptr())
    else:
        code = lib.fp6m_release_workspace(int(device), None)
    if code != OK:
        raise RuntimeError(f"fp6m_release_workspace: {strerror(code)} (hip error {lib.fp6m_last_hip_error()})")


def mul(A, B, C, s, workspace, quant_cols=-1, thread_k=-1, thread_n=-1, sms=-1, max_par=16, group_size=-1):
    """C = A @ dequant(B) * s on the current HIP stream.  Argument order of fp6_marlin/__init__.py:39-40
    (reference: fp6_marlin/fp6_marlin_cuda.cpp:47-92), plus `group_size`."""
    for name, t in (("A", A), ("B", B), ("C", C), ("s", s), ("workspace", workspace)):
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise RuntimeError(f"{name} must be a tensor on the GPU")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.device != A.device:
            raise RuntimeError("all operands must live on the same device")
    if A.dtype != torch.float16 or C.dtype != torch.float16 or s.dtype != torch.float16:
        raise RuntimeError("A, C and s must be float16")
    if B.element_size() != 4 or workspace.element_size() != 4:
        raise RuntimeError("B must be int32 (or another 4-byte type) and workspace a 4-byte type")
    m, k = A.shape
    n = C.shape[1]
    if C.shape[0] != m:
        raise RuntimeError("C must be [m, n]")
    if workspace.numel() < n // 128 * max_par:                       # fp6_marlin_cuda.cpp:62-63
        raise RuntimeError(f"workspace must be of size at least {n // 128 * max_par}.")
    qc = 0 if quant_cols in (-1, 0) else quant_cols
    n4 = n - qc
    if k % 32 == 0 and 0 <= qc <= n:
        need_b = k * n4 // 8 + k * qc * 3 // 16
        need_s = (n4 if group_size == -1 else (k // 128) * n4) + qc
        if B.numel() < need_b or s.numel() != need_s:                # a (2, n) scale tensor fails here, test.py:219-226
            raise RuntimeError(f"B must hold {need_b} words and s {need_s} scales for this problem")
    dev = A.device.index
    stream = torch.cuda.current_stream(A.device).cuda_stream
    code = lib.fp6m_mul(A.data_ptr(), B.data_ptr(), C.data_ptr(), s.data_ptr(), m, n, k, workspace.data_ptr(),
                        dev, stream, thread_k, thread_n, sms, max_par, quant_cols, group_size)
    if code == ERR_PROB_SHAPE:
        raise RuntimeError(f"Problem (m={m}, n={n}, k={k}) not compatible with thread_k={thread_k}, thread_n={thread_n}.")
    if code == ERR_KERN_SHAPE:
        raise RuntimeError(f"No kernel implementation for thread_k={thread_k}, thread_n={thread_n}.")
    if code != OK:
        raise RuntimeError(f"fp6m_mul: {strerror(code)} (hip error {lib.fp6m_last_hip_error()})")


def check_column_map(cols, size, permutation=False):
    """Validate an int32 CUDA map for `mul_fused` on the host side (one device sync): entries inside
    [0, size), and a permutation if asked.  Do it once per map, not per call."""
    if not isinstance(cols, torch.Tensor) or not cols.is_cuda or cols.dtype != torch.int32 or cols.dim() != 1:
        raise ValueError("a column map must be a 1-D CUDA int32 tensor")
    if cols.numel() and (int(cols.min()) < 0 or int(cols.max()) >= size):
        raise ValueError(f"column map entries must lie in [0, {size})")
    if permutation and (cols.numel() != size or int(torch.unique(cols).numel()) != size):
        raise ValueError(f"column map must be a permutation of 0..{size - 1}")
    return cols


LAYOUT_GFX950 = 1


def _mul_extended(A, B, C, s, workspace, quant_cols, group_size, quant_rows, a_cols, c_cols, bias, residual, sms, max_par,
                  layout="reference"):
    if layout not in ("reference", "gfx950"):
        raise ValueError("layout must be 'reference' or 'gfx950'")
    flags = LAYOUT_GFX950 if layout == "gfx950" else 0
    tensors = [("A", A), ("B", B), ("C", C), ("s", s), ("workspace", workspace)]
    tensors += [(nm, t) for nm, t in (("a_cols", a_cols), ("c_cols", c_cols), ("bias", bias), ("residual", residual))
                if t is not None]
    for name, t in tensors:
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise RuntimeError(f"{name} must be a tensor on the GPU")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.device != A.device:
            raise RuntimeError("all operands must live on the same device")
    if A.dtype != torch.float16 or C.dtype != torch.float16 or s.dtype != torch.float16:
        raise RuntimeError("A, C and s must be float16")
    if B.element_size() != 4 or workspace.element_size() != 4:
        raise RuntimeError("B must be int32 (or another 4-byte type) and workspace a 4-byte type")
    if A.dim() != 2 or C.dim() != 2 or C.shape[0] != A.shape[0]:
        raise RuntimeError("A must be [m, lda] and C [m, n]")
    m, lda = A.shape
    n = C.shape[1]
    k = lda if a_cols is None else a_cols.numel()
    for name, t, numel in (("a_cols", a_cols, k), ("c_cols", c_cols, n)):
        if t is not None and (t.dtype != torch.int32 or t.numel() != numel):
            raise RuntimeError(f"{name} must be int32 with {numel} entries")
    if bias is not None and (bias.dtype != torch.float16 or bias.numel() != n):
        raise RuntimeError(f"bias must be float16 with {n} entries")
    if residual is not None and (residual.dtype != torch.float16 or tuple(residual.shape) != (m, n)):
        raise RuntimeError("residual must be float16 [m, n]")
    if workspace.numel() < n // 128 * max_par:
        raise RuntimeError(f"workspace must be of size at least {n // 128 * max_par}.")
    if quant_rows:
        k4 = k - quant_rows
        if quant_rows < 0 or k4 <= 0:
            raise RuntimeError("quant_rows must be positive and below k")
        if k4 % 128 == 0 and quant_rows % 64 == 0:
            need_b, need_s = k4 * n // 8 + quant_rows * n * 3 // 16, (k4 // 128) * n + n
            if B.numel() < need_b or s.numel() != need_s:
                raise RuntimeError(f"B must hold {need_b} words and s {need_s} scales for this problem")
    else:
        qc = 0 if quant_cols in (-1, 0) else quant_cols
        n4 = n - qc
        if k % 32 == 0 and 0 <= qc <= n:
            need_b = k * n4 // 8 + k * qc * 3 // 16
            need_s = (n4 if group_size == -1 else (k // 128) * n4) + qc
            if B.numel() < need_b or s.numel() != need_s:
                raise RuntimeError(f"B must hold {need_b} words and s {need_s} scales for this problem")
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(A.device):
        stream = torch.cuda.current_stream().cuda_stream
        if quant_rows:
            name = "fp6m_mul_rows"
            code = lib.fp6m_mul_rows(A.data_ptr(), lda, B.data_ptr(), C.data_ptr(), s.data_ptr(), m, n, k,
                                     workspace.data_ptr(), A.device.index, stream, sms, max_par, quant_rows,
                                     ptr(a_cols), ptr(c_cols), ptr(bias), ptr(residual), flags)
        else:
            name = "fp6m_mul_fused"
            code = lib.fp6m_mul_fused(A.data_ptr(), lda, B.data_ptr(), C.data_ptr(), s.data_ptr(), m, n, k,
                                      workspace.data_ptr(), A.device.index, stream, sms, max_par, quant_cols, group_size,
                                      ptr(a_cols), ptr(c_cols), ptr(bias), ptr(residual), flags)
    if code == ERR_PROB_SHAPE:
        raise RuntimeError(f"Problem (m={m}, n={n}, k={k}) not compatible with the tile shape.")
    if code != OK:
        raise RuntimeError(f"{name}: {strerror(code)} (hip error {lib.fp6m_last_hip_error()})")


def mul_fused(A, B, C, s, workspace, quant_cols=-1, group_size=-1, a_cols=None, c_cols=None, bias=None, residual=None,
              sms=-1, max_par=16, layout="reference"):
    """`mul` with the reorders and additions around it folded into the launch (no counterpart in the reference,
    whose harness leaves them to the caller: the FP6 columns of its packed weight sit at the tail, test.py:123-152):

        C[:, c_cols] = fp16(A[:, a_cols] @ dequant(B) * s + bias[c_cols] + residual[:, c_cols])

    a_cols int32 [k] (columns of A, which may then be wider than k), c_cols int32 [n] permutation, bias float16 [n],
    residual float16 [m, n] (may be C).  Maps are trusted here: run `check_column_map` on them once.
    layout="gfx950": B went through `repack_gfx950`."""
    _mul_extended(A, B, C, s, workspace, quant_cols, group_size, 0, a_cols, c_cols, bias, residual, sms, max_par, layout)


def mul_rows(A, B, C, s, workspace, quant_rows, a_cols=None, c_cols=None, bias=None, residual=None, sms=-1, max_par=16,
             layout="reference"):
    """The GEMM for a weight mixed along k instead of n: the last `quant_rows` rows (input channels) of every
    column are FP6 with one scale per column, the rows before them INT4 with one scale per 128 rows and column.
    Both segments of a column tile accumulate into the same output tile inside one launch.  (The reference mixes
    along n only, fp6_marlin_cuda_kernel.cu:308-337; the same result there takes two `mul` calls and an addition.)

        B = INT4 words of rows [0, k - quant_rows) || FP6 2-bit plane of the last rows || their 4-bit plane
        s = INT4 group scales [(k - quant_rows) / 128, n] || FP6 column scales [n] (permuted order)

    (k - quant_rows) % 128 == 0, quant_rows % 64 == 0, n % 128 == 0.  The optional arguments are those of
    `mul_fused`; `a_cols` is how arbitrary input channels get to the FP6 tail."""
    if int(quant_rows) <= 0:
        raise RuntimeError("quant_rows must be positive and below k")
    _mul_extended(A, B, C, s, workspace, -1, 128, int(quant_rows), a_cols, c_cols, bias, residual, sms, max_par, layout)


def _plane_views(B, k, n, quant_cols, quant_rows):
    """(offset, rows, cols, words per lane) of the planes inside a B buffer."""
    if quant_rows:
        rows4, cols4, rows6, cols6 = k - quant_rows, n, quant_rows, n
    else:
        qc = 0 if quant_cols in (-1, 0) else quant_cols
        rows4, cols4, rows6, cols6 = k, n - qc, k, qc
    if rows4 <= 0 or rows4 % 16 or rows6 % 16 or cols4 % 128 or cols6 % 128 or cols4 < 0:
        raise ValueError("regions must have whole 128-column tiles and 16-row k-blocks")
    words4, words2 = rows4 * cols4 // 8, rows6 * cols6 // 16
    if B.numel() != words4 + 3 * words2:
        raise ValueError(f"B must hold {words4 + 3 * words2} words")
    planes = [(0, rows4, cols4, 4)] if cols4 else []
    if cols6:
        planes += [(words4, rows6, cols6, 2), (words4 + words2, rows6, cols6, 4)]
    return planes


def repack_gfx950(B, k, n, quant_cols=-1, quant_rows=0, to_gfx950=True):
    """Reorder the packed words of `B` (int32 1-D, on any device) between the reference's order and the gfx950
    one, in which every 128-column tile is one sequential stream in MFMA lane order (see fp6m_repack_gfx950 in
    include/fp6m.h, which this mirrors with tensor permutes so that it runs where the tensor lives).  Lossless;
    `to_gfx950=False` is the inverse.  Scales do not change."""
    if B.dtype != torch.int32 or B.dim() != 1:
        raise ValueError("B must be a 1-D int32 tensor")
    out = torch.empty_like(B)
    for off, rows, cols, words in _plane_views(B, k, n, quant_cols, quant_rows):
        size = rows * cols // 32 * words
        kb, tiles = rows // 16, cols // 128
        src = B[off:off + size]
        if to_gfx950:        # [kb][tile][sigma][l][i][w] -> [tile][kb][i][sigma][l][w]
            out[off:off + size] = src.view(kb, tiles, 2, 8, 4, words).permute(1, 0, 4, 2, 3, 5).reshape(-1)
        else:
            out[off:off + size] = src.view(tiles, kb, 4, 2, 8, words).permute(1, 0, 3, 4, 2, 5).reshape(-1)
    return out


def repack_gfx950_host(B, k, n, quant_cols=-1, quant_rows=0, to_gfx950=True):
    """The same conversion through the C ABI's host routine (CPU tensors)."""
    if B.dtype != torch.int32 or B.dim() != 1 or B.is_cuda:
        raise ValueError("B must be a 1-D int32 CPU tensor")
    B = B.contiguous()
    out = torch.empty_like(B)
    _plane_views(B, k, n, quant_cols, quant_rows)
    qc = 0 if quant_cols in (-1, 0) else quant_cols
    _raise_cpu(lib.fp6m_repack_gfx950(B.data_ptr(), out.data_ptr(), k, n, qc, quant_rows, int(bool(to_gfx950))))
    return out
