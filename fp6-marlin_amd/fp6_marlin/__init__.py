"""fp6_marlin for MI355X (gfx950): mixed INT4 / FP6-e3m2 weight-only, fp16-activation GEMM.

Same surface as liuchuan22/FP6-Marlin's ``fp6_marlin`` package (fp6_marlin/__init__.py:8-40):

    prepacking(fp6_tensor)            FP6 2+4-bit prepack on the CPU
    quantize(fp16_tensor)             FP16 -> FP6 e3m2 on the CPU
    dequantize(fp6_tensor, scales)    FP6 -> FP16 on the CPU
    mul(A, B, C, s, workspace, quant_cols=-1, thread_k=-1, thread_n=-1, sms=-1, max_par=16)

plus what the reference keeps in its test harness or lacks: ``Layer`` (pack / forward), the INT4
quantiser and packer, the scale permutation, the mixed-weight assembler, ``group_size=128`` scales and
``mul_fused`` (activation gather, output column scatter, bias and residual inside the GEMM call).
Everything is computed by ``libfp6m.so`` (C ABI in include/fp6m.h: host packers in C++, GEMM in
hand-written HIP for gfx950).  The four reference entry points go through ``_fp6m_torch``, a thin
PyTorch-ROCm C++ extension over that C ABI; ``fp6_marlin.cabi`` binds the same ABI with ctypes.
If either shared object is missing the import fails; there is no fallback.
"""
from . import cabi
try:
    from . import _fp6m_torch as _ext
except ImportError as e:  # pragma: no cover
    raise ImportError("fp6_marlin/_fp6m_torch.so is missing or does not load: build it with "
                      "`python fp6-marlin_amd/build.py`; there is no fallback implementation") from e
from .cabi import init, init_workspace, release_workspace, workspace_elems, pack_mixed_weight_device, mul_fused, mul_rows, check_column_map, repack_gfx950, repack_gfx950_host
from .layer import Layer, shared_workspace, pack_mixed_weight, pack_row_mix_weight, int4_quantize, int4_pack, permute_scales, unpack_to_fp16

__all__ = ["shared_workspace", "prepacking", "quantize", "dequantize", "mul", "Layer", "pack_mixed_weight", "pack_mixed_weight_device", "int4_quantize",
           "int4_pack", "permute_scales", "unpack_to_fp16", "init", "init_workspace", "release_workspace", "workspace_elems", "mul_fused", "mul_rows", "pack_row_mix_weight", "check_column_map", "repack_gfx950",
           "repack_gfx950_host"]


def prepacking(fp6_tensor):
    """Prepack the FP6 weight in 2+4 format (CPU).  int32 [OC, IC*3/16] -> int32 [IC*3/32, OC*2].
    Bit-exact with the reference (fp6_marlin/__init__.py:8-16, weight_prepacking.cpp:123-177)."""
    return _ext.prepacking_cpu(fp6_tensor)


def quantize(fp16_tensor):
    """Quantise a fake-quantised FP16 weight (|x| in {0} U [0.0625, 28]) to FP6 (CPU).
    float16 [OC, IC] -> int32 [IC, OC*3/16]  (fp6_marlin/__init__.py:18-26).

    Like the reference (pybind.cpp:52-57) this does NOT transpose: the contiguous buffer is read as IC
    rows of OC values.  ``Layer.pack`` transposes explicitly before calling it."""
    return _ext.quantization_cpu(fp16_tensor)


def dequantize(fp6_tensor, fp16_scales):
    """Dequantise FP6 to FP16 (CPU).  int32 [OC, IC*3/16], float16 [OC] -> float16 [OC, IC]
    (fp6_marlin/__init__.py:28-37)."""
    return _ext.dequantization_cpu(fp6_tensor, fp16_scales)


def mul(A, B, C, s, workspace, quant_cols=-1, thread_k=-1, thread_n=-1, sms=-1, max_par=16, group_size=-1):
    """Mixed INT4/FP6 x FP16 GEMM on the GPU (fp6_marlin/__init__.py:39-40).

    A          float16 [m, k]
    B          int32 1-D: INT4 words of columns [0, n-quant_cols) || FP6 2-bit plane || FP6 4-bit plane
    C          float16 [m, n], overwritten
    s          float16: INT4 scales || FP6 scales (per-column ones in the reference's permuted order)
    workspace  >= n // 128 * max_par zeroed 4-byte elements; left zeroed
    quant_cols -1: all INT4; n: all FP6; else the last quant_cols columns are FP6
    group_size -1: per-column INT4 scales; 128: INT4 scales [k/128, n-quant_cols] in natural column order
    """
    return _ext.mul(A, B, C, s, workspace, quant_cols, thread_k, thread_n, sms, max_par, group_size)
