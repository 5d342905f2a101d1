"""Weight preparation and the ``Layer`` module.

The reference keeps INT4 packing, the scale permutation and the mixed-weight concatenation in its test
harness (test.py:13-152) and has no ``Layer``; here they are library functions backed by the C ABI.
"""
import torch
import torch.nn as nn

from . import cabi

int4_quantize = cabi.int4_quantize
int4_pack = cabi.int4_pack
permute_scales = cabi.permute_scales
unpack_to_fp16 = cabi.unpack_to_fp16

FP6_MAX = 28.0
FP6_MIN = 0.0625


def _fp6_region(w):
    """test.py:13-58 on a [k, nq] float16 slice whose storage is [k, nq] row-major.
    Returns (B int32 [k*3/32, nq*2], s float16 [nq] permuted, w_ref float16 [k, nq])."""
    k, nq = w.shape
    s = torch.max(torch.abs(w), 0, keepdim=True)[0]
    s *= 1.0 / FP6_MAX
    s = s.reshape(-1, nq).contiguous().squeeze(0)
    w = w / s
    w = torch.where(torch.abs(w) < FP6_MIN, torch.zeros_like(w), w)
    w = torch.clamp(w, -FP6_MAX, FP6_MAX)
    q = cabi.fp6_quantize(w, strict=False)         # int32 [nq, k*3/16]: rows of the *flat* buffer
    w_ref = cabi.fp6_dequant(q, s).transpose(0, 1).contiguous()
    return cabi.fp6_prepack(q, strict=False), cabi.permute_scales(s), w_ref


def pack_mixed_weight(w, quant_cols=-1, group_size=-1, harness_layout=True):
    """Quantise and pack a float16 weight ``w`` [k, n] into the operands of ``mul``.

    The last ``quant_cols`` columns go to FP6 with one scale per column, the others to symmetric INT4
    with one scale per column (``group_size=-1``) or per 128 rows and column (``group_size=128``).
    Returns ``(B, s, w_ref)``: int32 1-D, float16 1-D, and the dequantised float16 [k, n] weight that
    ``mul`` multiplies by (the reference's check weight, test.py:37-38, 98).

    ``harness_layout=True`` reproduces the reference harness bit for bit, including the fact that its
    FP6 path quantises the [k, nq] buffer as if it were [nq, k] (no transpose, pybind.cpp:52-57), so the
    FP6 part of ``w_ref`` is a reshuffle of ``w``.  ``harness_layout=False`` transposes first, so that
    ``w_ref`` approximates ``w`` column for column: use that for real models (``Layer.pack`` does).

    A CUDA ``w`` is quantised and packed on the GPU (same bits; outputs stay on its device); a CPU ``w`` goes
    through the host routines.
    """
    if w.dtype != torch.float16 or w.dim() != 2:
        raise ValueError("w must be a 2-D float16 tensor")
    if w.is_cuda:
        qc_dev = 0 if quant_cols in (-1, 0) else quant_cols
        if qc_dev < 0 or qc_dev > w.shape[1] or qc_dev % 64:
            raise ValueError("quant_cols must be -1 or a multiple of 64 not above n")
        return cabi.pack_mixed_weight_device(w.detach(), quant_cols, group_size, harness_layout)
    w = w.detach().cpu().contiguous()
    k, n = w.shape
    qc = 0 if quant_cols in (-1, 0) else quant_cols
    if qc < 0 or qc > n or qc % 64:
        raise ValueError("quant_cols must be -1 or a multiple of 64 not above n")
    parts_b, parts_s, parts_ref = [], [], []
    if n - qc:
        w4 = w[:, : n - qc].contiguous()
        codes, scales, ref = cabi.int4_quantize(w4, group_size)
        parts_b.append(cabi.int4_pack(codes).reshape(-1))
        parts_s.append((cabi.permute_scales(scales) if group_size == -1 else scales).reshape(-1))
        parts_ref.append(ref)
    if qc:
        w6 = w[:, n - qc:].contiguous()
        if harness_layout:
            b6, s6, ref6 = _fp6_region(w6)
        else:
            # quantise the true transpose: feed quantize() a buffer whose flat view is [nq, k]
            s6 = torch.max(torch.abs(w6), 0)[0] * (1.0 / FP6_MAX)
            s6 = torch.where(s6 == 0, torch.ones_like(s6), s6)
            t = (w6 / s6).transpose(0, 1).contiguous()            # [nq, k]
            t = torch.where(torch.abs(t) < FP6_MIN, torch.zeros_like(t), t).clamp(-FP6_MAX, FP6_MAX)
            q = cabi.fp6_quantize(t.reshape(k, qc), strict=False)  # flat view read as [nq, k]
            ref6 = cabi.fp6_dequant(q, s6).transpose(0, 1).contiguous()
            b6, s6 = cabi.fp6_prepack(q, strict=False), cabi.permute_scales(s6)
        parts_b.append(b6.reshape(-1))
        parts_s.append(s6.reshape(-1))
        parts_ref.append(ref6)
    return (torch.cat(parts_b).contiguous(), torch.cat(parts_s).contiguous(),
            torch.cat(parts_ref, dim=1).contiguous())


def pack_row_mix_weight(w, quant_rows):
    """Quantise and pack a float16 weight ``w`` [k, n] for ``mul_rows``: the last ``quant_rows`` rows (input
    channels) go to FP6 with one scale per column, the rows before them to INT4 with one scale per 128 rows and
    column.  Returns ``(B, s, w_ref)`` like ``pack_mixed_weight``; both segments use its routines (on the GPU for
    a CUDA ``w``), the FP6 one in the layout that quantises each column by its own scale."""
    if w.dtype != torch.float16 or w.dim() != 2:
        raise ValueError("w must be a 2-D float16 tensor")
    k, n = w.shape
    k4 = k - quant_rows
    if quant_rows <= 0 or k4 <= 0 or k4 % 128 or quant_rows % 64 or n % 128:
        raise ValueError("need 0 < quant_rows < k, (k - quant_rows) % 128 == 0, quant_rows % 64 == 0 and n % 128 == 0")
    b4, s4, r4 = pack_mixed_weight(w[:k4].contiguous(), -1, 128)
    b6, s6, r6 = pack_mixed_weight(w[k4:].contiguous(), n, -1, harness_layout=False)
    return torch.cat([b4, b6]).contiguous(), torch.cat([s4, s6]).contiguous(), torch.cat([r4, r6], dim=0).contiguous()


_workspaces = {}


def shared_workspace(device, elems=0):
    """The zeroed int32 workspace that ``Layer.forward`` uses on `device` when the caller passes none: one per device,
    made on first use (65536 elements, enough for 524288 output features; it grows, as a new tensor, only beyond that).
    The library allows one call at a time per workspace, so this default suits models whose layers run one after
    the other on one stream -- also under HIP-graph capture, which changes the current stream but not the device.
    Callers that run layers concurrently on several streams pass ``forward`` a workspace of their own per stream."""
    device = torch.device(device)
    key = device.index if device.index is not None else torch.cuda.current_device()
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < elems:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("fp6_marlin: the default workspace of this device does not exist yet (or is too small "
                               "for this layer) and cannot be made while a HIP graph is being captured; run the layer "
                               "once before the capture, or pass forward() a workspace")
        ws = torch.zeros(max(int(elems), 65536), dtype=torch.int32, device=device)
        _workspaces[key] = ws                                      # (a smaller one stays alive with whoever captured it)
    return ws


class Layer(nn.Module):
    """Linear layer ``y = x @ W (+ bias)`` with W [infeatures, outfeatures] stored as mixed INT4 / FP6.

    Buffers (all on the module's device; ``B``, ``s``, ``meta`` and, if used, ``c_cols`` / ``bias`` are saved):
      ``B``          int32 1-D, the wire format of ``mul``
      ``s``          float16 1-D: INT4 scales (per column in the reference's permuted order, or
                     [infeatures/128, outfeatures-quant_cols] in natural column order when
                     ``groupsize=128``) followed by the FP6 per-column scales (permuted order)
      ``meta``       int32 [7]: format version, infeatures, outfeatures, quant_cols, groupsize, word order
                     (0 reference, 1 gfx950), quant_rows; a checkpoint whose ``meta`` differs is refused
    The GEMM's ``workspace`` (zeroed int32, outfeatures // 128 * 16 elements at least) is not a buffer of the layer:
    ``forward`` takes the one passed to it or else ``shared_workspace``'s tensor of the device, because the library
    keeps a partial-sum region per workspace address and calls that cannot overlap should share one.

    Which output features are kept in FP6: by default the *last* ``quant_cols`` ones (what the reference's
    harness does after moving its chosen columns to the tail, test.py:123-152).  With ``fp6_channels`` (indices
    of ``quant_cols`` output features) ``pack`` moves those columns to the tail itself and ``forward`` writes
    every result column back to its own place inside the GEMM (``mul_fused``), so callers see W's own order.
    ``layout="gfx950"`` stores the packed words as per-tile sequential streams (``repack_gfx950``).

    ``quant_rows`` instead keeps *input* features in FP6 (``mul_rows``: every column's last ``quant_rows`` rows FP6, the
    rows before them INT4 with group-128 scales); ``fp6_in_channels`` names which ones, and ``forward`` gathers the
    activations accordingly inside the call.
    """

    FORMAT_VERSION = 1

    def __init__(self, infeatures, outfeatures, groupsize=-1, quant_cols=-1, fp6_channels=None, bias=False,
                 layout="reference", quant_rows=0, fp6_in_channels=None):
        super().__init__()
        if groupsize not in (-1, 128):
            raise ValueError("Only groupsize -1 and 128 are supported.")
        if layout not in ("reference", "gfx950"):
            raise ValueError("layout must be 'reference' or 'gfx950'")
        qc = 0 if quant_cols in (-1, 0) else quant_cols
        if infeatures % 128 or outfeatures % 128 or qc % 128 or qc > outfeatures:
            raise ValueError("infeatures, outfeatures and quant_cols must be multiples of 128")
        qr = int(quant_rows)
        if qr:
            if qc or groupsize != 128 or fp6_channels is not None:
                raise ValueError("quant_rows (FP6 on input features) needs groupsize=128 and no quant_cols / fp6_channels")
            if qr < 0 or qr >= infeatures or qr % 128:
                raise ValueError("quant_rows must be a positive multiple of 128 below infeatures")
        elif fp6_in_channels is not None:
            raise ValueError("fp6_in_channels needs quant_rows")
        self.k, self.n, self.groupsize, self.quant_cols, self.layout = infeatures, outfeatures, groupsize, quant_cols, layout
        self.quant_rows = qr
        n4 = outfeatures - qc
        if qr:
            words = (infeatures - qr) * outfeatures // 8 + qr * outfeatures * 3 // 16
            nscale = (infeatures - qr) // 128 * outfeatures + outfeatures
        else:
            words = infeatures * n4 // 8 + infeatures * qc * 3 // 16
            nscale = (n4 if groupsize == -1 else infeatures // 128 * n4) + qc
        self.register_buffer("B", torch.empty(words, dtype=torch.int32))
        self.register_buffer("s", torch.empty(nscale, dtype=torch.float16))
        self.register_buffer("meta", torch.tensor([self.FORMAT_VERSION, infeatures, outfeatures, qc, groupsize,
                                                   int(layout == "gfx950"), qr], dtype=torch.int32))
        if fp6_in_channels is not None:
            picked = torch.as_tensor(fp6_in_channels, dtype=torch.int64).reshape(-1)
            if picked.numel() != qr or picked.unique().numel() != qr or picked.min() < 0 or picked.max() >= infeatures:
                raise ValueError("fp6_in_channels must name quant_rows distinct input features")
            keep = torch.ones(infeatures, dtype=torch.bool)
            keep[picked] = False
            # packed row kk multiplies input feature a_cols[kk]: the others in order, then the chosen ones
            self.register_buffer("a_cols", torch.cat([torch.nonzero(keep).reshape(-1), picked]).to(torch.int32))
        else:
            self.a_cols = None
        if fp6_channels is not None:
            picked = torch.as_tensor(fp6_channels, dtype=torch.int64).reshape(-1)
            if picked.numel() != qc or picked.unique().numel() != qc or (qc and (picked.min() < 0 or picked.max() >= outfeatures)):
                raise ValueError("fp6_channels must name quant_cols distinct output features")
            keep = torch.ones(outfeatures, dtype=torch.bool)
            keep[picked] = False
            # packed column j holds output feature c_cols[j]: the others in order, then the chosen ones
            self.register_buffer("c_cols", torch.cat([torch.nonzero(keep).reshape(-1), picked]).to(torch.int32))
        else:
            self.c_cols = None
        if bias:
            self.register_buffer("bias", torch.zeros(outfeatures, dtype=torch.float16))
        else:
            self.bias = None

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        meta = state_dict.get(prefix + "meta")
        if meta is not None and not torch.equal(meta.cpu().to(torch.int32), self.meta.cpu()):
            raise RuntimeError(f"{prefix}: checkpoint format {meta.tolist()} does not match this layer {self.meta.tolist()} "
                               "(version, infeatures, outfeatures, quant_cols, groupsize, word order, quant_rows)")
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def pack(self, linear):
        """Quantise and pack ``linear`` (an ``nn.Linear`` or a float16 weight [outfeatures, infeatures]).
        A weight that lives on a GPU is packed there (70B-size layers take milliseconds instead of the host
        packer's seconds); the result is the same bit for bit.  Returns the dequantised weight [k, n] in W's own
        column order."""
        w = linear.weight.data if isinstance(linear, nn.Module) else linear
        w = w.detach().to(torch.float16).t().contiguous()            # [k, n], on the weight's device
        if tuple(w.shape) != (self.k, self.n):
            raise ValueError("weight shape does not match the layer")
        if self.c_cols is not None:
            w = w[:, self.c_cols.long().to(w.device)].contiguous()
        if self.quant_rows:
            if self.a_cols is not None:
                w = w[self.a_cols.long().to(w.device)].contiguous()
            B, s, w_ref = pack_row_mix_weight(w, self.quant_rows)
            if self.a_cols is not None:                            # the check weight in W's own row order
                own = torch.empty_like(w_ref)
                own[self.a_cols.long().to(w_ref.device)] = w_ref
                w_ref = own
        else:
            B, s, w_ref = pack_mixed_weight(w, self.quant_cols, self.groupsize, harness_layout=False)
        if self.layout == "gfx950":
            B = cabi.repack_gfx950(B, self.k, self.n, self.quant_cols, self.quant_rows)
        self.B.copy_(B)
        self.s.copy_(s)
        if self.bias is not None and isinstance(linear, nn.Module) and getattr(linear, "bias", None) is not None:
            self.bias.copy_(linear.bias.data.detach().to(torch.float16))
        if self.c_cols is not None:
            own = torch.empty_like(w_ref)
            own[:, self.c_cols.long().to(w_ref.device)] = w_ref
            w_ref = own
        return w_ref

    def forward(self, x, residual=None, workspace=None):
        """y = x @ W (+ bias) (+ residual, float16 of y's shape), as one GEMM call.  ``workspace``: a zeroed int32 CUDA
        tensor of at least outfeatures // 128 * 16 elements that no overlapping call uses (default: the device's
        ``shared_workspace``)."""
        x2 = x.reshape(-1, x.shape[-1]).to(torch.float16).contiguous()
        out = torch.empty((x2.shape[0], self.n), dtype=torch.float16, device=x2.device)
        res = None if residual is None else residual.reshape(-1, self.n).to(torch.float16).contiguous()
        if workspace is None:
            workspace = shared_workspace(x2.device, self.n // 128 * 16)
        elif workspace.numel() < self.n // 128 * 16 or workspace.device != x2.device:
            raise ValueError("workspace must be an int32 tensor of at least outfeatures // 128 * 16 elements on x's device")
        if self.quant_rows:
            cabi.mul_rows(x2, self.B, out, self.s, workspace, self.quant_rows, a_cols=self.a_cols, bias=self.bias,
                          residual=res, layout=self.layout)
        elif self.c_cols is None and self.bias is None and residual is None and self.layout == "reference":
            cabi.mul(x2, self.B, out, self.s, workspace, self.quant_cols, -1, -1, -1, 16, self.groupsize)
        else:
            cabi.mul_fused(x2, self.B, out, self.s, workspace, self.quant_cols, self.groupsize, c_cols=self.c_cols,
                           bias=self.bias, residual=res, layout=self.layout)
        return out.reshape(x.shape[:-1] + (self.n,))
