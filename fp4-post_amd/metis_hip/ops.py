"""Tensor-level entry points over the C ABI: quantize, dequantize, fused norm+quant, GEMMs.

All functions take CUDA (ROCm) tensors, enqueue on torch's current stream and return tensors;
PyTorch is used only to own device memory and streams.
"""
from __future__ import annotations

import functools
from dataclasses import dataclass

import torch

from . import _lib
from ._lib import DTYPE_BF16, DTYPE_F32, MODE_P32, MODE_PB16, check, load

BLOCK = 16
_workspaces: dict = {}
# Derived copies of a cached weight cost memory beside its packed form (0.5625 B per parameter): the decode layout
# (0.5625 B) for decode-sized batches, and the tiled binary16 expansions (2 B each: one per arithmetic the layer runs in,
# one more per arithmetic for the transposed operand of the NV recipe).  Memory-bound deployments switch them off:
# without the tiled copies, binary32-arithmetic GEMMs run on the packed operands, and bf16-arithmetic GEMMs expand the
# weight on every call instead of once.  A plain unsplit product has the same bits either way; a low-rank term joins
# the binary32 sum at another point on the pipelined kernel than on the packed one (1e-6 relative in binary32).
decode_layout_weights = True
tiled_weight_copies = True
# Decode-sized activations (fewer than 256 rows, a multiple of 256 columns) leave the round-to-nearest quantizers in the
# decode layout as well: written by the quantizer's second launch, read by the decode-sized GEMM as whole lines.
decode_layout_activations = True


@dataclass
class PackedNVFP4:
    """NVFP4 tensor: value[i, k] = e2m1(codes) * e4m3(scales[i, k // 16]) * unit.

    `codes` [rows, cols/2] uint8 (element 2j in the low nibble), `scales` [rows, cols/16] uint8
    (float8_e4m3fn bytes), `unit` float32[1] on the device.  (rows, cols) is the logical shape in
    the packed orientation: for column-blocked packing of x[R, C] it is (C, R).
    """
    codes: torch.Tensor
    scales: torch.Tensor
    unit: torch.Tensor
    rows: int
    cols: int
    mode: int = MODE_P32
    expanded: torch.Tensor | None = None      # cached exact f16 expansion e2m1 * e4m3 * 2^-8, see expand()
    tiled: torch.Tensor | None = None         # exact binary16 expansion in the pipelined GEMM's tiled layout, see expand_tiled()
    tiled_pb16: torch.Tensor | None = None    # the reference's bf16 dequantized values in the same layout (bf16 arithmetic)
    transposed: "PackedNVFP4 | None" = None   # cached column-blocked packing of the same source tensor (dgrad operand)
    persistent: bool = False                  # lives across calls (a cached weight): worth keeping its tiled expansion
    shared: bool = False                      # an activation read by several GEMMs (a q/k/v or gate/up group): likewise, while it lives
    rht: int | None = None                    # NV recipe: the packed values are those of the ROTATED tensor (sign mask of the rotation)
    tiled_t: torch.Tensor | None = None       # tiled expansion of the transposed tensor (contraction over this tensor's rows)
    tiled_t_pb16: torch.Tensor | None = None
    # deferred scale bytes: the quantizer stopped after its first launch and parked the block maxima here; `scales` and
    # `unit` are produced on first access (one more launch), unless a consumer that forms the bytes itself
    # (expand_tiled) got there first and wrote the unit
    deferred: torch.Tensor | None = None
    decode_layout: torch.Tensor | None = None  # a persistent weight in the layout the decode-sized kernel streams as whole lines

    def dequantize(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        return dequantize(self, dtype)

    def held_bytes(self) -> dict:
        """Device bytes this tensor holds right now, by part: the packed form and every derived copy built so far."""
        d = self.__dict__
        parts = {"packed": self.codes.numel() + (d["_scales"].numel() if d.get("_scales") is not None else 0)}
        for name in ("expanded", "tiled", "tiled_pb16", "tiled_t", "tiled_t_pb16", "decode_layout", "deferred"):
            t = d.get(name)
            if t is not None:
                parts[name] = t.numel() * t.element_size()
        if self.transposed is not None:
            parts["transposed"] = sum(self.transposed.held_bytes().values())
        return parts

    def _materialize(self) -> None:
        d = self.__dict__
        scales = torch.empty(self.rows, self.cols // BLOCK, dtype=torch.uint8, device=self.codes.device)
        rc = load().metis_nvfp4_deferred_scales(d["deferred"].data_ptr(), self.rows, self.cols, self.mode, scales.data_ptr(),
                                                d["_unit"].data_ptr(), _stream())
        check(rc, "metis_nvfp4_deferred_scales", (self.rows, self.cols))
        d["_scales"], d["_unit_ready"] = scales, True


def _packed_scales(self):
    d = self.__dict__
    if d.get("_scales") is None and d.get("deferred") is not None:
        self._materialize()
    return d.get("_scales")


def _packed_unit(self):
    d = self.__dict__
    if d.get("deferred") is not None and not d.get("_unit_ready", False):
        self._materialize()
    return d.get("_unit")


PackedNVFP4.scales = property(_packed_scales, lambda self, v: self.__dict__.__setitem__("_scales", v))
PackedNVFP4.unit = property(_packed_unit, lambda self, v: self.__dict__.__setitem__("_unit", v))


@dataclass
class CenteredNVFP4:
    """Mean-mode activation: value[i, k] = mean[k] + deq(residual)[i, k] (the column mean over tokens stays in
    high precision, only the centred residual is NVFP4).  `mean` is float32 [cols] in binary32 arithmetic,
    bf16 [cols] in bf16 arithmetic."""
    residual: PackedNVFP4
    mean: torch.Tensor
    mean32: torch.Tensor | None = None       # the same values as float32 when the producer had them at hand

    @property
    def center32(self) -> torch.Tensor:
        return self.mean32 if self.mean32 is not None else self.mean

    @property
    def rows(self) -> int:
        return self.residual.rows

    @property
    def cols(self) -> int:
        return self.residual.cols

    def dequantize(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        return self.mean.to(dtype).unsqueeze(0) + dequantize(self.residual, dtype)


@dataclass
class LowRankNVFP4:
    """"svd"-mode activation: value = us @ deq(vt) + deq(residual) (reference src/Metis/Metis/bitlinear.py:296-303).
    `us` [rows, r] is U (after its QDQ) times diag(s), in the arithmetic's type; `vt` is V after its QDQ, kept packed
    (its QDQ is the packed tensor's dequantization), so that products with a packed weight run on the packed GEMM;
    `residual` packs x - ker.  `dense` (when the producer wrote it) is the reference's own tensor ker + QDQ(x - ker)."""
    residual: PackedNVFP4
    us: torch.Tensor
    vt: PackedNVFP4
    dense: torch.Tensor | None = None

    @property
    def rows(self) -> int:
        return self.residual.rows

    @property
    def cols(self) -> int:
        return self.residual.cols

    def dequantize(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        if self.dense is not None:
            return self.dense.to(dtype)
        # without the dense tensor: a library product in the arithmetic's type (agrees with the kernel's ker to rounding)
        return (self.us @ dequantize(self.vt, self.us.dtype)).to(dtype) + dequantize(self.residual, dtype)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of torch's current stream on the current device (the raw getter skips the Stream object: this is
    called several times per layer)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _workspace(rows: int, cols: int, device: torch.device) -> torch.Tensor:
    need = load().metis_nvfp4_workspace_bytes(rows, cols)
    key = (device.index, _stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        # zero-filled once by a fill kernel (not a memset, which must not be recorded into a captured graph)
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=device).fill_(0)
        _workspaces[key] = ws
    return ws


def _as_2d_bf16(x: torch.Tensor) -> torch.Tensor:
    if not x.is_cuda:
        raise _lib.MetisHipError("metis_hip ops need a ROCm device tensor; there is no CPU path")
    if x.dtype != torch.bfloat16:
        x = x.to(torch.bfloat16)
    x2 = x.reshape(-1, x.shape[-1])
    return x2 if x2.is_contiguous() else x2.contiguous()


def _as_2d_for_quant(x: torch.Tensor, mode: int) -> tuple[torch.Tensor, int]:
    """(2-D contiguous tensor, kernel mode).  bf16 tensors go to the bf16 kernels.  In binary32 arithmetic any
    other dtype is quantized from its binary32 values (they need not be bf16 values); in bf16 arithmetic the
    tensor is first cast to bf16, as the reference casts to its compute dtype."""
    if mode == MODE_P32 and x.dtype != torch.bfloat16:
        if not x.is_cuda:
            raise _lib.MetisHipError("metis_hip ops need a ROCm device tensor; there is no CPU path")
        x2 = x.to(torch.float32).reshape(-1, x.shape[-1])
        return (x2 if x2.is_contiguous() else x2.contiguous()), _lib.MODE_P32_F32
    return _as_2d_bf16(x), mode


def quantize(x: torch.Tensor, mode: int = MODE_P32, *, col: bool = False, sr: bool = False,
             noise: torch.Tensor | None = None, seed: int = 0, offset: int = 0,
             center: torch.Tensor | None = None, resident: bool = False, spin_limit: int = 0,
             deferred: bool = False) -> PackedNVFP4:
    """NVFP4-quantize x (flattened to [R, C]).

    col=False: blocks of 16 along C -> PackedNVFP4 of shape (R, C).
    col=True : blocks of 16 along R, written transposed -> shape (C, R).
    sr=True  : stochastic rounding; `noise` (same shape as x, float32 for P32 / bf16 for PB16)
               overrides the internal Philox stream keyed by (seed, offset).
    center   : [C] vector subtracted from every row first (the reference's mean mode), in the arithmetic's
               dtype: the packed tensor is that of x - center.
    resident : round-to-nearest rows of a bf16 tensor as ONE launch (metis_nvfp4_quant_row_resident), same bytes: a
               workgroup that gives up waiting for the grid's maximum after `spin_limit` polls (0: library default)
               leaves its scale bytes to the last workgroup.
    deferred : round-to-nearest rows of a bf16 tensor: only the first of the two launches now (codes, parked block
               maxima); `scales` and `unit` of the result appear on first access, or never if the only consumer is
               expand_tiled, which forms the bytes itself.  Same bits either way.
    """
    x2, kmode = _as_2d_for_quant(x, mode)
    rows, cols = x2.shape
    blocked = rows if col else cols
    if blocked % BLOCK:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(x.shape)}")
    prow, pcol = (cols, rows) if col else (rows, cols)
    dev = x2.device
    codes = torch.empty(prow, pcol // 2, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    L = load()
    if (deferred and not col and not sr and (center is None or kmode == MODE_PB16) and kmode in (MODE_P32, MODE_PB16)
            and x2.stride(0) == cols and rows * cols > 0):
        cen = None
        if center is not None:
            cen = center.reshape(-1).to(device=dev, dtype=torch.bfloat16).contiguous()
            if cen.numel() != cols:
                raise ValueError(f"center must have one value per column ({cols}), got {cen.numel()}")
        parked = torch.empty(L.metis_nvfp4_deferred_bytes(rows, cols), dtype=torch.uint8, device=dev)
        rc = L.metis_nvfp4_quant_row_deferred(x2.data_ptr(), rows, cols, kmode, None if cen is None else cen.data_ptr(),
                                              codes.data_ptr(), parked.data_ptr(), parked.numel(), _stream())
        check(rc, "metis_nvfp4_quant_row_deferred", x.shape)
        return PackedNVFP4(codes, None, unit, prow, pcol, mode, deferred=parked)
    scales = torch.empty(prow, pcol // BLOCK, dtype=torch.uint8, device=dev)
    ws = _workspace(rows, cols, dev)
    if center is not None:
        cen = center.reshape(-1).to(device=dev, dtype=torch.bfloat16 if mode == MODE_PB16 else torch.float32).contiguous()
        if cen.numel() != cols:
            raise ValueError(f"center must have one value per column ({cols}), got {cen.numel()}")
        nz = None
        if sr and noise is not None:
            nz = noise.reshape(rows, cols).to(torch.bfloat16 if mode == MODE_PB16 else torch.float32).contiguous()
        rc = L.metis_nvfp4_quant_centered(x2.data_ptr(), rows, cols, x2.stride(0), kmode, cen.data_ptr(), int(sr), int(col),
                                          None if nz is None else nz.data_ptr(), seed & (2 ** 64 - 1), offset,
                                          codes.data_ptr(), scales.data_ptr(), unit.data_ptr(), ws.data_ptr(), ws.numel(),
                                          _stream())
        check(rc, "metis_nvfp4_quant_centered", x.shape)
        return PackedNVFP4(codes, scales, unit, prow, pcol, mode)
    if sr:
        nz = None
        if noise is not None:
            want = torch.bfloat16 if mode == MODE_PB16 else torch.float32
            nz = noise.reshape(rows, cols).to(want).contiguous()
        fn = L.metis_nvfp4_quant_sr_col if col else L.metis_nvfp4_quant_sr_row
        rc = fn(x2.data_ptr(), rows, cols, x2.stride(0), kmode, None if nz is None else nz.data_ptr(),
                seed & (2 ** 64 - 1), offset, codes.data_ptr(), scales.data_ptr(), unit.data_ptr(),
                ws.data_ptr(), ws.numel(), _stream())
    elif resident and not col and kmode in (MODE_P32, MODE_PB16) and x2.stride(0) == cols:
        rc = L.metis_nvfp4_quant_row_resident(x2.data_ptr(), rows, cols, kmode, codes.data_ptr(), scales.data_ptr(),
                                              unit.data_ptr(), ws.data_ptr(), ws.numel(), int(spin_limit), _stream())
    elif (decode_layout_activations and not col and kmode in (MODE_P32, MODE_PB16) and 0 < rows < 256 and cols % 256 == 0
          and x2.stride(0) == cols):
        dec = torch.empty(L.metis_nvfp4_decode_weight_bytes(rows, cols), dtype=torch.uint8, device=dev)
        rc = L.metis_nvfp4_quant_row_decode(x2.data_ptr(), rows, cols, kmode, codes.data_ptr(), scales.data_ptr(), unit.data_ptr(),
                                            dec.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
        check(rc, "metis_nvfp4_quant_row_decode", x.shape)
        return PackedNVFP4(codes, scales, unit, prow, pcol, mode, decode_layout=dec)
    else:
        fn = L.metis_nvfp4_quant_col if col else L.metis_nvfp4_quant_row
        rc = fn(x2.data_ptr(), rows, cols, x2.stride(0), kmode, codes.data_ptr(), scales.data_ptr(),
                unit.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_nvfp4_quant", x.shape)
    return PackedNVFP4(codes, scales, unit, prow, pcol, mode)


def quantize_dequantize(x: torch.Tensor, mode: int = MODE_P32) -> tuple[PackedNVFP4, torch.Tensor]:
    """(quantize(x, mode), its dequantized bf16 tensor) of a bf16 tensor with round to nearest, from one call of two
    launches: the second forms scale bytes and dequantized values in one pass over the codes.  Same bytes as
    quantize() followed by dequantize()."""
    if x.dtype != torch.bfloat16 or mode not in (MODE_P32, MODE_PB16):
        p = quantize(x, mode)
        return p, dequantize(p, torch.bfloat16)
    x2 = _as_2d_bf16(x)
    rows, cols = x2.shape
    if cols % BLOCK:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(x.shape)}")
    dev = x2.device
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(rows, cols // BLOCK, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    out = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev)
    ws = _workspace(rows, cols, dev)
    rc = load().metis_nvfp4_quant_dequant_row(x2.data_ptr(), rows, cols, mode, codes.data_ptr(), scales.data_ptr(), unit.data_ptr(),
                                              out.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_nvfp4_quant_dequant_row", x.shape)
    return PackedNVFP4(codes, scales, unit, rows, cols, mode), out


def quantize_lowrank_residual(x: torch.Tensor, us: torch.Tensor, vt: torch.Tensor, mode: int = MODE_P32,
                              dense: bool = False) -> tuple[PackedNVFP4, torch.Tensor | None]:
    """The packed residual QDQ(x - ker) with ker = us @ vt formed in registers (the "svd" mode of the activation
    decomposition, src/Metis/Metis/bitlinear.py:296-303), and with dense=True also ker + QDQ(x - ker).
    MODE_P32: us, vt binary32, x bf16 or binary32, dense binary32; MODE_PB16: all bf16.  x [rows, cols], us [rows, r],
    vt [r, cols], r a multiple of 16.  ker sums its r products in the order k = 0 .. r-1 with fused multiply-adds."""
    if not x.is_cuda:
        raise RuntimeError("metis_hip kernels need tensors on the GPU")
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    rows, cols = x2.shape
    r = us.shape[-1]
    want = torch.float32 if mode == MODE_P32 else torch.bfloat16
    if mode not in (MODE_P32, MODE_PB16) or us.dtype != want or vt.dtype != want:
        raise ValueError("the factors come in the arithmetic's type: binary32 for MODE_P32, bf16 for MODE_PB16")
    if x2.dtype != torch.bfloat16 and not (mode == MODE_P32 and x2.dtype == torch.float32):
        raise ValueError(f"unsupported tensor type {x2.dtype} for this arithmetic")
    if tuple(us.shape) != (rows, r) or tuple(vt.shape) != (r, cols):
        raise ValueError(f"factors {tuple(us.shape)} x {tuple(vt.shape)} do not give {tuple(x2.shape)}")
    if cols % BLOCK or r % BLOCK or r == 0:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide {tuple(x.shape)} or the rank {r}")
    us, vt = us.contiguous(), vt.contiguous()
    dev = x2.device
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(rows, cols // BLOCK, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    out = torch.empty(rows, cols, dtype=want, device=dev) if dense else None
    ws = _workspace(rows, cols, dev)
    rc = load().metis_nvfp4_quant_lowrank_residual(x2.data_ptr(), DTYPE_F32 if x2.dtype == torch.float32 else DTYPE_BF16, us.data_ptr(),
                                                   vt.data_ptr(), rows, cols, r, mode, codes.data_ptr(), scales.data_ptr(),
                                                   unit.data_ptr(), None if out is None else out.data_ptr(), ws.data_ptr(),
                                                   ws.numel(), _stream())
    check(rc, "metis_nvfp4_quant_lowrank_residual", (rows, cols, r))
    return PackedNVFP4(codes, scales, unit, rows, cols, mode), out


def quantize_both_sr(x: torch.Tensor, mode: int = MODE_P32, *, seed: int = 0, offset_row: int = 0,
                     offset_col: int = 0) -> tuple[PackedNVFP4, PackedNVFP4]:
    """(quantize(x, sr=True, offset=offset_row), quantize(x, col=True, sr=True, offset=offset_col)) from ONE pass over x:
    the two packings of an output gradient that the input-gradient and weight-gradient products contract.  Same
    bytes as the two calls.  Both dimensions of x flattened to [R, C] have to be multiples of 16."""
    x2, kmode = _as_2d_for_quant(x, mode)
    rows, cols = x2.shape
    if rows % BLOCK or cols % BLOCK:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(x.shape)} both ways")
    dev = x2.device
    L = load()
    packs = []
    for prow, pcol in ((rows, cols), (cols, rows)):
        packs.append((torch.empty(prow, pcol // 2, dtype=torch.uint8, device=dev),
                      torch.empty(prow, pcol // BLOCK, dtype=torch.uint8, device=dev),
                      torch.empty(1, dtype=torch.float32, device=dev)))
    need = 2 * L.metis_nvfp4_workspace_bytes(rows, cols)
    key = (dev.index, _stream(), "both")
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=dev).fill_(0)
        _workspaces[key] = ws
    (cr, sr_, ur), (cc, sc, uc) = packs
    if rows * cols:
        rc = L.metis_nvfp4_quant_sr_both(x2.data_ptr(), rows, cols, x2.stride(0), kmode, seed & (2 ** 64 - 1), offset_row, offset_col,
                                         cr.data_ptr(), sr_.data_ptr(), ur.data_ptr(), cc.data_ptr(), sc.data_ptr(), uc.data_ptr(),
                                         ws.data_ptr(), ws.numel(), _stream())
        check(rc, "metis_nvfp4_quant_sr_both", x.shape)
    return PackedNVFP4(cr, sr_, ur, rows, cols, mode), PackedNVFP4(cc, sc, uc, cols, rows, mode)


def dequantize(p: PackedNVFP4, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("dequantize: dtype must be bfloat16 or float32")
    out = torch.empty(p.rows, p.cols, dtype=dtype, device=p.codes.device)
    rc = load().metis_nvfp4_dequant(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols,
                                    p.mode, out.data_ptr(), DTYPE_F32 if dtype == torch.float32 else DTYPE_BF16,
                                    _stream())
    check(rc, "metis_nvfp4_dequant", (p.rows, p.cols))
    if p.rht is not None:                     # packed in the rotated domain: back to the tensor's own
        out = hadamard16(out, p.rht, inverse=True)
    return out


def hadamard16(x: torch.Tensor, sign_mask: int, inverse: bool = False) -> torch.Tensor:
    """Tiled random Hadamard rotation along the last dimension, tiles of 16: (x * sign) H, or the rotation back
    (x H) / 16 * sign (reference bitlinear.py:195-202).  bf16 or float32, same dtype out."""
    if x.dtype not in (torch.bfloat16, torch.float32) or not x.is_cuda:
        raise ValueError("hadamard16: bf16 or float32 device tensor")
    cols = x.shape[-1]
    x2 = x.reshape(-1, cols)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    out = torch.empty_like(x2)
    rc = load().metis_hadamard16(x2.data_ptr(), x2.shape[0], cols, cols, DTYPE_F32 if x.dtype == torch.float32 else DTYPE_BF16,
                                 int(inverse), int(sign_mask), out.data_ptr(), cols, _stream())
    check(rc, "metis_hadamard16", tuple(x.shape))
    return out.reshape(x.shape)


def quantize_rht(x: torch.Tensor, mode: int, sign_mask: int, *, sr: bool = False, seed: int = 0, offset: int = 0) -> PackedNVFP4:
    """Row quantizer of the ROTATED tensor (NV recipe): rotation and quantization in one pass over x.  The result
    carries `rht` = sign_mask; its dequantize() and tiled expansions rotate back."""
    x2, kmode = _as_2d_for_quant(x, mode)
    rows, cols = x2.shape
    if cols % BLOCK:
        raise ValueError(f"last dimension {cols} is not a multiple of {BLOCK}")
    dev = x2.device
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(rows, cols // BLOCK, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    ws = _workspace(rows, cols, dev)
    rc = load().metis_nvfp4_quant_row_rht(x2.data_ptr(), rows, cols, x2.stride(0), kmode, int(sign_mask), int(sr), int(seed), int(offset),
                                          codes.data_ptr(), scales.data_ptr(), unit.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_nvfp4_quant_row_rht", (rows, cols))
    return PackedNVFP4(codes, scales, unit, rows, cols, MODE_PB16 if mode == MODE_PB16 else MODE_P32, rht=int(sign_mask))


def column_sum(x: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Sum over the rows of x flattened to [R, C] -> [C] (binary32 accumulation; bf16 or float32 in and out)."""
    return column_mean(x, out_dtype, _sum_only=True)


def column_mean(x: torch.Tensor, out_dtype: torch.dtype = torch.float32, _sum_only: bool = False) -> torch.Tensor:
    """Mean over the rows of x flattened to [R, C] -> [C] (binary32 accumulation; bf16 or float32 in and out)."""
    if not x.is_cuda:
        raise _lib.MetisHipError("metis_hip ops need a ROCm device tensor; there is no CPU path")
    if x.dtype not in (torch.bfloat16, torch.float32) or out_dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("column_mean: bfloat16 or float32 tensors only")
    x2 = x.reshape(-1, x.shape[-1])
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    rows, cols = x2.shape
    out = torch.empty(cols, dtype=out_dtype, device=x2.device)
    L = load()
    ws = torch.empty(L.metis_column_mean_workspace_bytes(cols), dtype=torch.uint8, device=x2.device)
    fn = L.metis_column_sum if _sum_only else L.metis_column_mean
    rc = fn(x2.data_ptr(), rows, cols, x2.stride(0), DTYPE_F32 if x2.dtype == torch.float32 else DTYPE_BF16,
            out.data_ptr(), DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16, ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_column_sum" if _sum_only else "metis_column_mean", x.shape)
    return out


def column_mean_running(x: torch.Tensor, cached: torch.Tensor | None, cached_count: int,
                        out_dtype: torch.dtype = torch.float32) -> tuple[torch.Tensor, torch.Tensor]:
    """(me, me as float32) with me = (cached * cached_count + mean(x) * rows) / (cached_count + rows), each operation
    rounded to out_dtype (cached None: me = mean(x)).  One reduction and one small kernel; in float32 both results
    are the same tensor."""
    if not x.is_cuda:
        raise _lib.MetisHipError("metis_hip ops need a ROCm device tensor; there is no CPU path")
    if x.dtype not in (torch.bfloat16, torch.float32) or out_dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("column_mean_running: bfloat16 or float32 tensors only")
    x2 = x.reshape(-1, x.shape[-1])
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    rows, cols = x2.shape
    if cached is not None:
        cached = cached.reshape(-1).to(device=x2.device, dtype=out_dtype).contiguous()
        if cached.numel() != cols:
            raise ValueError(f"cached mean has {cached.numel()} values, the tensor {cols} columns")
    out = torch.empty(cols, dtype=out_dtype, device=x2.device)
    out32 = out if out_dtype == torch.float32 else torch.empty(cols, dtype=torch.float32, device=x2.device)
    L = load()
    ws = torch.empty(L.metis_column_mean_workspace_bytes(cols), dtype=torch.uint8, device=x2.device)
    rc = L.metis_column_mean_running(x2.data_ptr(), rows, cols, x2.stride(0), DTYPE_F32 if x2.dtype == torch.float32 else DTYPE_BF16,
                                     None if cached is None else cached.data_ptr(), int(cached_count), out.data_ptr(),
                                     None if out32 is out else out32.data_ptr(),
                                     DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16, ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_column_mean_running", x.shape)
    return out, out32


def matvec(p: PackedNVFP4, v: torch.Tensor | None = None, alpha: float = 1.0, *, out: torch.Tensor | None = None,
           split: torch.Tensor | None = None, split_col: int = 0, z: torch.Tensor | None = None,
           beta: float = 0.0) -> torch.Tensor | None:
    """y[i] = alpha * sum_k deq(p)[i, k] * v[k] (+ beta * z[i]) in binary32 (v=None: all ones, i.e. row sums).

    Returns y as float32 [rows] (written into `out` when given).  With `split` (a bf16 matrix with at least
    split_col + 3 columns) y is also stored as three bf16 terms hi + mid + lo in columns split_col..+2 of
    its rows; with split given and out=None nothing else is allocated and None is returned."""
    dev = p.codes.device
    vp = None
    if v is not None:
        v = v.reshape(-1).to(device=dev, dtype=torch.float32).contiguous()
        if v.numel() != p.cols:
            raise ValueError(f"vector length {v.numel()} does not match the packed tensor's {p.cols} columns")
        vp = v.data_ptr()
    if out is None and (split is None or z is not None):
        out = torch.empty(p.rows, dtype=torch.float32, device=dev)
    if z is not None:
        if split is not None:
            raise ValueError("matvec: the affine tail and the split output are separate entry points")
        z = z.reshape(-1).to(device=dev, dtype=torch.float32).contiguous()
        if z.numel() != p.rows:
            raise ValueError(f"z must have one value per packed row ({p.rows}), got {z.numel()}")
        rc = load().metis_nvfp4_matvec_affine(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols, vp,
                                              float(alpha), z.data_ptr(), float(beta), out.data_ptr(), _stream())
        check(rc, "metis_nvfp4_matvec_affine", (p.rows, p.cols))
        return out
    sp, sld = None, 0
    if split is not None:
        if split.dtype != torch.bfloat16 or split.dim() != 2 or split.shape[0] != p.rows or split.stride(1) != 1:
            raise ValueError("split must be a bf16 matrix with one row per packed row and unit column stride")
        sp, sld = split.data_ptr(), split.stride(0)
    rc = load().metis_nvfp4_matvec(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols, vp,
                                   float(alpha), None if out is None else out.data_ptr(), sp, sld, int(split_col), _stream())
    check(rc, "metis_nvfp4_matvec", (p.rows, p.cols))
    return out


def rank_one_operands(n: int, k: int, first: tuple | None, second: tuple | None = None):
    """(t [n, 32], u [k, 32]) bf16 with t u^T = a1 b1^T (+ a2 b2^T) to binary32 precision; first = (a1 [n], b1 [k]),
    second = (a2, b2) or None.  They go into linear_fwd as its low-rank operands."""
    pairs = [pr for pr in (first, second) if pr is not None]
    if not pairs:
        raise ValueError("rank_one_operands: at least one (a, b) pair")
    dev = pairs[0][0].device
    ptrs, keep = [], []
    for a, b in pairs:
        a = a.reshape(-1).to(torch.float32).contiguous()
        b = b.reshape(-1).to(torch.float32).contiguous()
        if a.numel() != n or b.numel() != k:
            raise ValueError("rank_one_operands: a must have n values and b must have k")
        keep += [a, b]
        ptrs += [a.data_ptr(), b.data_ptr()]
    while len(ptrs) < 4:
        ptrs.append(None)
    t = torch.empty(n, 32, dtype=torch.bfloat16, device=dev)
    u = torch.empty(k, 32, dtype=torch.bfloat16, device=dev)
    rc = load().metis_rank_one_operands(ptrs[0], ptrs[1], ptrs[2], ptrs[3], n, k, t.data_ptr(), u.data_ptr(), _stream())
    check(rc, "metis_rank_one_operands", (n, k))
    return t, u


def expand(p: PackedNVFP4) -> torch.Tensor:
    """Exact binary16 expansion e2m1(code) * e4m3(scale) * 2^-8 of a packed tensor, cached on it.

    Costs 2 B/element of HBM; it is what the compute-bound GEMM path consumes (MFMA and LDS reads only
    in its inner loop)."""
    if p.expanded is None:
        out = torch.empty(p.rows, p.cols, dtype=torch.float16, device=p.codes.device)
        rc = load().metis_nvfp4_expand_f16(p.codes.data_ptr(), p.scales.data_ptr(), p.rows, p.cols, out.data_ptr(), _stream())
        check(rc, "metis_nvfp4_expand_f16", (p.rows, p.cols))
        p.expanded = out
    return p.expanded


def expand_tiled(p: PackedNVFP4, cache: bool = True, mode: int = MODE_P32, center: torch.Tensor | None = None) -> torch.Tensor:
    """16-bit expansion of a packed tensor in the tiled layout of the pipelined GEMM (uint8 buffer): exact binary16
    values e2m1 * e4m3 * 2^-8 (mode P32) or the reference's bf16 dequantized values, unit included (mode PB16).
    cache=True keeps it on the packed tensor (weights); activations are expanded per call.
    center (bf16 [cols], mode PB16): p packs a centred residual; the operand is the mean mode's center + QDQ(x - center)
    rounded to bf16, the tensor the reference multiplies with in bf16 arithmetic."""
    L = load()
    d = p.__dict__
    lazy = d.get("deferred") is not None and d.get("_scales") is None and p.rht is None and p.cols % 32 == 0
    if center is not None:
        if mode != MODE_PB16 or p.rht is not None:
            raise ValueError("a centre goes into the bf16-arithmetic operand of an unrotated tensor")
        center = center.reshape(-1).to(torch.bfloat16).contiguous()
        if center.numel() != p.cols:
            raise ValueError(f"center must have {p.cols} values, got {center.numel()}")
        key = (center.data_ptr(), center._version)
        kept = d.get("_tiled_centered")
        if cache and kept is not None and kept[0] == key:
            return kept[1]
        out = torch.empty(L.metis_nvfp4_expand_tiled_bytes(p.rows, p.cols), dtype=torch.uint8, device=p.codes.device)
        if cache:
            d["_tiled_centered"] = (key, out, center)                 # (the centre is kept alive with its address)
        if lazy:
            rc = L.metis_nvfp4_expand_tiled_deferred(p.codes.data_ptr(), d["deferred"].data_ptr(), p.rows, p.cols, p.mode, mode,
                                                     center.data_ptr(), d["_unit"].data_ptr(), out.data_ptr(), _stream())
            d["_unit_ready"] = True
        else:
            rc = L.metis_nvfp4_expand_tiled_centered(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols,
                                                     center.data_ptr(), out.data_ptr(), _stream())
        check(rc, "metis_nvfp4_expand_tiled_centered", (p.rows, p.cols))
        return out
    have = p.tiled_pb16 if mode == MODE_PB16 else p.tiled
    if have is not None:
        return have
    out = torch.empty(L.metis_nvfp4_expand_tiled_bytes(p.rows, p.cols), dtype=torch.uint8, device=p.codes.device)
    if lazy:
        # the scale bytes were never written: this kernel forms them from the parked block maxima, and writes the unit
        rc = L.metis_nvfp4_expand_tiled_deferred(p.codes.data_ptr(), d["deferred"].data_ptr(), p.rows, p.cols, p.mode, mode,
                                                 None, d["_unit"].data_ptr(), out.data_ptr(), _stream())
        check(rc, "metis_nvfp4_expand_tiled_deferred", (p.rows, p.cols))
        d["_unit_ready"] = True
    elif p.rht is not None:                   # NV recipe: the operand holds the values rotated back
        rc = L.metis_nvfp4_expand_tiled_rht(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols, mode,
                                            p.rht, 1, 0, out.data_ptr(), _stream())
    else:
        rc = L.metis_nvfp4_expand_tiled(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols, mode,
                                        out.data_ptr(), _stream())
    check(rc, "metis_nvfp4_expand_tiled", (p.rows, p.cols))
    if cache and (tiled_weight_copies or not p.persistent):
        if mode == MODE_PB16:
            p.tiled_pb16 = out
        else:
            p.tiled = out
    return out


def expand_tiled_transposed(p: PackedNVFP4, cache: bool = False, mode: int = MODE_P32) -> torch.Tensor:
    """expand_tiled of the TRANSPOSED tensor: the operand [cols, rows] of a GEMM that contracts over this tensor's
    rows (rows % 32 == 0); a rotated tensor (NV recipe) is rotated back block by block on the way."""
    have = p.tiled_t_pb16 if mode == MODE_PB16 else p.tiled_t
    if have is not None:
        return have
    L = load()
    out = torch.empty(L.metis_nvfp4_expand_tiled_bytes(p.cols, p.rows), dtype=torch.uint8, device=p.codes.device)
    rc = L.metis_nvfp4_expand_tiled_rht(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols, mode,
                                        p.rht or 0, int(p.rht is not None), 1, out.data_ptr(), _stream())
    check(rc, "metis_nvfp4_expand_tiled_rht", (p.rows, p.cols))
    if cache and (tiled_weight_copies or not p.persistent):
        if mode == MODE_PB16:
            p.tiled_t_pb16 = out
        else:
            p.tiled_t = out
    return out


def decode_operand(p: PackedNVFP4, mode: int = MODE_P32, center: torch.Tensor | None = None, rotate: int | None = None) -> torch.Tensor:
    """The activation of a decode-sized call (rows < 256, cols % 256 == 0) as ready 16-bit MFMA operands for
    metis_linear_fwd_grouped_operand: exact binary16 values (mode P32), the reference's bf16 dequantized values (mode
    PB16), or with `center` (bf16 [cols], PB16) the mean mode's center + QDQ(x - center) rounded to bf16.
    rotate (sign mask): the call multiplies with a weight packed in the rotated domain (NV recipe); the operand then
    holds the activation's dequantized blocks rotated forward and scaled by 1/16, which gives the product with the
    weight rotated back."""
    L = load()
    out = torch.empty(L.metis_nvfp4_decode_operand_bytes(p.rows, p.cols), dtype=torch.uint8, device=p.codes.device)
    if rotate is not None:
        if center is not None or p.rht is not None:
            raise ValueError("a rotated operand is built from an unrotated, uncentred activation")
        d = p.__dict__
        lazy = d.get("deferred") is not None and d.get("_scales") is None
        rc = L.metis_nvfp4_decode_operand_rht(p.codes.data_ptr(), None if lazy else p.scales.data_ptr(),
                                              d["_unit"].data_ptr() if lazy else p.unit.data_ptr(),
                                              d["deferred"].data_ptr() if lazy else None, p.rows, p.cols, p.mode, mode, int(rotate),
                                              out.data_ptr(), _stream())
        check(rc, "metis_nvfp4_decode_operand_rht", (p.rows, p.cols))
        if lazy:
            d["_unit_ready"] = True
        return out
    if center is not None:
        center = center.reshape(-1).to(torch.bfloat16).contiguous()
        if center.numel() != p.cols:
            raise ValueError(f"center must have {p.cols} values, got {center.numel()}")
    d = p.__dict__
    if d.get("deferred") is not None and d.get("_scales") is None:
        # the scale bytes were never written: this kernel forms them from the parked block maxima, and writes the unit
        rc = L.metis_nvfp4_decode_operand_deferred(p.codes.data_ptr(), d["deferred"].data_ptr(), p.rows, p.cols, p.mode, mode,
                                                   None if center is None else center.data_ptr(), d["_unit"].data_ptr(),
                                                   out.data_ptr(), _stream())
        check(rc, "metis_nvfp4_decode_operand_deferred", (p.rows, p.cols))
        d["_unit_ready"] = True
        return out
    rc = L.metis_nvfp4_decode_operand(p.codes.data_ptr(), p.scales.data_ptr(), p.unit.data_ptr(), p.rows, p.cols, mode,
                                      None if center is None else center.data_ptr(), out.data_ptr(), _stream())
    check(rc, "metis_nvfp4_decode_operand", (p.rows, p.cols))
    return out


def grouped_operand_applies(a: PackedNVFP4, weights, ranks, center: torch.Tensor | None, reference_rounding: bool) -> bool:
    """Whether linear_fwd_grouped(a, members, center=center, reference_rounding=...) reads the activation as ready
    operands (decode_operand): bf16 arithmetic on every tensor, decode-sized shapes in wide runs.  weights: the
    members' packed weights, ranks: the widths of their low-rank terms (0 without)."""
    M, K = a.rows, a.cols
    return bool(reference_rounding and (center is None or center.dtype == torch.bfloat16) and a.mode == MODE_PB16
                and all(b.mode == MODE_PB16 and b.rht is None for b in weights) and len(weights) <= 4 and K % 256 == 0
                and all(_decode_kernel_takes(M, b.rows, K, r) for b, r in zip(weights, ranks))
                and all(b.scales.data_ptr() % 8 == 0 for b in weights))


def project_and_operand_applies(x2: torch.Tensor, v: torch.Tensor, s: torch.Tensor, p: PackedNVFP4) -> bool:
    """project_and_operand takes these: the decode-sized domain of lowrank_project (with s), and a packed form of the
    same shape whose quantizer call deferred its scale bytes, never materialized since."""
    M, K = x2.shape
    R = v.shape[0]
    d = p.__dict__
    return bool(x2.is_cuda and x2.dtype == torch.bfloat16 and v.dtype == torch.bfloat16 and s.dtype == torch.bfloat16
                and 0 < M < 256 and K % 256 == 0 and v.shape[1] == K and R % 32 == 0 and 0 < R <= 256 and s.numel() == R
                and x2.stride(1) == 1 and x2.stride(0) % 8 == 0 and x2.data_ptr() % 16 == 0
                and p.rows == M and p.cols == K and p.rht is None
                and d.get("deferred") is not None and d.get("_scales") is None)


def project_and_operand(x2: torch.Tensor, v: torch.Tensor, s: torch.Tensor, p: PackedNVFP4, mode: int = MODE_PB16,
                        center: torch.Tensor | None = None, pending: torch.Tensor | None = None, rotate: int | None = None):
    """(xv, t, operand) = lowrank_project(x2, v, s) and decode_operand(p, mode, center) of one decode-sized activation
    in two launches instead of three: the projection's finishing step rides in the operand launch.  Same bits.
    pending: the projection's partial sums as quantize_project_decode left them (the first of the two launches already
    ran beside the quantizer): one launch.  rotate (sign mask): the operand of decode_operand(p, mode, rotate=...)."""
    if rotate is not None and center is not None:
        raise ValueError("a rotated operand takes no centre")
    if not project_and_operand_applies(x2, v, s, p):
        raise ValueError("project_and_operand: outside the call's domain (see project_and_operand_applies)")
    M, K = x2.shape
    R = v.shape[0]
    L = load()
    dev = x2.device
    v = v.contiguous()
    s = s.contiguous()
    if center is not None:
        center = center.reshape(-1).to(torch.bfloat16).contiguous()
        if center.numel() != K:
            raise ValueError(f"center must have {K} values, got {center.numel()}")
    xv = torch.empty(M, R, dtype=torch.bfloat16, device=dev)
    t = torch.empty_like(xv)
    out = torch.empty(L.metis_nvfp4_decode_operand_bytes(M, K), dtype=torch.uint8, device=dev)
    need = L.metis_lowrank_project_workspace_bytes(M, R, K)
    if pending is not None and (pending.numel() < need or pending.device != dev or R > 128):
        raise ValueError("project_and_operand: `pending` is not what quantize_project_decode returns for these shapes")
    ws = pending if pending is not None else torch.empty(need, dtype=torch.uint8, device=dev)
    d = p.__dict__
    rc = L.metis_decode_prepare_deferred(None if pending is not None else x2.data_ptr(), x2.stride(0), v.data_ptr(), R, s.data_ptr(),
                                         xv.data_ptr(), t.data_ptr(),
                                         ws.data_ptr(), need, p.codes.data_ptr(), d["deferred"].data_ptr(), M, K, p.mode, mode,
                                         None if center is None else center.data_ptr(), d["_unit"].data_ptr(), out.data_ptr(),
                                         int(rotate is not None), int(rotate or 0), _stream())
    check(rc, "metis_decode_prepare_deferred", (M, K, R))
    d["_unit_ready"] = True
    return xv, t, out


def decode_weight(p: PackedNVFP4, cache: bool = True) -> torch.Tensor | None:
    """The packed weight in the decode layout (same 0.5625 B per element): rows in tiles of 32, K in steps of 256, the
    pieces of a wave's 64 lanes side by side, so that the decode-sized kernel's loads cover whole lines.  None when
    K % 256 != 0.  Kept on a persistent (cached) weight."""
    if p.decode_layout is not None:
        return p.decode_layout
    if p.cols % 256:
        return None
    L = load()
    out = torch.empty(L.metis_nvfp4_decode_weight_bytes(p.rows, p.cols), dtype=torch.uint8, device=p.codes.device)
    rc = L.metis_nvfp4_decode_weight(p.codes.data_ptr(), p.scales.data_ptr(), p.rows, p.cols, out.data_ptr(), _stream())
    check(rc, "metis_nvfp4_decode_weight", (p.rows, p.cols))
    if cache:
        p.decode_layout = out
    return out


def dense_expand_tiled(x: torch.Tensor, mode: int = MODE_P32, col_scale: torch.Tensor | None = None) -> torch.Tensor:
    """A dense [rows, cols] bf16 or float32 tensor as a tiled GEMM operand (see expand_tiled): binary16 values in mode
    P32 (pair it with a unit of 2^-8, see gemm_tiled), bf16 values in mode PB16.  col_scale (bf16 [cols]) multiplies
    column k first."""
    if x.dim() != 2 or x.dtype not in (torch.bfloat16, torch.float32) or not x.is_cuda:
        raise ValueError("dense_expand_tiled: a 2-D bf16 or float32 device tensor")
    if x.stride(1) != 1 or x.data_ptr() % 16 or x.stride(0) % (4 if x.dtype == torch.float32 else 8):
        x = x.contiguous()
    rows, cols = x.shape
    L = load()
    out = torch.empty(L.metis_nvfp4_expand_tiled_bytes(rows, cols), dtype=torch.uint8, device=x.device)
    cs = None if col_scale is None else col_scale.to(torch.bfloat16).contiguous()
    rc = L.metis_dense_expand_tiled(x.data_ptr(), rows, cols, x.stride(0), DTYPE_F32 if x.dtype == torch.float32 else DTYPE_BF16,
                                    None if cs is None else cs.data_ptr(), mode, out.data_ptr(), _stream())
    check(rc, "metis_dense_expand_tiled", (rows, cols))
    return out


@functools.lru_cache(maxsize=4096)
def _tiled_workspace_bytes(M: int, N: int, K: int, mode: int, device_index: int) -> int:
    return int(load().metis_linear_tiled_workspace_bytes(M, N, K, mode))


def gemm_tiled(ax: torch.Tensor, a_unit: torch.Tensor, bx: torch.Tensor, b_unit: torch.Tensor, M: int, N: int, K: int, *,
               mode: int = MODE_P32, t: torch.Tensor | None = None, u: torch.Tensor | None = None,
               bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16, split_k: bool = True) -> torch.Tensor:
    """out[M, N] = A B^T (+ t u^T + bias) on tiled 16-bit operands ax [M, K], bx [N, K] (see expand_tiled); mode P32:
    binary16 operands, the product times a_unit * b_unit; mode PB16: bf16 operands that hold their units, the
    reference's bf16 roundings in the epilogue."""
    dev = ax.device
    r = 0
    if t is not None:
        t = t.to(torch.bfloat16).contiguous()
        u = u.to(torch.bfloat16).contiguous()
        r = t.shape[1]
        if t.shape != (M, r) or u.shape != (N, r):
            raise ValueError("low-rank operands must be t[M, r], u[N, r]")
    bias_f32 = bias is not None and bias.dtype == torch.float32
    if bias is not None:
        bias = bias.contiguous() if bias_f32 else bias.to(torch.bfloat16).contiguous()
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    need = _tiled_workspace_bytes(M, N, K, mode, dev.index or 0) if split_k else 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
    rc = load().metis_linear_fwd_tiled(ax.data_ptr(), a_unit.data_ptr(), bx.data_ptr(), b_unit.data_ptr(), M, N, K,
                                       None if t is None else t.data_ptr(), None if u is None else u.data_ptr(), r,
                                       None if bias is None else bias.data_ptr(), int(bias_f32), out.data_ptr(),
                                       DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16, mode,
                                       None if ws is None else ws.data_ptr(), need, _stream())
    check(rc, "metis_linear_fwd_tiled", (M, N, K))
    return out


def linear_fwd_tiled(a: PackedNVFP4, b: PackedNVFP4, *, t: torch.Tensor | None = None, u: torch.Tensor | None = None,
                     bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16,
                     a_tiled: torch.Tensor | None = None, reference_rounding: bool = False,
                     split_k: bool = True, center: torch.Tensor | None = None) -> torch.Tensor:
    """linear_fwd on tiled 16-bit expansions: b's is cached on b when b is persistent, a's is made here unless given.

    reference_rounding (both operands packed in bf16 arithmetic): operands are the reference's bf16 dequantized
    values and the epilogue rounds where the reference's all-bf16 forward rounds; otherwise exact products.
    center (bf16 [K], with reference_rounding): `a` packs the centred residual of the mean mode and the activation
    operand is the reference's bf16 tensor center + QDQ(x - center)."""
    if a.cols != b.cols:
        raise ValueError(f"contraction mismatch: {a.cols} vs {b.cols}")
    mode = MODE_P32
    if reference_rounding:
        if a.mode != MODE_PB16 or b.mode != MODE_PB16:
            raise ValueError("reference_rounding needs both operands packed in bf16 arithmetic")
        mode = MODE_PB16
    elif center is not None:
        raise ValueError("a centre inside the operand belongs to reference_rounding")
    bx = expand_tiled(b, cache=b.persistent, mode=mode)
    ax = a_tiled if a_tiled is not None else expand_tiled(a, cache=a.shared, mode=mode, center=center)
    return gemm_tiled(ax, a.unit, bx, b.unit, a.rows, b.rows, a.cols, mode=mode, t=t, u=u, bias=bias, out_dtype=out_dtype,
                      split_k=split_k)


def rmsnorm_quantize(x: torch.Tensor, gamma: torch.Tensor, eps: float, mode: int = MODE_P32,
                     want_normed: bool = True, deferred: bool = False):
    """Fused RMSNorm -> NVFP4.  Returns (normed bf16 or None, PackedNVFP4).  deferred: as in quantize (one launch; scale
    bytes and unit on first access, or formed by expand_tiled)."""
    x2 = _as_2d_bf16(x)
    rows, cols = x2.shape
    if cols % BLOCK:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(x.shape)}")
    g = gamma.to(device=x2.device, dtype=torch.bfloat16).contiguous()
    dev = x2.device
    normed = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev) if want_normed else None
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    if deferred and rows * cols > 0:
        L = load()
        parked = torch.empty(L.metis_nvfp4_deferred_bytes(rows, cols), dtype=torch.uint8, device=dev)
        rc = L.metis_rmsnorm_nvfp4_quant_deferred(x2.data_ptr(), g.data_ptr(), float(eps), rows, cols, mode,
                                                  None if normed is None else normed.data_ptr(), codes.data_ptr(),
                                                  parked.data_ptr(), parked.numel(), _stream())
        check(rc, "metis_rmsnorm_nvfp4_quant_deferred", x.shape)
        if normed is not None:
            normed = normed.reshape(x.shape)
        return normed, PackedNVFP4(codes, None, unit, rows, cols, mode, deferred=parked)
    scales = torch.empty(rows, cols // BLOCK, dtype=torch.uint8, device=dev)
    ws = _workspace(rows, cols, dev)
    dec = None
    if decode_layout_activations and 0 < rows < 256 and cols % 256 == 0:
        L = load()
        dec = torch.empty(L.metis_nvfp4_decode_weight_bytes(rows, cols), dtype=torch.uint8, device=dev)
        rc = L.metis_rmsnorm_nvfp4_quant_decode(x2.data_ptr(), g.data_ptr(), float(eps), rows, cols, mode,
                                                None if normed is None else normed.data_ptr(), codes.data_ptr(),
                                                scales.data_ptr(), unit.data_ptr(), dec.data_ptr(), ws.data_ptr(), ws.numel(),
                                                _stream())
    else:
        rc = load().metis_rmsnorm_nvfp4_quant(x2.data_ptr(), g.data_ptr(), float(eps), rows, cols, mode,
                                              None if normed is None else normed.data_ptr(), codes.data_ptr(),
                                              scales.data_ptr(), unit.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_rmsnorm_nvfp4_quant", x.shape)
    if normed is not None:
        normed = normed.reshape(x.shape)
    return normed, PackedNVFP4(codes, scales, unit, rows, cols, mode, decode_layout=dec)


def rmsnorm_colmean(x: torch.Tensor, gamma: torch.Tensor, eps: float, mean_dtype: torch.dtype = torch.float32,
                    cached: torch.Tensor | None = None, cached_count: int = 0):
    """RMSNorm for the mean mode: (normed bf16 [R, C], column mean of normed over its rows in mean_dtype, the same as
    float32) from one pass over x plus one small kernel.  cached / cached_count: the weighted running mean of
    single-token decode calls, as column_mean_running.  C <= 4096."""
    x2 = _as_2d_bf16(x)
    rows, cols = x2.shape
    if cols % BLOCK:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(x.shape)}")
    if mean_dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("rmsnorm_colmean: the mean is bfloat16 or float32")
    dev = x2.device
    g = gamma.to(device=dev, dtype=torch.bfloat16).contiguous()
    normed = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev)
    me = torch.empty(cols, dtype=mean_dtype, device=dev)
    me32 = me if mean_dtype == torch.float32 else torch.empty(cols, dtype=torch.float32, device=dev)
    L = load()
    ws = torch.empty(max(L.metis_rmsnorm_colmean_workspace_bytes(rows, cols), 16), dtype=torch.uint8, device=dev)
    cp = None
    if cached is not None:
        cached = cached.reshape(-1).to(device=dev, dtype=mean_dtype).contiguous()
        if cached.numel() != cols:
            raise ValueError(f"cached mean must have one value per column ({cols}), got {cached.numel()}")
        cp = cached.data_ptr()
    rc = L.metis_rmsnorm_colmean(x2.data_ptr(), g.data_ptr(), float(eps), rows, cols, normed.data_ptr(), me.data_ptr(),
                                 DTYPE_F32 if mean_dtype == torch.float32 else DTYPE_BF16, cp, int(cached_count),
                                 None if me32 is me else me32.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_rmsnorm_colmean", x.shape)
    return normed, me, me32


@functools.lru_cache(maxsize=16)
def _device_cus(device_index: int) -> int:
    return int(torch.cuda.get_device_properties(device_index).multi_processor_count)


def _tiled_applies(a: PackedNVFP4, b: PackedNVFP4) -> bool:
    """The pipelined GEMM on tiled binary16 expansions pays when the weight-side expansion is reused across calls
    (a cached weight) and the batch fills a 256-row tile; the activation side is expanded per call (2.56 B/element,
    about 2 % of the GEMM's time at such shapes)."""
    if not ((b.persistent and tiled_weight_copies) or b.tiled is not None):
        return False
    M, N, K = a.rows, b.rows, a.cols
    return M >= 256 and N >= 256 and K % 32 == 0 and K >= 128


@functools.lru_cache(maxsize=4096)
def _linear_workspace_bytes(M: int, N: int, K: int, device_index: int) -> int:
    return int(load().metis_linear_workspace_bytes(M, N, K))          # depends on the device's CU count only


@functools.lru_cache(maxsize=4096)
def _lowrank_workspace_bytes(M: int, R: int, K: int) -> int:
    return int(load().metis_lowrank_project_workspace_bytes(M, R, K))


@functools.lru_cache(maxsize=4096)
def _grouped_plan(M: int, K: int, ns: tuple, device_index: int) -> tuple[int, bool]:
    """(split-K scratch bytes, whether a centre can ride inside the launch) of a grouped call; shape-only queries."""
    import ctypes
    arr = (_lib.LinearMember * len(ns))()
    for i, n in enumerate(ns):
        arr[i].N = n
    ap = ctypes.cast(arr, ctypes.c_void_p)
    L = load()
    need = int(L.metis_linear_grouped_workspace_bytes(M, K, ap, len(ns)))
    return need, bool(L.metis_linear_grouped_centered_supported(M, K, ap, len(ns), int(need > 0)))


def _gemm_workspace(M: int, N: int, K: int, device: torch.device) -> torch.Tensor | None:
    """Split-K scratch for an M x N output contracted over K, or None when the shape is not split.

    Taken from torch's caching allocator per call (stream-ordered, so overlapping streams and captured
    graphs each get their own) rather than cached here."""
    if M >= 256 and N < 256:
        return None
    need = _linear_workspace_bytes(M, N, K, device.index or 0)
    return torch.empty(need, dtype=torch.uint8, device=device) if need else None


def nv_decode_applies(a: PackedNVFP4, weights, ranks) -> bool:
    """A decode-sized call against weights packed in the rotated domain (NV recipe) runs on the decode-sized kernel,
    the rotation carried by the activation's operand: one rotation for all members, an unrotated activation, the
    kernel's shapes in wide runs."""
    masks = {b.rht for b in weights}
    return bool(len(masks) == 1 and None not in masks and a.rht is None and len(weights) <= 4 and a.cols % 256 == 0
                and all(_decode_kernel_takes(a.rows, b.rows, a.cols, r) for b, r in zip(weights, ranks))
                and all(b.scales.data_ptr() % 8 == 0 for b in weights))


def nv_operand_mode(a: PackedNVFP4, weights, reference_rounding: bool) -> int:
    """The format of the rotated operand of a decode-sized NV-recipe call: the reference's bf16 values when the call
    follows its all-bf16 evaluation (every tensor packed in bf16 arithmetic), exact binary16 otherwise."""
    return MODE_PB16 if (reference_rounding and a.mode == MODE_PB16 and all(b.mode == MODE_PB16 for b in weights)) else MODE_P32


def _decode_kernel_takes(M: int, N: int, K: int, r: int) -> bool:
    """Shapes of the decode-sized kernel (waves split K over packed operands streamed from global memory)."""
    return 0 < M < 256 and K % 64 == 0 and N % 4 == 0 and r % 32 == 0


def linear_fwd(a: PackedNVFP4, b: PackedNVFP4, *, t: torch.Tensor | None = None, u: torch.Tensor | None = None,
               bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16,
               expanded: bool | None = None, split_k: bool = True, tiled: bool | None = None,
               reference_rounding: bool = False, a_operand: torch.Tensor | None = None) -> torch.Tensor:
    """out[M, N] = deq(a)[M, K] . deq(b)[N, K]^T (+ t[M, r] . u[N, r]^T) (+ bias[N]).

    tiled=None picks the pipelined kernel on tiled binary16 expansions when b is a cached weight and the shape is
    large (see _tiled_applies), or when the product is large enough to pay for expansions made for this one call
    (_tiled_backward_pays); True / False force the choice.  Same products either way; a plain unsplit product has the
    same bits, a low-rank term joins the binary32 sum at another point (1e-6 relative in binary32).
    reference_rounding: the forward of a layer whose arithmetic is bf16 (both operands packed in that mode): follow the
    reference's all-bf16 evaluation (twice-rounded bf16 operands, residual product and bias add rounded to bf16): the
    pipelined kernel from 256 rows on, the decode-sized kernel below (shapes it does not take get exact products).

    split_k=False withholds the split-K workspace: the contraction then runs unsplit in one launch.

    expanded=True runs on cached exact f16 expansions of a and b (2 B/element extra HBM, inner loop of
    MFMA + LDS reads only); the default works on the packed operands directly.
    a_operand: as in linear_fwd_grouped (a decode-sized call in bf16 arithmetic)."""
    if a.cols != b.cols:
        raise ValueError(f"contraction mismatch: {a.cols} vs {b.cols}")
    if (tiled is None and not expanded and b.rht is not None
            and nv_decode_applies(a, [b], [0 if t is None else t.shape[1]])):
        # NV recipe at decode size: the packed rotated weight is streamed as it is, the activation's operand is rotated
        return _linear_fwd_grouped(a, [(b, t, u, bias)], out_dtype=out_dtype, split_k=split_k,
                                   reference_rounding=reference_rounding, a_operand=a_operand)[0]
    if a.rht is not None or b.rht is not None:
        # NV recipe: only the tiled operands know how to rotate a block back
        if a.cols % 32:
            raise ValueError("a rotated operand needs a contraction that is a multiple of 32")
        tiled = True
    rounded = reference_rounding and a.mode == MODE_PB16 and b.mode == MODE_PB16
    faithful = rounded and (a.rows >= 256 or tiled) and a.cols % 32 == 0
    if tiled is None:
        tiled = faithful or (not expanded and (_tiled_applies(a, b) or _tiled_backward_pays(a.rows, b.rows, a.cols, a.codes.device.index or 0)))
    if tiled:
        return linear_fwd_tiled(a, b, t=t, u=u, bias=bias, out_dtype=out_dtype, reference_rounding=faithful, split_k=split_k)
    M, N, K = a.rows, b.rows, a.cols
    if rounded and not expanded and _decode_kernel_takes(M, N, K, 0 if t is None else t.shape[1]):
        return _linear_fwd_grouped(a, [(b, t, u, bias)], out_dtype=out_dtype, split_k=split_k, reference_rounding=True,
                                   a_operand=a_operand)[0]
    dev = a.codes.device
    r = 0
    if t is not None:
        t = t.to(torch.bfloat16).contiguous()
        u = u.to(torch.bfloat16).contiguous()
        r = t.shape[1]
        if t.shape != (M, r) or u.shape != (N, r):
            raise ValueError("low-rank operands must be t[M, r], u[N, r]")
    bias_f32 = bias is not None and bias.dtype == torch.float32     # e.g. bias + W^ me of the mean mode
    if bias is not None:
        bias = bias.contiguous() if bias_f32 else bias.to(torch.bfloat16).contiguous()
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    dt = DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16
    tp = None if t is None else t.data_ptr()
    up = None if u is None else u.data_ptr()
    bp = None if bias is None else bias.data_ptr()
    if expanded is None:
        # measured on MI355X: the packed kernel (expansion inside the K loop, 16 KiB/step of operand traffic)
        # is within 5 % of the expanded one at 8192x4096x14336 and faster on smaller shapes, so it is the default
        expanded = False
    if expanded and bias_f32:
        raise ValueError("the expanded-operand path takes a bf16 bias")
    if expanded:
        ae, be = expand(a), expand(b)
        rc = load().metis_linear_fwd_expanded(ae.data_ptr(), a.unit.data_ptr(), be.data_ptr(), b.unit.data_ptr(), M, N, K,
                                              tp, up, r, bp, out.data_ptr(), dt, _stream())
        check(rc, "metis_linear_fwd_expanded", (M, N, K))
        return out
    ws = _gemm_workspace(M, N, K, dev) if split_k else None
    if bias_f32:
        rc = load().metis_linear_fwd_f32bias(a.codes.data_ptr(), a.scales.data_ptr(), a.unit.data_ptr(), b.codes.data_ptr(),
                                             b.scales.data_ptr(), b.unit.data_ptr(), M, N, K, tp, up, r, bp, out.data_ptr(), dt,
                                             None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), _stream())
        check(rc, "metis_linear_fwd_f32bias", (M, N, K))
        return out
    if ws is not None:
        rc = load().metis_linear_fwd_ws(a.codes.data_ptr(), a.scales.data_ptr(), a.unit.data_ptr(), b.codes.data_ptr(),
                                        b.scales.data_ptr(), b.unit.data_ptr(), M, N, K, tp, up, r, bp, out.data_ptr(), dt,
                                        ws.data_ptr(), ws.numel(), _stream())
        check(rc, "metis_linear_fwd_ws", (M, N, K))
        return out
    rc = load().metis_linear_fwd(a.codes.data_ptr(), a.scales.data_ptr(), a.unit.data_ptr(), b.codes.data_ptr(),
                                 b.scales.data_ptr(), b.unit.data_ptr(), M, N, K, tp, up, r, bp, out.data_ptr(), dt, _stream())
    check(rc, "metis_linear_fwd", (M, N, K))
    return out


def lowrank_project(x2: torch.Tensor, v: torch.Tensor, s: torch.Tensor | None = None):
    """Rank-r projection of the low-rank branch: xv = x2[M, K] . v[R, K]^T in bf16 (binary32 accumulation) and, with
    `s` [R], t = bf16(xv * s): returns xv or (xv, t).  Decode-sized batches (M < 256, R <= 256) run on the library's
    split-K kernel, larger ones (R in 32 / 64 / 128) on its one-pass kernel; other shapes are a torch matmul."""
    M, K = x2.shape
    R = v.shape[0]
    common = (x2.is_cuda and x2.dtype == torch.bfloat16 and v.dtype == torch.bfloat16 and M > 0 and K % 64 == 0 and v.shape[1] == K
              and x2.stride(1) == 1 and x2.stride(0) % 8 == 0 and x2.data_ptr() % 16 == 0 and (s is None or s.dtype == torch.bfloat16))
    small = common and M < 256 and R % 32 == 0 and 0 < R <= 256
    large = common and M >= 256 and R in (32, 64, 128)
    if not (small or large):
        xv = torch.matmul(x2, v.T)
        return xv if s is None else (xv, xv * s.to(xv.dtype))
    v = v.contiguous()
    L = load()
    xv = torch.empty(M, R, dtype=torch.bfloat16, device=x2.device)
    t = None if s is None else torch.empty_like(xv)
    sp = None if s is None else s.contiguous().data_ptr()
    if large:
        need = L.metis_lowrank_project_rows_workspace_bytes(M, R, K)
        ws = torch.empty(need, dtype=torch.uint8, device=x2.device) if need else None
        rc = L.metis_lowrank_project_rows_ws(x2.data_ptr(), x2.stride(0), v.data_ptr(), M, R, K, sp, xv.data_ptr(),
                                             None if t is None else t.data_ptr(), None if ws is None else ws.data_ptr(), need, _stream())
        check(rc, "metis_lowrank_project_rows_ws", (M, R, K))
        return xv if s is None else (xv, t)
    ws = torch.empty(_lowrank_workspace_bytes(M, R, K), dtype=torch.uint8, device=x2.device)
    rc = L.metis_lowrank_project(x2.data_ptr(), x2.stride(0), v.data_ptr(), M, R, K, sp,
                                 xv.data_ptr(), None if t is None else t.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    check(rc, "metis_lowrank_project", (M, R, K))
    return xv if s is None else (xv, t)


def quantize_project_applies(x2: torch.Tensor, v: torch.Tensor, mode: int) -> bool:
    """quantize_project takes this activation: a contiguous bf16 [M, K] from 256 to 65536 rows, K a multiple of 64, a bf16
    V of 32 or 64 rows."""
    M, K = x2.shape
    return (x2.is_cuda and x2.dtype == torch.bfloat16 and v.dtype == torch.bfloat16 and 256 <= M <= 65536 and K % 64 == 0
            and v.shape[0] in (32, 64) and v.shape[1] == K and x2.is_contiguous() and x2.data_ptr() % 16 == 0
            and mode in (MODE_P32, MODE_PB16))


def quantize_project(x2: torch.Tensor, v: torch.Tensor, s: torch.Tensor, mode: int = MODE_P32):
    """(quantize(x2, mode, deferred=True), xv, t) from ONE pass over the activation: the packed tensor that feeds the
    residual branch and the rank-r projection xv = x2 . v^T, t = bf16(xv * s) of the low-rank branch (lowrank_project).
    The packed tensor has the bytes of quantize(); xv is the K-sliced sum of lowrank_project."""
    if not quantize_project_applies(x2, v, mode):
        raise ValueError("quantize_project: shape or dtype outside the kernel's domain (see quantize_project_applies)")
    M, K = x2.shape
    R = v.shape[0]
    dev = x2.device
    L = load()
    v = v.contiguous()
    s = s.to(torch.bfloat16).contiguous()
    xv = torch.empty(M, R, dtype=torch.bfloat16, device=dev)
    t = torch.empty_like(xv)
    codes = torch.empty(M, K // 2, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    parked = torch.empty(L.metis_nvfp4_deferred_bytes(M, K), dtype=torch.uint8, device=dev)
    need = L.metis_lowrank_project_rows_workspace_bytes(M, R, K)
    ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
    rc = L.metis_nvfp4_quant_project_deferred(x2.data_ptr(), M, K, mode, v.data_ptr(), R, s.data_ptr(), xv.data_ptr(), t.data_ptr(),
                                              codes.data_ptr(), parked.data_ptr(), parked.numel(),
                                              None if ws is None else ws.data_ptr(), need, _stream())
    check(rc, "metis_nvfp4_quant_project_deferred", (M, K, R))
    return PackedNVFP4(codes, None, unit, M, K, mode, deferred=parked), xv, t


def quantize_project_decode_applies(x2: torch.Tensor, v: torch.Tensor, mode: int) -> bool:
    """quantize_project_decode takes this activation: a contiguous bf16 [M, K] of fewer than 256 rows, K a multiple of
    256 (what the consumer of the pending sums, project_and_operand, needs), a bf16 V of 32 to 128 rows."""
    M, K = x2.shape
    return bool(x2.is_cuda and x2.dtype == torch.bfloat16 and v.dtype == torch.bfloat16 and 0 < M < 256 and K % 256 == 0
                and v.shape[0] % 32 == 0 and 0 < v.shape[0] <= 128 and v.shape[1] == K and x2.is_contiguous()
                and x2.data_ptr() % 16 == 0 and mode in (MODE_P32, MODE_PB16))


def quantize_project_decode(x2: torch.Tensor, v: torch.Tensor, mode: int = MODE_PB16):
    """(quantize(x2, mode, deferred=True), pending) from ONE launch over a decode-sized activation: the packed tensor and
    the partial sums of its rank-r projection x2 . v^T, which project_and_operand(..., pending=pending) finishes in the
    launch that also builds the GEMM operands.  Same bits as the separate calls."""
    if not quantize_project_decode_applies(x2, v, mode):
        raise ValueError("quantize_project_decode: outside the call's domain (see quantize_project_decode_applies)")
    M, K = x2.shape
    R = v.shape[0]
    dev = x2.device
    L = load()
    v = v.contiguous()
    codes = torch.empty(M, K // 2, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    parked = torch.empty(L.metis_nvfp4_deferred_bytes(M, K), dtype=torch.uint8, device=dev)
    need = L.metis_lowrank_project_workspace_bytes(M, R, K)
    pending = torch.empty(need, dtype=torch.uint8, device=dev)
    rc = L.metis_decode_quant_project_deferred(x2.data_ptr(), M, K, mode, codes.data_ptr(), parked.data_ptr(), parked.numel(),
                                               v.data_ptr(), R, pending.data_ptr(), need, _stream())
    check(rc, "metis_decode_quant_project_deferred", (M, K, R))
    return PackedNVFP4(codes, None, unit, M, K, mode, deferred=parked), pending


def lowrank_contract_tokens(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                            transpose: bool = False) -> torch.Tensor:
    """sum_l a[l, C] b[l, R] -> [C, R] (or [R, C] with transpose): the rank-r products of the backward pass that
    contract over tokens, bf16 operands, binary32 accumulation.  R in 32 / 64 / 128 on the library's kernel; other
    shapes are a torch matmul."""
    Lt, C = a.shape
    R = b.shape[1]
    ok = (a.is_cuda and a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16 and b.shape[0] == Lt and Lt > 0 and R in (32, 64, 128)
          and C % 8 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
          and out_dtype in (torch.bfloat16, torch.float32))
    if not ok:
        out = torch.matmul(a.T, b).to(out_dtype)
        return out.T.contiguous() if transpose else out
    b = b.contiguous()
    L = load()
    out = torch.empty((R, C) if transpose else (C, R), dtype=out_dtype, device=a.device)
    need = int(L.metis_lowrank_tokens_workspace_bytes(Lt, C, R))
    ws = torch.empty(need, dtype=torch.uint8, device=a.device)
    rc = L.metis_lowrank_contract_tokens(a.data_ptr(), a.stride(0), b.data_ptr(), Lt, C, R, out.data_ptr(),
                                         DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16, int(transpose),
                                         ws.data_ptr(), need, _stream())
    check(rc, "metis_lowrank_contract_tokens", (Lt, C, R))
    return out


def lowrank_scale_grad(g: torch.Tensor, xv: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """sum_l bf16(g[l, :] * xv[l, :]) -> [R]: the gradient of s in y = s * (x V^T), as (g * xv).sum(0, dtype=float32) on bf16
    tensors computes it (the product rounded to bf16), in one launch and a fixed summation order; out_dtype bfloat16
    rounds the binary32 sum once, as .to(bfloat16) would."""
    R = g.shape[-1]
    if not (g.is_cuda and g.dtype == torch.bfloat16 and xv.dtype == torch.bfloat16 and g.shape == xv.shape and g.dim() == 2
            and R % 8 == 0 and g.is_contiguous() and xv.is_contiguous() and g.data_ptr() % 16 == 0 and xv.data_ptr() % 16 == 0
            and out_dtype in (torch.float32, torch.bfloat16)):
        return (g * xv).sum(dim=0, dtype=torch.float32).to(out_dtype)
    out = torch.empty(R, dtype=out_dtype, device=g.device)
    rc = load().metis_lowrank_scale_grad(g.data_ptr(), xv.data_ptr(), g.shape[0], R, out.data_ptr(),
                                         DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16, _stream())
    check(rc, "metis_lowrank_scale_grad", tuple(g.shape))
    return out


def linear_fwd_grouped(a: PackedNVFP4, members, out_dtype: torch.dtype = torch.bfloat16,
                       center: torch.Tensor | None = None, split_k: bool = True,
                       reference_rounding: bool = False, a_operand: torch.Tensor | None = None) -> list[torch.Tensor]:
    return _linear_fwd_grouped(a, members, out_dtype, center, split_k, reference_rounding, a_operand)


def _linear_fwd_grouped(a: PackedNVFP4, members, out_dtype: torch.dtype = torch.bfloat16,
                        center: torch.Tensor | None = None, split_k: bool = True,
                        reference_rounding: bool = False, a_operand: torch.Tensor | None = None) -> list[torch.Tensor]:
    """[linear_fwd(a, b, t=t, u=u, bias=bias) for (b, t, u, bias) in members] in one call: a projection group
    (q/k/v, gate/up) that shares one packed activation.  Decode-sized batches run as a single launch.

    reference_rounding (every operand packed in bf16 arithmetic): the reference's all-bf16 evaluation, as in
    linear_fwd; shapes the decode-sized kernel does not take are served member by member.  A bf16 `center` then goes
    into the activation operand itself (the reference's bf16 tensor center + QDQ(x - center)); a float32 centre keeps
    exact products with the centre's share accumulated in binary32.

    center (mean mode: `a` packs the centred residual X - center): every output row also receives deq(b) . center,
    inside the same launch where the shape allows, else through matvec and a binary32 bias.

    a_operand: decode_operand(a, MODE_PB16, center) when the caller has it already (project_and_operand); read only
    where grouped_operand_applies says the call reads ready operands."""
    import ctypes
    M, K = a.rows, a.cols
    dev = a.codes.device
    rounded = (reference_rounding and (center is None or center.dtype == torch.bfloat16) and a.mode == MODE_PB16
               and all(m[0].mode == MODE_PB16 for m in members))
    takes = len(members) <= 4 and all(_decode_kernel_takes(M, m[0].rows, K, 0 if m[1] is None else m[1].shape[1]) for m in members)
    # NV recipe: weights packed in the rotated domain.  The decode-sized kernel streams them as they are and the
    # activation's operand carries the rotation (decode_operand(rotate=...)); callers check nv_decode_applies first
    rotate = None
    masks = {m[0].rht for m in members}
    if masks != {None}:
        if len(masks) != 1 or a.rht is not None or center is not None or not takes or K % 256 \
                or any(m[0].scales.data_ptr() % 8 for m in members):
            raise ValueError("rotated weights: one rotation for all members of a decode-sized call on an unrotated, uncentred "
                             "activation (see nv_decode_applies); other calls take the tiled GEMM")
        rotate = masks.pop()
    # ready operands (built once for the group): wide runs only
    operand = grouped_operand_applies(a, [m[0] for m in members], [0 if m[1] is None else m[1].shape[1] for m in members],
                                      center, reference_rounding)
    if rounded and center is not None and not operand:
        if M >= 256 and K % 32 == 0:
            ax = expand_tiled(a, cache=a.shared, mode=MODE_PB16, center=center)
            return [linear_fwd_tiled(a, b, t=t, u=u, bias=bias, out_dtype=out_dtype, a_tiled=ax, reference_rounding=True, split_k=split_k)
                    for b, t, u, bias in members]
        rounded = False                                        # exact products, the centre's share in binary32
    if rounded and not takes:
        return [linear_fwd(a, b, t=t, u=u, bias=bias, out_dtype=out_dtype, split_k=split_k, reference_rounding=True)
                for b, t, u, bias in members]
    arr = (_lib.LinearMember * len(members))()
    outs, keep = [], []
    for i, (b, t, u, bias) in enumerate(members):
        if b.cols != K:
            raise ValueError(f"contraction mismatch: {K} vs {b.cols}")
        r = ldt = 0
        if t is not None:
            t, u = t.to(torch.bfloat16), u.to(torch.bfloat16).contiguous()
            r = t.shape[1]
            if t.shape != (M, r) or u.shape != (b.rows, r):
                raise ValueError("low-rank operands must be t[M, r], u[N, r]")
            # a column slice of a stacked projection is taken as it is by the single-launch path
            strided_ok = M < 256 and K % 64 == 0 and t.stride(1) == 1 and t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0
            if t.is_contiguous() or not strided_ok:
                t = t.contiguous()
            else:
                ldt = t.stride(0)
        bias_f32 = bias is not None and bias.dtype == torch.float32
        if bias is not None:
            bias = bias.contiguous() if bias_f32 else bias.to(torch.bfloat16).contiguous()
        out = torch.empty(M, b.rows, dtype=out_dtype, device=dev)
        keep += [t, u, bias]
        outs.append(out)
        # a cached weight is streamed in its decode layout (whole lines per load instruction) by the decode-sized kernel
        dec = decode_weight(b) if (b.persistent and takes and M < 256 and decode_layout_weights) else None
        arr[i] = _lib.LinearMember(b.codes.data_ptr(), b.scales.data_ptr(), b.unit.data_ptr(),
                                   None if t is None else t.data_ptr(), None if u is None else u.data_ptr(), r,
                                   None if bias is None else bias.data_ptr(), out.data_ptr(), b.rows, int(bias_f32), ldt,
                                   None if dec is None else dec.data_ptr())
    L = load()
    ap = ctypes.cast(arr, ctypes.c_void_p)
    # split-K scratch (long K, few columns) and whether a centre fits the launch: functions of the shape alone
    need, centre_ok = _grouped_plan(M, K, tuple(m[0].rows for m in members), dev.index or 0)
    if not split_k:
        need, centre_ok = 0, bool(load().metis_linear_grouped_centered_supported(
            M, K, ctypes.cast(arr, ctypes.c_void_p), len(members), 0))
    ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
    dt = DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16
    if rotate is not None:
        op_mode = MODE_PB16 if rounded else MODE_P32          # (nv_operand_mode: what a caller that brings a_operand built it in)
        aop = a_operand if a_operand is not None else decode_operand(a, op_mode, None, rotate=rotate)
        rc = L.metis_linear_fwd_grouped_operand(aop.data_ptr(), a.unit.data_ptr(), M, K, ap, len(members), dt, op_mode,
                                                None if ws is None else ws.data_ptr(), need, _stream())
        check(rc, "metis_linear_fwd_grouped_operand", (M, K, [m[0].rows for m in members]))
        return outs
    if operand:
        # (a quantizer call that deferred its scale bytes never gets them: the operand kernel forms them on the way)
        aop = a_operand if a_operand is not None else decode_operand(a, MODE_PB16, center)
        rc = L.metis_linear_fwd_grouped_operand(aop.data_ptr(), a.unit.data_ptr(), M, K, ap, len(members), dt, MODE_PB16,
                                                None if ws is None else ws.data_ptr(), need, _stream())
        check(rc, "metis_linear_fwd_grouped_operand", (M, K, [m[0].rows for m in members]))
        return outs
    # the activation's decode layout (written by its quantizer) in place of the row-major packing: wide runs only
    a_dec = a.decode_layout if (takes and K % 256 == 0 and all(m[0].scales.data_ptr() % 8 == 0 for m in members)) else None
    a_codes, a_scales = (a_dec.data_ptr(), None) if a_dec is not None else (a.codes.data_ptr(), a.scales.data_ptr())
    if center is not None:
        center = center.reshape(-1).to(device=dev, dtype=torch.float32).contiguous()
        if center.numel() != K:
            raise ValueError(f"center must have {K} values, got {center.numel()}")
        aligned = center.data_ptr() % 16 == 0 and all(m[0].scales.data_ptr() % 8 == 0 for m in members) and a.scales.data_ptr() % 8 == 0
        if aligned and centre_ok:
            rc = L.metis_linear_fwd_grouped_centered(a_codes, a_scales, a.unit.data_ptr(), M, K, ap,
                                                     len(members), dt, center.data_ptr(),
                                                     None if ws is None else ws.data_ptr(), need, _stream())
            check(rc, "metis_linear_fwd_grouped_centered", (M, K, [m[0].rows for m in members]))
            return outs
        # two passes: W^ center as a binary32 bias per member
        shifted = []
        for b, t, u, bias in members:
            w_mean = matvec(b, center)
            shifted.append((b, t, u, w_mean if bias is None else w_mean + bias.float()))
        return _linear_fwd_grouped(a, shifted, out_dtype)
    fn = L.metis_linear_fwd_grouped_bf16 if rounded else L.metis_linear_fwd_grouped
    rc = fn(a_codes, a_scales, a.unit.data_ptr(), M, K, ap, len(members),
            dt, None if ws is None else ws.data_ptr(), need, _stream())
    check(rc, "metis_linear_fwd_grouped_bf16" if rounded else "metis_linear_fwd_grouped", (M, K, [m[0].rows for m in members]))
    return outs


def _tiled_backward_pays(M: int, N: int, K: int, device_index: int) -> bool:
    """Whether a backward product out[M, N] over a contraction of K goes to the pipelined kernel on tiled expansions made
    for this one call: from about 2e11 flop on, with at least one 256 x 256 tile per compute unit, the faster GEMM more
    than pays for writing the expansions (8192 x 4096 x 14336: input gradient 858 -> 749 us with the weight's
    expansion cached, weight gradient 915 -> 835 us with both operands expanded; 4096 x 1536 x 8960: 134 -> 149 and
    117 -> 141 us, so small products stay on the packed kernel).  Plain products keep their bits; with a low-rank term
    the binary32 sums are taken in another order."""
    return (tiled_weight_copies and M >= 256 and N >= 256 and K % 32 == 0 and 2.0 * M * N * K >= 2e11
            and (M // 256) * (N // 256) >= _device_cus(device_index))


def linear_dgrad(dy: PackedNVFP4, wt: PackedNVFP4, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """grad_input[L, K] from dY packed along N [L, N] and W packed along N (column-blocked) [K, N]."""
    if dy.cols != wt.cols:
        raise ValueError(f"contraction mismatch: {dy.cols} vs {wt.cols}")
    L, N, K = dy.rows, dy.cols, wt.rows
    if dy.mode == wt.mode and _tiled_backward_pays(L, K, N, dy.codes.device.index or 0):
        return linear_fwd(dy, wt, out_dtype=out_dtype, tiled=True)          # out = deq(dy) . deq(wt)^T: the same product
    out = torch.empty(L, K, dtype=out_dtype, device=dy.codes.device)
    dt = DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16
    ws = _gemm_workspace(L, K, N, out.device)
    if ws is not None:
        rc = load().metis_linear_dgrad_ws(dy.codes.data_ptr(), dy.scales.data_ptr(), dy.unit.data_ptr(), wt.codes.data_ptr(),
                                          wt.scales.data_ptr(), wt.unit.data_ptr(), L, N, K, out.data_ptr(), dt,
                                          ws.data_ptr(), ws.numel(), _stream())
        check(rc, "metis_linear_dgrad_ws", (L, N, K))
        return out
    rc = load().metis_linear_dgrad(dy.codes.data_ptr(), dy.scales.data_ptr(), dy.unit.data_ptr(), wt.codes.data_ptr(),
                                   wt.scales.data_ptr(), wt.unit.data_ptr(), L, N, K, out.data_ptr(), dt, _stream())
    check(rc, "metis_linear_dgrad", (L, N, K))
    return out


def linear_wgrad(dyt: PackedNVFP4, xt: PackedNVFP4, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """grad_weight[N, K] from dY and X both packed along tokens: dyt [N, L], xt [K, L]."""
    if dyt.cols != xt.cols:
        raise ValueError(f"contraction mismatch: {dyt.cols} vs {xt.cols}")
    N, L, K = dyt.rows, dyt.cols, xt.rows
    if dyt.mode == xt.mode and _tiled_backward_pays(N, K, L, dyt.codes.device.index or 0):
        return linear_fwd(dyt, xt, out_dtype=out_dtype, tiled=True)
    out = torch.empty(N, K, dtype=out_dtype, device=dyt.codes.device)
    dt = DTYPE_F32 if out_dtype == torch.float32 else DTYPE_BF16
    ws = _gemm_workspace(N, K, L, out.device)
    if ws is not None:
        rc = load().metis_linear_wgrad_ws(dyt.codes.data_ptr(), dyt.scales.data_ptr(), dyt.unit.data_ptr(),
                                          xt.codes.data_ptr(), xt.scales.data_ptr(), xt.unit.data_ptr(), L, N, K,
                                          out.data_ptr(), dt, ws.data_ptr(), ws.numel(), _stream())
        check(rc, "metis_linear_wgrad_ws", (L, N, K))
        return out
    rc = load().metis_linear_wgrad(dyt.codes.data_ptr(), dyt.scales.data_ptr(), dyt.unit.data_ptr(),
                                   xt.codes.data_ptr(), xt.scales.data_ptr(), xt.unit.data_ptr(), L, N, K,
                                   out.data_ptr(), dt, _stream())
    check(rc, "metis_linear_wgrad", (L, N, K))
    return out
