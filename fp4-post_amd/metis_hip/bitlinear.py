"""Metis low-bit linear modules with the reference's interface, computing on HIP kernels.

Mirrors src/Metis/Metis/bitlinear.py: ``LinearLowbitFunction`` (autograd function with class-level
configuration, 18-513), ``LinearLowbit`` (515-595) and ``BitLinear`` (597-940) keep their names,
constructor arguments, attributes, state-dict keys and error behaviour, so model patching code written
for the reference works unchanged.

What differs underneath
  * NVFP4 quantizers emit packed codes + E4M3 scale bytes (ops.PackedNVFP4) and the matmuls run as
    block-scaled MFMA GEMMs on the packed operands; nothing is dequantized to HBM on the hot path.
  * BitLinear.forward evaluates both branches in one kernel:
        y = ((x V^T) * s) U^T + deq(Q(x)) deq(Q(W_res))^T + b        (fp32 accumulate)
    with the rank-r branch on the raw activations in bf16 (as bitlinear_new.py:376-388,473-488 does);
    the reference's current file feeds the quantized activation and a quantized V to that branch
    (bitlinear.py:752, 863-879).
  * Backward re-quantizes dY and X with stochastic rounding along the contraction dimension of each
    GEMM (tokens for wgrad), which a block-scaled GEMM needs; the reference quantizes dY along its last
    dimension only and reuses the forward X^ (bitlinear.py:488-508).
Quantizer classes other than the kernel-backed NVFP4 pair (e.g. Cast2Fp32 or user subclasses) take a
generic path that follows the reference line by line with torch matmuls.
"""
from __future__ import annotations

import math
import weakref
from types import SimpleNamespace

import torch
import torch.nn as nn
import torch.nn.init as init

from . import ops
from .ops import CenteredNVFP4, LowRankNVFP4, PackedNVFP4
from .quant import (Cast2Fp32, Cast2NVFp4e2m1Block, Cast2NVFp4e2m1BlockNOSR, QuantFunc, is_hip_nvfp4, quant_func)

__all__ = ["LinearLowbitFunction", "LinearLowbit", "BitLinear"]


def _pkey(p: torch.Tensor) -> tuple:
    """Cache key of a parameter: its identity and storage as well as its version counter, so that a Parameter that is
    REPLACED (load_state_dict(assign=True), `m.s = nn.Parameter(...)`) is seen although a fresh one starts at the same
    version.  (A write through `.data`, which moves neither, stays invisible, as it does to the reference's own cache.)"""
    return (id(p), p.data_ptr(), p._version)


def _flat2d(x: torch.Tensor) -> torch.Tensor:
    return x.reshape(-1, x.shape[-1])


def _packable(x: torch.Tensor, q) -> bool:
    """Fast path available: kernel-backed quantizer, device tensor, shapes the GEMM accepts (the contraction a
    multiple of 32).  A device tensor that misses it only by its shape or dtype is reported once."""
    if not (is_hip_nvfp4(q) and x.is_cuda):
        return False
    ok = x.shape[-1] % 32 == 0 and x.dtype in (torch.float32, torch.bfloat16)
    if not ok:
        _warn_generic_path(f"a tensor of shape {tuple(x.shape)}, dtype {x.dtype}")
    return ok


_generic_path_warned: set = set()


def _warn_generic_path(what: str) -> None:
    """Said once per distinct situation: an NVFP4 call on a device tensor left the packed kernels for the generic
    path (dequantized tensors and torch matmuls: same formula as the reference, several times slower, and in backward
    quantized along the last dimension instead of the contraction)."""
    if what not in _generic_path_warned:
        _generic_path_warned.add(what)
        import warnings
        warnings.warn(f"metis_hip: {what} does not fit the packed NVFP4 kernels; using the generic path", RuntimeWarning,
                      stacklevel=3)


def _token_sum(flat: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Sum over tokens of a [L, N] gradient with the result in `dtype` (the bias gradient, reference 455): one pass of the
    library's column reduction on the device, torch elsewhere."""
    if flat.is_cuda and flat.dtype in (torch.float32, torch.bfloat16) and dtype in (torch.float32, torch.bfloat16) \
            and flat.shape[1] % 4 == 0 and flat.shape[0] > 0:
        src = flat if (dtype == torch.float32 or flat.dtype == torch.bfloat16) else flat.to(dtype)
        return ops.column_sum(src, out_dtype=dtype)
    return flat.to(dtype).sum(dim=0)


class LinearLowbitFunction(torch.autograd.Function):
    """Low-bit GEMM with quantized activations / weights / gradients (reference 18-513).

    Class attributes are configured by BitLinear.__init__ exactly as in the reference; they are
    process-wide mutable state there too (last constructed layer wins).
    """
    q_forward_input = Cast2NVFp4e2m1BlockNOSR
    q_forward_weight = Cast2NVFp4e2m1BlockNOSR
    q_backward_input = Cast2NVFp4e2m1Block
    q_backward_weight = Cast2NVFp4e2m1Block
    q_backward_outputgrad = Cast2NVFp4e2m1Block

    enable_nv_recipe = False
    hadamard_workspace_mb = 128
    hadamard_tile_size = 16
    hadamard_backend = "auto"

    activation_lowrank_niter = 0
    backward_lowrank_niter = 0
    enable_activation_svd = False
    activation_lowrank_svd = -1
    enable_backward_svd = False
    backward_lowrank_svd = -1
    activation_broadcast_dim = -1
    backward_broadcast_dim = -1

    tp_simulate = False
    tp_parts = 4

    compute_dtype = torch.float32
    # bf16 arithmetic (compute_dtype = bfloat16): forward GEMMs of 256 rows or more follow the reference's all-bf16
    # evaluation rounding for rounding (operands bf16(bf16(e4m3 * unit) * v / 2), residual product and bias add rounded
    # to bf16).  False keeps exact products and one rounding at the end, as every smaller batch does.
    reference_rounding = True
    metis_mode = "mean"
    mean_cache = None
    mean_cache_key = "default"

    # ------------------------------------------------------------------ activation paths
    # ------------------------------------------------------------------ tiled random Hadamard rotation
    _hadamard_cache: dict = {}
    _hadamard_sign_cache: dict = {}

    @staticmethod
    def _get_hadamard(size: int, device, dtype) -> torch.Tensor:
        """Sylvester Hadamard matrix H_size (entries +-1), cached per (size, device, dtype); reference 75-96."""
        F = LinearLowbitFunction
        key = (int(size), device, dtype)
        if key not in F._hadamard_cache:
            if size <= 0 or size & (size - 1):
                raise ValueError(f"Hadamard block size must be a power of two, got {size}")
            h = torch.ones((1, 1), device=device, dtype=dtype)
            while h.shape[0] < size:
                h = torch.cat((torch.cat((h, h), dim=1), torch.cat((h, -h), dim=1)), dim=0)
            F._hadamard_cache[key] = h
        return F._hadamard_cache[key]

    @staticmethod
    def _get_hadamard_sign(size: int, device, dtype) -> torch.Tensor:
        """The one +-1 vector shared by every tile of a given size: CPU generator seeded with
        1729 + size, so it is the same vector the reference draws (reference 98-111)."""
        F = LinearLowbitFunction
        key = (int(size), device, dtype)
        if key not in F._hadamard_sign_cache:
            gen = torch.Generator(device="cpu")
            gen.manual_seed(1729 + size)
            bits = torch.randint(0, 2, (size,), generator=gen, dtype=torch.int8)
            F._hadamard_sign_cache[key] = (bits * 2 - 1).to(device=device, dtype=dtype)
        return F._hadamard_sign_cache[key]

    @staticmethod
    def _hadamard_mask() -> int:
        """The shared sign vector of the 16-wide rotation as a bit mask for the kernels: bit j set <=> sign[j] = -1."""
        signs = LinearLowbitFunction._get_hadamard_sign(16, torch.device("cpu"), torch.float32)
        return sum(1 << j for j in range(16) if float(signs[j]) < 0)

    @staticmethod
    def _nv_on_kernels() -> bool:
        """NV recipe with the tile the scale blocks have: rotation, quantizer and GEMM operands stay on the library's
        kernels (a rotated tile is one block of 16).  hadamard_backend "torch_gemm" asks for the reference's portable
        formula instead: rotation as a small GEMM, dequantized tensors, torch matmuls."""
        F = LinearLowbitFunction
        return F.enable_nv_recipe and int(F.hadamard_tile_size) == 16 and F.hadamard_backend == "auto"

    @staticmethod
    def _apply_hadamard_blocks(value: torch.Tensor, inverse: bool = False) -> torch.Tensor:
        """Rotate every tile of `hadamard_tile_size` consecutive elements of the last dimension:
        forward (x * S) H, inverse (y H) / d * S (reference 125-211).  All tiles go through one
        small GEMM per row chunk, in binary32 for 16-bit inputs; chunks are sized so that the
        binary32 workspace stays within `hadamard_workspace_mb`."""
        F = LinearLowbitFunction
        dim = value.shape[-1]
        if dim <= 1 or value.numel() == 0:
            return value
        tile = int(F.hadamard_tile_size)
        if tile <= 0 or tile & (tile - 1):
            raise ValueError(f"Hadamard tile size must be a positive power of two, got {tile}")
        if dim % tile:
            raise ValueError(f"RHT tile size {tile} must divide hidden dimension {dim}; "
                             "set --metis_hadamard_tile_size to a compatible power of two")
        if F.hadamard_backend not in {"auto", "dao_cuda", "torch_gemm"}:
            raise ValueError(f"Unsupported Hadamard backend: {F.hadamard_backend}")
        if F.hadamard_backend == "dao_cuda":
            raise RuntimeError("Hadamard backend dao_cuda was requested but fast_hadamard_transform is unavailable "
                               "in this build; use 'auto' or 'torch_gemm'")
        if tile == 16 and value.is_cuda and value.dtype in (torch.float32, torch.bfloat16) and F.hadamard_backend == "auto":
            # in-register butterflies, one pass over the tensor; "torch_gemm" keeps the reference's fallback formula
            return ops.hadamard16(value, F._hadamard_mask(), inverse=inverse)
        work_dtype = torch.float32 if value.dtype in (torch.float16, torch.bfloat16) else value.dtype
        h = F._get_hadamard(tile, value.device, work_dtype)
        signs = F._get_hadamard_sign(tile, value.device, work_dtype)
        tiles = value.reshape(-1, tile)
        out = torch.empty_like(tiles)
        budget = max(1, int(F.hadamard_workspace_mb)) * 1024 * 1024
        chunk = max(1, budget // (8 * tile * torch.empty((), dtype=work_dtype).element_size()))
        for r0 in range(0, tiles.shape[0], chunk):
            work = tiles[r0:r0 + chunk].to(work_dtype)
            if inverse:
                rotated = torch.mm(work, h).mul_(1.0 / tile).mul_(signs)
            else:
                rotated = torch.mm(work * signs, h)
            out[r0:r0 + chunk].copy_(rotated)
        return out.reshape(value.shape)

    @staticmethod
    def svd_quant(input_, quant_func, rank=60, niter=0, broadcast_dim=-1, tp_simulate=False, tp_parts=4,
                  metis_mode="mean", mean_cache=None, cache_key="default"):
        """Low-rank (or mean) part kept in high precision + quantized residual (reference 213-369).

        "mean": the column mean over tokens stays in high precision, the centred residual goes through
        the quantizer's fused QDQ and the mean is added back; single-token decode calls use a weighted
        running mean per cache key (311-336).  "svd": a randomized rank-`rank` SVD of the (optionally
        broadcast-sliced) input, U and V through the three-call QDQ, S untouched, residual through the
        fused QDQ (243-309).  With tp_simulate the last dimension is cut into tp_parts chunks that are
        treated independently in "svd" style and concatenated (338-360).
        """
        F = LinearLowbitFunction

        def lowrank_single(chunk):
            if broadcast_dim < 0 and F._svd_mode_on_kernels(chunk, quant_func, rank):
                return F._lowrank_decompose(chunk, quant_func, rank, niter, dense=True).dense.view(chunk.shape)
            picked = broadcast_dim >= 0
            rep = chunk.select(broadcast_dim, 0) if picked else chunk
            shape = rep.shape
            rep2 = rep.reshape(-1, shape[-1]) if len(shape) == 3 else rep
            flat = chunk.reshape(-1, shape[-1]) if len(shape) == 3 else chunk
            dtype = rep2.dtype
            with torch.amp.autocast(rep2.device.type, enabled=False):
                ug, sg, vg = torch.svd_lowrank(rep2.to(torch.float32), q=rank, niter=niter)
            ug, sg, vg = ug.to(dtype), sg.to(dtype), vg.to(dtype).T
            us, vs = quant_func.get_scalar(ug), quant_func.get_scalar(vg)
            ug = quant_func.rquant(quant_func.quant(ug, us), us)
            vg = quant_func.rquant(quant_func.quant(vg, vs), vs)
            ker = ug @ torch.diag(sg) @ vg
            if picked:
                ker = ker.unsqueeze(broadcast_dim)
            out = ker + quant_func.quantize_dequantize(flat - ker)
            return out.view(shape[0], shape[1], -1) if len(shape) == 3 else out

        def mean_single(x):
            shape = x.shape
            flat = _flat2d(x)
            seq_len = shape[1] if len(shape) == 3 else shape[0]
            if seq_len == 1 and mean_cache is not None and cache_key in mean_cache:
                cached_mean, cached_count = mean_cache[cache_key]
                new_count = cached_count + flat.shape[0]
                this_mean = flat.mean(dim=0, keepdim=True)
                me = (cached_mean * cached_count + this_mean * flat.shape[0]) / new_count
                mean_cache[cache_key] = (me.detach(), new_count)
            else:
                me = flat.mean(dim=0, keepdim=True)
                if mean_cache is not None:
                    mean_cache[cache_key] = (me.detach(), flat.shape[0])
            out = me + quant_func.quantize_dequantize(flat - me)
            return out.view(shape) if len(shape) == 3 else out

        if tp_simulate:
            width, parts = input_.shape[-1], max(1, int(tp_parts))
            edges = [(width * p) // parts for p in range(parts + 1)]
            return torch.cat([lowrank_single(input_[..., a:b]) for a, b in zip(edges, edges[1:]) if b > a], dim=-1)
        if metis_mode == "svd":
            return lowrank_single(input_)
        if metis_mode == "mean":
            return mean_single(input_)
        raise ValueError(f"Unsupported metis_mode: {metis_mode}")

    @staticmethod
    def quantize_input(input_: torch.Tensor, mean_cache: dict = None, cache_key: str = "default") -> torch.Tensor:
        """Dequantized activation, as the reference returns it (371-393)."""
        F = LinearLowbitFunction
        input_ = input_.to(F.compute_dtype)
        if F.enable_activation_svd:
            return F.svd_quant(input_, quant_func=F.q_forward_input, rank=F.activation_lowrank_svd,
                               niter=F.activation_lowrank_niter, broadcast_dim=F.activation_broadcast_dim,
                               tp_simulate=F.tp_simulate, tp_parts=F.tp_parts, metis_mode=F.metis_mode,
                               mean_cache=mean_cache, cache_key=cache_key)
        return F.q_forward_input.quantize_dequantize(input_)

    @staticmethod
    def _token_mean(input_: torch.Tensor, mean_cache=None, cache_key="default") -> torch.Tensor:
        """Column mean over tokens in the compute dtype ([C]); single-token decode calls update a weighted
        running mean per cache key instead (reference 311-329).  The cache holds ([1, C] mean, count) as the
        reference's does."""
        return LinearLowbitFunction._token_mean2(input_, mean_cache, cache_key)[0]

    @staticmethod
    def _token_mean2(input_: torch.Tensor, mean_cache=None, cache_key="default"):
        """(mean in the compute dtype, the same values as float32 or None).  On the device the reduction and the
        running update are one reduction kernel and one small kernel."""
        cd = LinearLowbitFunction.compute_dtype
        flat = _flat2d(input_)
        rows = flat.shape[0]
        seq_len = input_.shape[1] if input_.dim() == 3 else input_.shape[0]
        running = seq_len == 1 and mean_cache is not None and cache_key in mean_cache
        cached_mean, cached_count = mean_cache[cache_key] if running else (None, 0)
        if flat.is_cuda and flat.dtype in (torch.float32, torch.bfloat16) and flat.shape[1] % 4 == 0 and \
                cd in (torch.float32, torch.bfloat16) and cached_count + rows <= 2 ** 24:
            # one pass over the tensor; a bf16 tensor is read as it is in either arithmetic
            src = flat if (cd == torch.float32 or flat.dtype == torch.bfloat16) else flat.to(cd)
            me, me32 = ops.column_mean_running(src, cached_mean, cached_count, out_dtype=cd)
            if mean_cache is not None:
                mean_cache[cache_key] = (me.detach().unsqueeze(0), cached_count + rows)
            return me, me32
        if cd == torch.float32:
            this_mean = flat.mean(dim=0, keepdim=True, dtype=torch.float32)
        else:
            this_mean = flat.to(cd).mean(dim=0, keepdim=True)
        if running:
            new_count = cached_count + rows
            me = (cached_mean * cached_count + this_mean * rows) / new_count
            mean_cache[cache_key] = (me.detach(), new_count)
        else:
            me = this_mean
            if mean_cache is not None:
                mean_cache[cache_key] = (me.detach(), rows)
        return me.reshape(-1), None

    @staticmethod
    def _mean_mode_packable() -> bool:
        F = LinearLowbitFunction
        return F.metis_mode == "mean" and not F.tp_simulate and not F.enable_nv_recipe

    @staticmethod
    def _svd_mode_on_kernels(x: torch.Tensor, q, rank: int) -> bool:
        """The fused kernel of the "svd" mode takes this tensor: round-to-nearest NVFP4 on a device tensor in binary32 or
        bf16 arithmetic, rank and width multiples of the block."""
        return (q is Cast2NVFp4e2m1BlockNOSR and x.is_cuda and x.dtype in (torch.float32, torch.bfloat16) and x.numel() > 0
                and rank > 0 and rank % 16 == 0 and x.shape[-1] % 16 == 0 and x.dim() in (2, 3))

    @staticmethod
    def _lowrank_decompose(x: torch.Tensor, q, rank: int, niter: int, dense: bool, arith: torch.dtype | None = None) -> LowRankNVFP4:
        """Reference 262-303 with the factors from torch.svd_lowrank (randomized, as there): U and V through the
        quantizer (V stays packed: its three-call QDQ is the packed tensor's dequantization, bit for bit), then ONE
        fused kernel forms ker = U diag(s) V in registers, encodes x - ker and, with dense, writes ker + QDQ(x - ker).
        arith: the arithmetic's type when it is not x's own (a bf16 tensor under binary32 arithmetic is widened in the
        kernel's registers, not copied)."""
        x2 = _flat2d(x)
        dt = x2.dtype if arith is None else arith
        if dt != torch.float32:
            x2 = x2.to(torch.bfloat16)
        with torch.amp.autocast(x2.device.type, enabled=False):
            ug, sg, vg = torch.svd_lowrank(x2.to(torch.float32), q=rank, niter=niter)
        ug, sg, vt = ug.to(dt), sg.to(dt), vg.to(dt).T.contiguous()
        s_u = q.get_scalar(ug)
        us = q.rquant(q.quant(ug, s_u), s_u) * sg              # == ugq @ diag(sg): one nonzero term per sum
        p_vt = q.pack(vt)
        mode = ops.MODE_P32 if dt == torch.float32 else ops.MODE_PB16
        residual, out = ops.quantize_lowrank_residual(x2, us, ops.dequantize(p_vt, dt), mode, dense=dense)
        return LowRankNVFP4(residual, us, p_vt, out)

    @staticmethod
    def _scales_formed_by_consumer(rows: int, weights_cached: bool) -> bool:
        """Whether the GEMM that will read a packed activation forms its scale bytes itself, so that the quantizer may
        stop after its first launch: the tiled expansion does (it is chosen from 256 rows on when the weight side's
        expansion is kept, i.e. for cached weights with ops.tiled_weight_copies), and so does every consumer under bf16
        arithmetic with the reference's roundings.  The packed-operand kernels read the bytes: deferring there only
        moves the second launch."""
        F = LinearLowbitFunction
        return F._bf16_rounding() or (rows >= 256 and weights_cached and ops.tiled_weight_copies)

    @staticmethod
    def _prepare_input(input_: torch.Tensor, mean_cache=None, cache_key="default", weights_cached: bool = True,
                       keep_dense: bool | None = None):
        """Packed activation when a kernel path applies (direct: PackedNVFP4; mean mode: CenteredNVFP4; svd mode:
        LowRankNVFP4), else the dequantized tensor.  weights_cached: the layers that will read it keep their packed
        weights across calls.  keep_dense (svd mode): a backward pass will follow; default: autograd is recording."""
        F = LinearLowbitFunction
        if (not F.enable_nv_recipe or F._nv_on_kernels()) and _packable(input_, F.q_forward_input):
            if not F.enable_activation_svd:
                # the kernels read bf16 values and take the arithmetic as a mode: no upcast copy of a bf16 tensor
                x2 = _flat2d(input_)
                more = {"deferred": True} if F._scales_formed_by_consumer(x2.shape[0], weights_cached) else {}
                return F.q_forward_input.pack(x2, arith=F.compute_dtype, **more)
            if (F.metis_mode == "svd" and not F.tp_simulate and not F.enable_nv_recipe and F.activation_broadcast_dim < 0
                    and F._svd_mode_on_kernels(input_, F.q_forward_input, F.activation_lowrank_svd)
                    and F.compute_dtype in (torch.float32, torch.bfloat16)):
                # ker + QDQ(x - ker) (reference 243-309): packed residual + the factors; the dense tensor as well when
                # a backward pass will want it (the factors are randomized: it cannot be derived again)
                return F._lowrank_decompose(input_, F.q_forward_input, F.activation_lowrank_svd, F.activation_lowrank_niter,
                                            dense=torch.is_grad_enabled() if keep_dense is None else keep_dense,
                                            arith=F.compute_dtype)
            if F._mean_mode_packable():
                # mean + QDQ(x - mean) (reference 311-336) without materialising either: the subtraction happens
                # inside the quantizer and the mean's contribution to a matmul is a rank-one term
                me, me32 = F._token_mean2(input_, mean_cache=mean_cache, cache_key=cache_key)
                more = {"deferred": True} if (F._bf16_rounding() and me.dtype == torch.bfloat16) else {}
                return CenteredNVFP4(F.q_forward_input.pack(_flat2d(input_), arith=F.compute_dtype, center=me, **more), me, me32)
        return F.quantize_input(input_, mean_cache=mean_cache, cache_key=cache_key)

    @staticmethod
    def _packed_grads(dy2, x2, pw_col, center_x, gx_dtype, gw_dtype, gx_lowrank=None):
        """(grad_input [L, K], grad_weight [N, K]) on packed operands.  dgrad contracts over N, wgrad over tokens.

        Direct mode: dY^ = SR-Q(dY).  Mean mode (enable_backward_svd): dY^ = 1 me_dy^T + SR-Q(dY - me_dy)
        (reference 462-474 with 311-336).  The saved activation enters the weight gradient as
        1 center_x^T + SR-Q(X - center_x) along tokens (center_x None: plain SR-Q(X)).  The means contribute
        rank-one terms:
            gX = R_dy W^ + 1 (W^^T me_dy)^T
            gW = R_dy^T R_x + (sum_l R_dy) center_x^T + me_dy (sum_l R_x + L center_x)^T
        gx_lowrank = (t [L, r], u [K, r]) adds t u^T to grad_input inside the same launch (the rank-r branch's share).
        """
        F = LinearLowbitFunction
        cd = F.compute_dtype
        qg, qi = F.q_backward_outputgrad, F.q_backward_input
        me_dy = F._token_mean(dy2) if F.enable_backward_svd else None
        # The weight gradient contracts over tokens in steps of 32.  A ragged token count is padded, not sent down
        # another code path: rows equal to the centre (zero rows in direct mode) have a zero residual, so they change
        # no block maximum, no tensor unit and no sum; the padded rows of grad_input are dropped at the end.
        L = dy2.shape[0]
        pad = (-L) % 32
        if pad:
            def padded(v, centre):
                if centre is None:
                    return torch.cat((v, v.new_zeros(pad, v.shape[1])), dim=0)
                if v.dtype != centre.dtype:
                    v = v.to(centre.dtype)                     # the padding rows must equal the centre exactly
                return torch.cat((v, centre.reshape(1, -1).expand(pad, -1)), dim=0)
            dy2, x2 = padded(dy2, me_dy), padded(x2, center_x)
            if gx_lowrank is not None:
                gx_lowrank = (padded(gx_lowrank[0], None), gx_lowrank[1])
        if me_dy is None and hasattr(qg, "pack_both"):
            p_dy, p_dyt = qg.pack_both(dy2, arith=cd)          # one pass over dY for both products
        else:
            p_dy, p_dyt = qg.pack(dy2, arith=cd, center=me_dy), None
        if me_dy is None and gx_lowrank is None:
            gx = ops.linear_dgrad(p_dy, pw_col, out_dtype=gx_dtype)
        else:
            lt, lu = gx_lowrank if gx_lowrank is not None else (None, None)
            gx = ops.linear_fwd(p_dy, pw_col, t=lt, u=lu, bias=None if me_dy is None else ops.matvec(pw_col, me_dy),
                                out_dtype=gx_dtype)
        if pad:
            gx = gx[:L]
        if p_dyt is None:
            p_dyt = qg.pack(dy2, col=True, arith=cd, center=me_dy)
        p_xt = qi.pack(x2, col=True, arith=cd, center=center_x)
        if me_dy is None and center_x is None:
            # autograd rounds the gradient to the parameter's dtype anyway: let the GEMM epilogue do that rounding
            return gx, ops.linear_wgrad(p_dyt, p_xt, out_dtype=gw_dtype)
        # the rank-one terms ride in the GEMM's low-rank operands (three bf16 terms per factor: binary32 precision)
        first = second = None
        if center_x is not None:
            first = (ops.matvec(p_dyt), center_x)
        if me_dy is not None:
            tail = ops.matvec(p_xt) if center_x is None else ops.matvec(p_xt, z=center_x, beta=float(L))
            second = (me_dy, tail)
        t, u = ops.rank_one_operands(p_dyt.rows, p_xt.rows, first or second, second if first else None)
        return gx, ops.linear_fwd(p_dyt, p_xt, t=t, u=u, out_dtype=gw_dtype)

    @staticmethod
    def _packed_grads_nv(dy2, x2, pw, gx_dtype, gw_dtype, gx_lowrank=None):
        """(grad_input, grad_weight) of the NV recipe (reference 443-513 with 395-405, 495-501) without leaving the
        packed kernels.  The reference rotates dY and the saved (already quantized) input tile by tile along their
        last dimension, quantizes, dequantizes and rotates back, and multiplies the results:
            dY~ = rot^-1(QDQ(rot(dY))),  X~ = rot^-1(QDQ(rot(QDQ(x)))),  gW = dY~^T X~,  gX = dY~ W~
        with W~ the forward weight (577-585).  Here rot + quantizer is one kernel, and every GEMM operand is the tiled
        16-bit expansion of a packed tensor with the rotation back applied block by block on the way: dY~ [L, N] and
        W~^T [K, N] for the input gradient (contraction over N), dY~^T [N, L] and X~^T [K, L] for the weight gradient
        (contraction over tokens; the expansion transposes).  Quantization blocks run along the last dimension, as the
        reference's do.  gx_lowrank = (t [L, r], u [K, r]) adds t u^T to grad_input inside the same launch."""
        F = LinearLowbitFunction
        cd = F.compute_dtype
        mask = pw.rht
        gmode = ops.MODE_PB16 if (cd != torch.float32 and F.reference_rounding and pw.mode == ops.MODE_PB16) else ops.MODE_P32
        L, N = dy2.shape
        K = x2.shape[1]
        pad = (-L) % 32                                        # the token contraction runs in steps of 32: zero rows add nothing
        lt, lu = gx_lowrank if gx_lowrank is not None else (None, None)
        if pad:
            dy2 = torch.cat((dy2, dy2.new_zeros(pad, N)), dim=0)
            x2 = torch.cat((x2, x2.new_zeros(pad, K)), dim=0)
            if lt is not None:
                lt = torch.cat((lt, lt.new_zeros(pad, lt.shape[1])), dim=0)
        p_dy = F.q_backward_outputgrad.pack(dy2, arith=cd, rht=mask)
        xq = F.q_forward_input.pack(x2, arith=cd).dequantize(torch.float32 if cd == torch.float32 else torch.bfloat16)
        p_x = F.q_backward_input.pack(xq, arith=cd, rht=mask)
        a_dy = ops.expand_tiled(p_dy, cache=False, mode=gmode)
        b_wt = ops.expand_tiled_transposed(pw, cache=pw.persistent, mode=gmode)
        gx = ops.gemm_tiled(a_dy, p_dy.unit, b_wt, pw.unit, L + pad, K, N, mode=gmode, t=lt, u=lu, out_dtype=gx_dtype)
        a_dyt = ops.expand_tiled_transposed(p_dy, mode=gmode)
        b_xt = ops.expand_tiled_transposed(p_x, mode=gmode)
        gw = ops.gemm_tiled(a_dyt, p_dy.unit, b_xt, p_x.unit, N, K, L + pad, mode=gmode, out_dtype=gw_dtype)
        return (gx[:L] if pad else gx), gw

    @staticmethod
    def _check_backward_config() -> None:
        F = LinearLowbitFunction
        if F.enable_backward_svd and F.backward_lowrank_svd <= 0:
            # the reference takes a full SVD of the output gradient here (bitlinear.py:476-486); neither path of this
            # library implements that branch, and the low-rank / mean-residual QDQ it would silently get instead is
            # another method
            raise NotImplementedError("enable_backward_svd with backward_lowrank_svd <= 0 (the reference's full-SVD branch, "
                                      "bitlinear.py:476-486) is not implemented; use a positive rank")

    @staticmethod
    def _packed_backward_applies(L: int, N: int, grad_output: torch.Tensor) -> bool:
        """Backward on the packed kernels.  Any token count L qualifies (ragged counts are padded inside
        _packed_grads); the output width N is the contraction of the input gradient and has to be a multiple of 32.
        A device NVFP4 configuration that does not qualify takes the generic path and says so once."""
        F = LinearLowbitFunction
        if not (is_hip_nvfp4(F.q_backward_outputgrad) and is_hip_nvfp4(F.q_backward_input)):
            return False
        ok = N % 32 == 0 and L > 0 and grad_output.dtype in (torch.float32, torch.bfloat16)
        if ok and F.enable_backward_svd:
            ok = F.backward_lowrank_svd > 0 and F._mean_mode_packable()
        if ok and F.enable_nv_recipe:
            ok = F._nv_on_kernels()
        if not ok and grad_output.is_cuda:
            _warn_generic_path(f"backward with {L} tokens, {N} output features, dtype {grad_output.dtype}, "
                               f"metis_mode={F.metis_mode!r}, nv_recipe={F.enable_nv_recipe}")
        return ok

    @staticmethod
    def _quantize_wgrad_operand(value: torch.Tensor, quantizer) -> torch.Tensor:
        """Three-call QDQ of one backward operand, between a tiled random Hadamard rotation and its
        inverse under the NV recipe (reference 395-405)."""
        F = LinearLowbitFunction
        if F.enable_nv_recipe:
            value = F._apply_hadamard_blocks(value, inverse=False)
        scalar = quantizer.get_scalar(value)
        value = quantizer.quant(value, scalar)
        value = quantizer.rquant(value, scalar)
        if F.enable_nv_recipe:
            value = F._apply_hadamard_blocks(value, inverse=True)
        return value

    @staticmethod
    def _bf16_rounding() -> bool:
        """bf16 arithmetic with the reference's roundings: every consumer of a packed activation (tiled expansion, ready
        decode operands) forms the scale bytes itself, so the quantizer may always defer them."""
        F = LinearLowbitFunction
        return F.reference_rounding and F.compute_dtype != torch.float32

    @staticmethod
    def _mean_in_operand(px, pw) -> bool:
        """Mean mode in bf16 arithmetic with reference_rounding: the GEMM's activation operand is the reference's own
        bf16 tensor me + QDQ(x - me) (reference 330-333), so the forward follows its all-bf16 evaluation; otherwise the
        mean's share is a separate binary32 term next to exact products of the packed residual."""
        F = LinearLowbitFunction
        return (F.reference_rounding and F.compute_dtype != torch.float32 and px.residual.mode == ops.MODE_PB16
                and pw.mode == ops.MODE_PB16 and pw.rht is None and px.mean.dtype == torch.bfloat16 and px.cols % 32 == 0)

    # ------------------------------------------------------------------ autograd
    @staticmethod
    def forward(ctx, input_, weight, bias, quantized_weight, quantized_input):
        F = LinearLowbitFunction
        if quantized_input is None:
            quantized_input = F._prepare_input(input_, mean_cache=F.mean_cache, cache_key=F.mean_cache_key,
                                               weights_cached=bool(getattr(quantized_weight, "persistent", False)),
                                               keep_dense=any(ctx.needs_input_grad[:3]))
        lead = input_.shape[:-1]
        ctx.lead = lead
        ctx.has_bias = bias is not None
        ctx.packed = (isinstance(quantized_input, (PackedNVFP4, CenteredNVFP4, LowRankNVFP4))
                      and isinstance(quantized_weight, PackedNVFP4))
        ctx.lowrank = False
        if ctx.packed and isinstance(quantized_input, LowRankNVFP4):
            # "svd" mode: (us V^ + R^) W^^T = R^ W^^T + us (V^ W^^T) -- both products on packed operands, the rank-r
            # correction a library product in binary32.  The backward pass multiplies with the reference's dense
            # activation (its factors are randomized and cannot be derived again), kept only when autograd will ask.
            ctx.pw = quantized_weight
            ctx.weight_ref = weight
            ctx.center = None
            ctx.lowrank = True
            saved = quantized_input.dense if quantized_input.dense is not None else input_.new_empty(0)
            ctx.save_for_backward(saved, bias if bias is not None else input_.new_empty(0))
            vw = ops.linear_fwd(quantized_input.vt, quantized_weight, out_dtype=torch.float32)            # [r, N]
            out = ops.linear_fwd(quantized_input.residual, quantized_weight, bias=bias, out_dtype=torch.float32)
            out.addmm_(quantized_input.us.float(), vw)
            return out.reshape(*lead, quantized_weight.rows).to(F.compute_dtype)
        if ctx.packed:
            ctx.pw = quantized_weight
            ctx.weight_ref = weight
            ctx.save_for_backward(input_, bias if bias is not None else input_.new_empty(0))
            ctx.center = None
            out_dtype = torch.float32 if F.compute_dtype == torch.float32 else torch.bfloat16
            if isinstance(quantized_input, CenteredNVFP4) and F._mean_in_operand(quantized_input, quantized_weight):
                ctx.center = quantized_input.mean
                out = ops.linear_fwd_grouped(quantized_input.residual, [(quantized_weight, None, None, bias)], out_dtype=out_dtype,
                                             center=quantized_input.mean, reference_rounding=True)[0]
                return out.reshape(*lead, quantized_weight.rows).to(F.compute_dtype)
            if isinstance(quantized_input, CenteredNVFP4):
                # (1 me^T + R) W^^T = R W^^T + 1 (W^ me)^T: the mean's term rides in a binary32 bias
                ctx.center = quantized_input.mean
                w_mean = ops.matvec(quantized_weight, quantized_input.mean)
                bias = w_mean if bias is None else w_mean + bias.float()
                quantized_input = quantized_input.residual
            out = ops.linear_fwd(quantized_input, quantized_weight, bias=bias, out_dtype=out_dtype,
                                 reference_rounding=F.reference_rounding and ctx.center is None)
            return out.reshape(*lead, quantized_weight.rows).to(F.compute_dtype)
        if isinstance(quantized_input, (PackedNVFP4, CenteredNVFP4, LowRankNVFP4)):
            quantized_input = quantized_input.dequantize(F.compute_dtype).reshape(input_.shape)
        if isinstance(quantized_weight, PackedNVFP4):
            quantized_weight = quantized_weight.dequantize(F.compute_dtype)
        ctx.save_for_backward(quantized_input, quantized_weight, bias if bias is not None else input_.new_empty(0))
        output = torch.matmul(quantized_input, quantized_weight.T)
        if bias is not None:
            output = output + bias
        return output

    @staticmethod
    def backward(ctx, grad_output):
        F = LinearLowbitFunction
        F._check_backward_config()
        grad_bias = None
        if ctx.has_bias:
            grad_bias = _token_sum(_flat2d(grad_output), F.compute_dtype).to(torch.float32)
        if ctx.packed:
            input_, _ = ctx.saved_tensors
            L, N = _flat2d(grad_output).shape
            if not ctx.lowrank and F._packed_backward_applies(L, N, grad_output):
                # dgrad: contraction over N; wgrad: contraction over tokens.  Operands are packed straight from the
                # tensors autograd hands over, in compute_dtype arithmetic (no upcast copies of bf16 tensors).
                cd = F.compute_dtype
                # binary32 arithmetic quantizes the tensors as they are (binary32 gradients need not be bf16 values);
                # bf16 arithmetic casts to the compute dtype first, as the reference does (453): one pass per tensor,
                # shared by its row and column packing
                dy2, x2 = _flat2d(grad_output), _flat2d(input_)
                if cd != torch.float32:
                    dy2, x2 = dy2.to(torch.bfloat16), x2.to(torch.bfloat16)
                gx_dtype = input_.dtype if input_.dtype in (torch.float32, torch.bfloat16) else torch.float32
                gw_dtype = torch.bfloat16 if ctx.weight_ref.dtype == torch.bfloat16 else torch.float32
                if ctx.pw.rht is not None:
                    gx, gw = F._packed_grads_nv(dy2, x2, ctx.pw, gx_dtype, gw_dtype)
                    return gx.reshape(*ctx.lead, gx.shape[-1]), gw, grad_bias, None, None
                pw_col = ctx.pw.transposed                    # lives as long as the (possibly cached) packed weight
                if pw_col is None:
                    pw_col = ctx.pw.transposed = F.q_forward_weight.pack(ctx.weight_ref, col=True, arith=cd)
                gx, gw = F._packed_grads(dy2, x2, pw_col, ctx.center, gx_dtype, gw_dtype)
                return gx.reshape(*ctx.lead, gx.shape[-1]), gw, grad_bias, None, None
            grad_output = grad_output.to(F.compute_dtype)
            dy2 = _flat2d(grad_output)
            x2 = _flat2d(input_.to(F.compute_dtype))
            if ctx.lowrank:
                if x2.numel() == 0:
                    raise RuntimeError("the svd-mode activation was prepared without autograd (no dense tensor kept) but a "
                                       "backward pass asks for it")
                xq = x2                                          # the reference's saved activation ker + QDQ(x - ker) itself
            elif ctx.center is not None:
                xq = ctx.center.to(F.compute_dtype) + F.q_forward_input.quantize_dequantize(x2 - ctx.center.to(F.compute_dtype))
            else:
                xq = F.q_forward_input.quantize_dequantize(x2)
            wq = ctx.pw.dequantize(F.compute_dtype)
        else:
            grad_output = grad_output.to(F.compute_dtype)
            dy2 = _flat2d(grad_output)
            xq, wq, _ = ctx.saved_tensors
            xq = _flat2d(xq)
        if F.enable_backward_svd:
            dyq = F.svd_quant(grad_output, quant_func=F.q_backward_outputgrad, rank=F.backward_lowrank_svd,
                              niter=F.backward_lowrank_niter, broadcast_dim=F.backward_broadcast_dim,
                              tp_simulate=F.tp_simulate, tp_parts=F.tp_parts, metis_mode=F.metis_mode)
            dyq = _flat2d(dyq)
        else:
            dyq = _flat2d(F._quantize_wgrad_operand(dy2, F.q_backward_outputgrad))
        if F.enable_nv_recipe:                                             # reference 495-501: only the two wgrad operands
            xq = _flat2d(F._quantize_wgrad_operand(xq, F.q_backward_input))
        grad_weight = torch.matmul(dyq.T, xq).to(torch.float32)            # reference 502-510
        grad_input = torch.matmul(dyq, wq).reshape(*ctx.lead, wq.shape[-1])  # reference 507-508
        return grad_input, grad_weight, grad_bias, None, None


class LinearLowbit(nn.Module):
    """nn.Linear replacement whose matmul runs on quantized operands (reference 515-595)."""

    def __init__(self, in_features: int, out_features: int, bias=True, args=None, device=None,
                 storage_dtype=torch.float32, compute_dtype=torch.float32) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.storage_dtype = storage_dtype
        self.compute_dtype = compute_dtype
        self.cache_quantized_weight = getattr(args, "cache_quantized_weight", False)
        self._quantized_weight_cache = None
        dev = getattr(args, "device", None) if device is None else device
        self.weight = nn.Parameter(torch.empty((out_features, in_features), dtype=storage_dtype, device=dev))
        if bias:
            self.bias = nn.Parameter(torch.empty((out_features,), dtype=storage_dtype, device=dev))
        else:
            self.bias = None
        self.reset_parameters()

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            init.uniform_(self.bias, -bound, bound)

    def forward(self, input, quantized_input=None):
        F = LinearLowbitFunction
        bias_compute = self.bias.to(self.compute_dtype) if self.bias is not None else None
        if quantized_input is None and F.enable_activation_svd and F.metis_mode == "svd":
            # decomposed here, where autograd's recording state is visible (inside the Function it never is): the dense
            # activation is written only when a backward pass can follow
            quantized_input = F._prepare_input(input, mean_cache=F.mean_cache, cache_key=F.mean_cache_key,
                                               weights_cached=self.cache_quantized_weight)
        if (not F.enable_nv_recipe or F._nv_on_kernels()) and _packable(self.weight, F.q_forward_weight) and self.weight.shape[0] % 4 == 0:
            # kernel path: packed straight from the stored parameter in compute_dtype arithmetic, so a cache hit
            # costs no pass over the weight at all
            quantized_weight = self._get_quantized_weight(self.weight, arith=self.compute_dtype)
            return F.apply(input, self.weight, bias_compute, quantized_weight, quantized_input)
        weight_compute = self.weight.to(self.compute_dtype)
        quantized_weight = self._get_quantized_weight(weight_compute)
        return F.apply(input, weight_compute, bias_compute, quantized_weight, quantized_input)

    @torch.no_grad()
    def _get_quantized_weight(self, weight_compute, arith=None):
        """Quantized weight, cached on Parameter._version when enabled (reference 563-589).  Returns a
        PackedNVFP4 when the kernel path applies, otherwise the dequantized tensor."""
        F = LinearLowbitFunction
        key = (_pkey(self.weight), weight_compute.device, arith or weight_compute.dtype, F.q_forward_weight, F.enable_nv_recipe)
        if self.cache_quantized_weight and self._quantized_weight_cache is not None:
            cached_key, cached = self._quantized_weight_cache
            if cached_key == key:
                return cached
        if F._nv_on_kernels() and arith is not None and _packable(weight_compute, F.q_forward_weight) and weight_compute.shape[0] % 4 == 0:
            # reference 577-585 on the kernels: the packed tensor holds the ROTATED weight's codes, rotated in the
            # quantizer's registers; whoever reads it (tiled GEMM operand, dequantize) rotates back
            q = F.q_forward_weight.pack(weight_compute, arith=arith, rht=F._hadamard_mask())
        elif F.enable_nv_recipe:                                           # reference 577-585
            q = F._apply_hadamard_blocks(weight_compute, inverse=False)
            q = F._apply_hadamard_blocks(F.q_forward_weight.quantize_dequantize(q), inverse=True)
        elif _packable(weight_compute, F.q_forward_weight) and weight_compute.shape[0] % 4 == 0:
            q = F.q_forward_weight.pack(weight_compute, arith=arith)
        else:
            q = F.q_forward_weight.quantize_dequantize(weight_compute)
        if self.cache_quantized_weight:
            if isinstance(q, PackedNVFP4):
                q.persistent = True                  # reused until the parameter changes: derived layouts may be kept on it
            self._quantized_weight_cache = (key, q)
        return q

    def _apply(self, fn, recurse=True):
        self._quantized_weight_cache = None
        return super()._apply(fn, recurse=recurse)


class _MetisFusedFunction(torch.autograd.Function):
    """y = ((x V^T) * s) U^T + deq(Q(x)) deq(Q(R))^T + b in one GEMM launch, with its gradients."""

    @staticmethod
    def forward(ctx, x, v, s, u, res, bias, px, p_res, xv=None, t=None, pending=None):
        F = LinearLowbitFunction
        cd = torch.bfloat16
        aop = None
        if pending is not None:
            # the quantizer's launch left the projection's partial sums (BitLinear._quantize_and_project)
            if p_res.rht is not None:
                xv, t, aop = ops.project_and_operand(_flat2d(x).to(cd), v.to(cd), s.to(cd), px,
                                                     ops.nv_operand_mode(px, [p_res], F.reference_rounding), pending=pending, rotate=p_res.rht)
            else:
                xv, t, aop = ops.project_and_operand(_flat2d(x).to(cd), v.to(cd), s.to(cd), px, ops.MODE_PB16, None, pending=pending)
        elif xv is None:
            # [L, r] rank-r projection and its product with s (bf16) on the library's kernels (split-K below 256 rows,
            # one pass over x from there on); the caller has it already when the quantizer's pass produced it
            x2, vb, sb = _flat2d(x).to(cd), v.to(cd), s.to(cd)
            in_operand = isinstance(px, CenteredNVFP4) and F._mean_in_operand(px, p_res)
            target = px.residual if in_operand else px
            if (isinstance(px, PackedNVFP4) and p_res.rht is not None and ops.nv_decode_applies(px, [p_res], [vb.shape[0]])
                    and ops.project_and_operand_applies(x2, vb, sb, px)):
                # NV recipe at decode size: the same merged launch, the operand rotated for the weight's domain
                xv, t, aop = ops.project_and_operand(x2, vb, sb, px, ops.nv_operand_mode(px, [p_res], F.reference_rounding), rotate=p_res.rht)
            elif ((in_operand or (isinstance(px, PackedNVFP4) and F.reference_rounding)) and p_res.rht is None
                    and ops.grouped_operand_applies(target, [p_res], [vb.shape[0]], px.mean if in_operand else None, True)
                    and ops.project_and_operand_applies(x2, vb, sb, target)):
                # decode-sized call in bf16 arithmetic: the projection's finishing step and the activation's GEMM
                # operands in one launch
                xv, t, aop = ops.project_and_operand(x2, vb, sb, target, ops.MODE_PB16, px.mean if in_operand else None)
            else:
                xv, t = ops.lowrank_project(x2, vb, sb)
        out_dtype = torch.float32 if F.compute_dtype == torch.float32 else torch.bfloat16
        ctx.center = None
        # binary32 arithmetic keeps a binary32 bias (as LinearLowbit and the centred path do); bf16 arithmetic adds it in bf16
        gemm_bias = None if bias is None else (bias.float() if F.compute_dtype == torch.float32 else bias.to(cd))
        if isinstance(px, CenteredNVFP4):
            # mean mode: the residual branch sees 1 me^T + R
            ctx.center = px.mean
            if F._mean_in_operand(px, p_res):
                # bf16 arithmetic: the activation operand is the reference's bf16 tensor me + QDQ(x - me)
                y = ops.linear_fwd_grouped(px.residual, [(p_res, t, u.to(cd), gemm_bias)], out_dtype=out_dtype, center=px.mean,
                                           reference_rounding=True, a_operand=aop)[0]
            elif px.rows < 256:
                # decode-sized: W^ me is accumulated inside the GEMM launch
                y = ops.linear_fwd_grouped(px.residual, [(p_res, t, u.to(cd), None if bias is None else bias.float())],
                                           out_dtype=out_dtype, center=px.center32)[0]
            else:
                # the mean term rides in a binary32 bias
                w_mean = ops.matvec(p_res, px.center32)
                y = ops.linear_fwd(px.residual, p_res, t=t, u=u.to(cd), bias=w_mean if bias is None else w_mean + bias.float(),
                                   out_dtype=out_dtype)
        else:
            y = ops.linear_fwd(px, p_res, t=t, u=u.to(cd), bias=gemm_bias, out_dtype=out_dtype,
                               reference_rounding=F.reference_rounding, a_operand=aop)
        ctx.save_for_backward(x, v, s, u, res, xv, t)               # t = bf16(xv * s): [L, r], kept for the gradient of U
        ctx.p_res = p_res
        ctx.has_bias = bias is not None
        ctx.lead = x.shape[:-1]
        return y.reshape(*ctx.lead, y.shape[-1]).to(F.compute_dtype)

    @staticmethod
    def _transposed_bf16(w: torch.Tensor) -> torch.Tensor:
        """w^T in bf16, contiguous, cached on the tensor until it is modified in place (the rank-r kernels read both
        factors with the rank as the slow dimension)."""
        key = (w._version, w.device, w.dtype)
        hit = getattr(w, "_metis_transposed", None)
        if hit is None or hit[0] != key:
            hit = (key, w.detach().to(torch.bfloat16).T.contiguous())
            try:
                w._metis_transposed = hit
            except AttributeError:                                   # a tensor subclass without a dict: no cache
                pass
        return hit[1]

    @staticmethod
    def backward(ctx, dy):
        F = LinearLowbitFunction
        F._check_backward_config()
        x, v, s, u, res, xv, t = ctx.saved_tensors
        cd = torch.bfloat16
        dy2 = _flat2d(dy).to(cd)
        x2 = _flat2d(x).to(cd)
        L, N = dy2.shape
        # rank-r branch in bf16: one pass over dY for dY U, one for dY^T t, one over x for g_xv^T x
        # dY U [L, r] and its product with s (the gradient with respect to x V^T) from the same launch
        g_t, g_xv = ops.lowrank_project(dy2, _MetisFusedFunction._transposed_bf16(u), s.to(cd))
        g_u = ops.lowrank_contract_tokens(dy2, t)                           # [N, r]
        # sum of the bf16 products, as autograd forms it for torch.mul(s, y); rounded once to the parameter's dtype
        g_s = ops.lowrank_scale_grad(g_t, xv, out_dtype=s.dtype if s.dtype in (torch.float32, torch.bfloat16) else torch.float32)
        g_v = ops.lowrank_contract_tokens(x2, g_xv, transpose=True)         # [r, K]
        # residual branch on re-quantized operands
        qg = F.q_backward_outputgrad
        if F._packed_backward_applies(L, N, dy2) and ctx.p_res.rht is not None:
            # NV recipe: rotated operands, blocks along the last dimension (see _packed_grads_nv)
            ar = F.compute_dtype
            dyq, xq_src = (_flat2d(dy), _flat2d(x)) if ar == torch.float32 else (dy2, x2)
            gx, g_res = F._packed_grads_nv(dyq, xq_src, ctx.p_res, cd, torch.bfloat16 if res.dtype == torch.bfloat16 else torch.float32,
                                           gx_lowrank=(g_xv, _MetisFusedFunction._transposed_bf16(v)))
        elif F._packed_backward_applies(L, N, dy2):
            ar = F.compute_dtype                               # arithmetic of the quantizers
            p_res_col = ctx.p_res.transposed                   # lives as long as the (cached) packed residual
            if p_res_col is None:
                p_res_col = ctx.p_res.transposed = F.q_forward_weight.pack(res, col=True, arith=ar)
            # binary32 arithmetic quantizes the tensors autograd handed over, not their bf16 roundings
            dyq, xq_src = (_flat2d(dy), _flat2d(x)) if ar == torch.float32 else (dy2, x2)
            # the rank-r branch's share of grad_input, g_xv V, rides in the dgrad launch as its low-rank extension
            gx, g_res = F._packed_grads(dyq, xq_src, p_res_col, ctx.center, cd,
                                        torch.bfloat16 if res.dtype == torch.bfloat16 else torch.float32,
                                        gx_lowrank=(g_xv, _MetisFusedFunction._transposed_bf16(v)))
        else:
            gx = torch.matmul(g_xv, v.to(cd))                  # [L, K]
            cdt = F.compute_dtype
            if F.enable_backward_svd:
                dyq = _flat2d(F.svd_quant(dy2.to(cdt), quant_func=qg, rank=F.backward_lowrank_svd, niter=F.backward_lowrank_niter,
                                          broadcast_dim=F.backward_broadcast_dim, tp_simulate=F.tp_simulate,
                                          tp_parts=F.tp_parts, metis_mode=F.metis_mode))
            else:
                dyq = F._quantize_wgrad_operand(dy2.to(cdt), qg)
            if ctx.center is not None:
                xq = ctx.center.to(cdt) + F.q_forward_input.quantize_dequantize(x2.to(cdt) - ctx.center.to(cdt))
            else:
                xq = F.q_forward_input.quantize_dequantize(x2.to(cdt))
            wq = F.q_forward_weight.quantize_dequantize(res.to(F.compute_dtype))
            gx = gx + torch.matmul(dyq, wq).to(cd)
            g_res = torch.matmul(dyq.T, xq).to(torch.float32)
        g_b = _token_sum(dy2, torch.float32) if ctx.has_bias else None
        return (gx.reshape(x.shape).to(x.dtype), g_v.to(v.dtype), g_s.to(s.dtype), g_u.to(u.dtype),
                g_res, g_b, None, None, None, None, None)


class BitLinear(nn.Module):
    """Drop-in for nn.Linear: W = U diag(s) V + W_res with the residual in NVFP4 (reference 597-940)."""
    rollout_merge_active = False
    # False (default): the rank-r branch sees the raw activation and bf16 V, U, s and is folded into the residual
    # GEMM's launch.  True: it consumes the quantized activation and the quantized V through their own GEMM, as the
    # reference's current file does (752, 863-879): two packed GEMMs and a dense rank-r GEMM per call.
    quantized_lowrank_branch = False

    def __init__(self, in_features, out_features, args=None, bias=True, dtype=torch.float32, compute_dtype=None):
        super().__init__()
        self.storage_dtype = dtype
        self.compute_dtype = compute_dtype if compute_dtype is not None else dtype
        if self.compute_dtype not in [torch.float32, torch.float16, torch.bfloat16]:
            raise ValueError(f"Unsupported compute_dtype: {self.compute_dtype}")
        if getattr(args, "enable_te", False):
            raise NotImplementedError("transformer_engine layers are not part of this build")
        if args.enable_forward_svd is False and args.enable_lowbit is True:
            self.warmup_linear = LinearLowbit(in_features, out_features, bias=bias, args=args,
                                              storage_dtype=self.storage_dtype, compute_dtype=self.compute_dtype)
        else:
            self.warmup_linear = nn.Linear(in_features, out_features, bias=bias, device=args.device, dtype=self.storage_dtype)
        self.ulinear = None
        self.vlinear = None
        self.s = None

        F = LinearLowbitFunction
        F.q_forward_input = quant_func[args.q_forward_input]
        F.q_forward_weight = quant_func[args.q_forward_weight]
        F.q_backward_input = quant_func[args.q_backward_input]
        F.q_backward_weight = quant_func[args.q_backward_weight]
        F.q_backward_outputgrad = quant_func[args.q_backward_outputgrad]
        F.enable_backward_svd = args.enable_backward_svd
        F.backward_lowrank_svd = args.backward_lowrank_svd
        F.backward_lowrank_niter = args.backward_lowrank_niter
        F.enable_activation_svd = args.enable_activation_svd
        F.activation_lowrank_svd = args.activation_lowrank_svd
        F.activation_lowrank_niter = args.activation_lowrank_niter
        F.activation_broadcast_dim = args.activation_broadcast_dim
        F.backward_broadcast_dim = args.backward_broadcast_dim
        F.enable_nv_recipe = args.enable_nv_recipe
        F.hadamard_workspace_mb = getattr(args, "hadamard_workspace_mb", 128)
        F.hadamard_tile_size = getattr(args, "hadamard_tile_size", 16)
        F.hadamard_backend = getattr(args, "hadamard_backend", "auto")
        F.tp_simulation = args.tp_simulation          # the reference writes this name and reads tp_simulate
        F.tp_parts = args.tp_parts
        F.compute_dtype = self.compute_dtype
        F.metis_mode = args.metis_mode

        self.args = args
        self.is_svd_quant = False
        if args.forward_svd_warmup_steps <= 0 and args.enable_forward_svd:
            self.split()
        self.mean_cache = {}
        self.activation_group = None
        self._merged_rollout_weight_cache = None
        self._merged_rollout_tiled = None
        self.layer_name = ""

    def _weights_cached(self) -> bool:
        """The packed weights of this layer's quantized branches live across calls (cache_quantized_weight)."""
        return bool(getattr(self.args, "cache_quantized_weight", False))

    # ------------------------------------------------------------------ shared activation (reference 676-702)
    def _get_shared_quantized_input(self, x: torch.Tensor):
        F = LinearLowbitFunction
        group = getattr(self, "activation_group", None)
        if group is None:
            return F._prepare_input(x, mean_cache=self.mean_cache, cache_key=f"{self.layer_name}.shared",
                                    weights_cached=self._weights_cached())
        input_ref = group.get("input_ref")
        if input_ref is not None and input_ref() is x:
            return group["quantized_input"]
        quantized_input = F._prepare_input(x, mean_cache=group["mean_cache"], cache_key=f"{group['name']}.shared",
                                           weights_cached=all(m._weights_cached() for m in group.get("members", ())))

        def clear_cached_input(ref):
            if group.get("input_ref") is ref:
                group["input_ref"] = None
                group["quantized_input"] = None

        group["input_ref"] = weakref.ref(x, clear_cached_input)
        group["quantized_input"] = quantized_input
        # every member's GEMM reads this activation: its tiled expansion is made once and kept while it lives
        packed = quantized_input.residual if isinstance(quantized_input, CenteredNVFP4) else quantized_input
        if isinstance(packed, PackedNVFP4):
            packed.shared = True
        return quantized_input

    @torch.no_grad()
    def _get_merged_rollout_weight(self, dtype: torch.dtype) -> torch.Tensor:
        """(U diag s) Q(V) + Q(W_res), cached on the parameters' versions (reference 704-730)."""
        F = LinearLowbitFunction
        key = (_pkey(self.vlinear.weight), _pkey(self.ulinear.weight), _pkey(self.s),
               _pkey(self.warmup_linear.weight), self.vlinear.weight.device, dtype, F.q_forward_weight, F.enable_nv_recipe)
        if self._merged_rollout_weight_cache is not None:
            cached_key, cached = self._merged_rollout_weight_cache
            if cached_key == key:
                return cached

        def deq(q):
            return q.dequantize(dtype) if isinstance(q, PackedNVFP4) else q

        qv = self.vlinear._get_quantized_weight(self.vlinear.weight.to(dtype))
        residual = deq(self.warmup_linear._get_quantized_weight(self.warmup_linear.weight.to(dtype)))
        us = self.ulinear.weight.to(dtype) * self.s.to(dtype).unsqueeze(0)
        r = us.shape[1]
        if (dtype == torch.bfloat16 and isinstance(qv, PackedNVFP4) and qv.rht is None and qv.mode == ops.MODE_PB16 and r % 32 == 0
                and qv.cols % 4 == 0):
            # bf16 arithmetic (the rollout's own configuration): the rank-r product on the tiled GEMM, bf16 operands,
            # binary32 accumulation, one rounding to bf16 -- what the reference's bf16 matmul computes; Q(V)^T [K, r] is
            # the transposed tiled expansion of the packed V
            low = ops.gemm_tiled(ops.dense_expand_tiled(us, ops.MODE_PB16), qv.unit, ops.expand_tiled_transposed(qv, mode=ops.MODE_PB16),
                                 qv.unit, us.shape[0], qv.cols, r, mode=ops.MODE_PB16, out_dtype=torch.bfloat16)
            merged = low + residual
        else:
            merged = us @ deq(qv) + residual
        self._merged_rollout_weight_cache = (key, merged)
        self._merged_rollout_tiled = None
        return merged

    def _rollout_forward(self, shared_input, x_shape):
        """y = QDQ(x) . merged^T (+ bias), the reference's one-matmul rollout forward (752-757).  bf16 arithmetic with a
        packed activation: the tiled GEMM on the activation's bf16 expansion and the merged weight as a dense tiled
        operand (cached with it), rounding the product and the bias add to bf16 as the reference's bf16 ops do.
        Otherwise the reference's formula on dequantized tensors."""
        F = LinearLowbitFunction
        bias = self.warmup_linear.bias
        if (isinstance(shared_input, PackedNVFP4) and shared_input.mode == ops.MODE_PB16 and shared_input.rht is None
                and F.compute_dtype == torch.bfloat16 and shared_input.cols % 32 == 0 and self.warmup_linear.weight.shape[0] % 4 == 0):
            merged = self._get_merged_rollout_weight(torch.bfloat16)
            if self._merged_rollout_tiled is None:
                self._merged_rollout_tiled = ops.dense_expand_tiled(merged, ops.MODE_PB16)
            y = ops.gemm_tiled(ops.expand_tiled(shared_input, cache=False, mode=ops.MODE_PB16), shared_input.unit, self._merged_rollout_tiled,
                               shared_input.unit, shared_input.rows, merged.shape[0], shared_input.cols, mode=ops.MODE_PB16,
                               bias=None if bias is None else bias.to(torch.bfloat16), out_dtype=torch.bfloat16)
            return y.reshape(*x_shape[:-1], merged.shape[0])
        if isinstance(shared_input, (PackedNVFP4, CenteredNVFP4, LowRankNVFP4)):
            shared_input = shared_input.dequantize(F.compute_dtype).reshape(x_shape)
        merged = self._get_merged_rollout_weight(shared_input.dtype)
        y = torch.matmul(shared_input, merged.T)
        if bias is not None:
            y = y + bias.to(y.dtype)
        return y

    def _apply(self, fn, recurse=True):
        self._merged_rollout_weight_cache = None
        self._merged_rollout_tiled = None
        self._bias_cast_cache = None
        group = getattr(self, "activation_group", None)
        if group is not None:
            group.pop("stacked_v", None)                         # parameters are replaced: versions start over
        return super()._apply(fn, recurse=recurse)

    # ------------------------------------------------------------------ projection group in one launch (inference)
    grouped_inference = True      # q/k/v and gate/up of a decode-sized batch as one GEMM launch when autograd is off

    def _packed_residual(self):
        """Packed residual weight for the fused launch, or None when the kernel path does not apply."""
        F = LinearLowbitFunction
        wl = self.warmup_linear
        if (not F.enable_nv_recipe or F._nv_on_kernels()) and _packable(wl.weight, F.q_forward_weight) and wl.weight.shape[0] % 4 == 0:
            p_res = wl._get_quantized_weight(wl.weight, arith=self.compute_dtype)       # cache hit: no pass over W
        else:
            p_res = wl._get_quantized_weight(wl.weight.to(self.compute_dtype))
        return p_res if isinstance(p_res, PackedNVFP4) else None

    def _fusable(self) -> bool:
        r = self.args.forward_svd_rank
        return (self.is_svd_quant and isinstance(self.vlinear, LinearLowbit) and isinstance(self.warmup_linear, LinearLowbit)
                and r > 0 and r % 32 == 0 and self.ulinear.bias is None and not BitLinear.quantized_lowrank_branch)

    def _quantize_and_project(self, x: torch.Tensor):
        """(packed activation, x V^T, bf16((x V^T) s)) from one pass over an activation that no sibling shares (direct
        mode, round to nearest, bf16 tensor of 256 rows or more), or None: both branches of the layer read x, the
        residual branch through the quantizer and the rank-r branch as it is.  A decode-sized activation in bf16
        arithmetic gives (packed activation, None, None, pending partial sums of the projection)."""
        F = LinearLowbitFunction
        if (F.enable_activation_svd or (F.enable_nv_recipe and not F._nv_on_kernels()) or F.q_forward_input is not Cast2NVFp4e2m1BlockNOSR
                or not x.is_cuda or x.dtype != torch.bfloat16 or F.compute_dtype not in (torch.float32, torch.bfloat16)):
            return None
        x2 = _flat2d(x)
        v = self.vlinear.weight
        if v.dtype != torch.bfloat16 or self._packed_residual() is None:
            return None
        mode = ops.MODE_P32 if F.compute_dtype == torch.float32 else ops.MODE_PB16
        if not F.enable_nv_recipe and ops.quantize_project_applies(x2, v, mode):
            return ops.quantize_project(x2, v.detach(), self.s.detach(), mode)
        # decode-sized call: the quantizer's launch carries the projection's first step, and the launch that builds the
        # GEMM's activation operands its finishing step (bf16 arithmetic; under the NV recipe either arithmetic, the
        # operand rotated for the weight's domain)
        p_res = self._packed_residual()
        if (self.s.dtype == torch.bfloat16 and ops.quantize_project_decode_applies(x2, v, mode) and x2.shape[0] * x2.shape[1] > 0
                and (p_res.rht is not None or (mode == ops.MODE_PB16 and F.reference_rounding))):
            probe = SimpleNamespace(rows=x2.shape[0], cols=x2.shape[1], mode=mode, rht=None)   # what the packed activation will be
            takes = (ops.nv_decode_applies(probe, [p_res], [v.shape[0]]) if p_res.rht is not None
                     else ops.grouped_operand_applies(probe, [p_res], [v.shape[0]], None, True))
            if takes:
                px, pending = ops.quantize_project_decode(x2, v.detach(), mode)
                return px, None, None, pending
        return None

    def _forward_group(self, x: torch.Tensor, shared_input):
        """All members of this layer's projection group on the shared activation in one call (no autograd):
        {id(member): output}, or None when the group does not qualify.  The siblings pick their result up when they
        are called with the same tensor object."""
        F = LinearLowbitFunction
        group = self.activation_group
        members = group["members"]
        rows = x.numel() // max(x.shape[-1], 1)
        if rows >= 256 or not all(m._fusable() and m.compute_dtype == self.compute_dtype for m in members):
            return None
        packed = [m._packed_residual() for m in members]
        if any(p is None for p in packed):
            return None
        rotated = any(p.rht is not None for p in packed)          # NV recipe: the activation's operand carries the rotation
        cd = torch.bfloat16
        x2 = _flat2d(x).to(cd)
        # one product for every member's rank-r projection: V of all members stacked, cached on their versions
        key = tuple((_pkey(m.vlinear.weight), _pkey(m.s)) for m in members) + (x2.device,)
        cached = group.get("stacked_v")
        if cached is None or cached[0] != key:
            cached = (key, torch.cat([m.vlinear.weight.to(cd) for m in members], dim=0),
                      torch.cat([m.s.to(cd) for m in members], dim=0))
            group["stacked_v"] = cached
        centre = shared_input.center32 if isinstance(shared_input, CenteredNVFP4) else None
        px = shared_input.residual if centre is not None else shared_input
        if centre is not None and all(F._mean_in_operand(shared_input, p) for p in packed):
            centre = shared_input.mean                             # bf16: goes into the activation operand (reference's bf16 tensor)
        if rotated and (centre is not None or not ops.nv_decode_applies(px, packed, [m.args.forward_svd_rank for m in members])):
            return None                                            # member by member on the tiled GEMM
        aop = None
        if rotated and ops.project_and_operand_applies(x2, cached[1], cached[2], px):
            # (the same launch with the operand rotated for the weights' domain)
            _, t_all, aop = ops.project_and_operand(x2, cached[1], cached[2], px, ops.nv_operand_mode(px, packed, F.reference_rounding),
                                                    rotate=packed[0].rht)
        elif (ops.grouped_operand_applies(px, packed, [m.args.forward_svd_rank for m in members], centre, F.reference_rounding)
                and ops.project_and_operand_applies(x2, cached[1], cached[2], px)):
            # the projection's finishing step and the activation's GEMM operands in one launch
            _, t_all, aop = ops.project_and_operand(x2, cached[1], cached[2], px, ops.MODE_PB16, centre)
        else:
            _, t_all = ops.lowrank_project(x2, cached[1], cached[2])
        calls, c0 = [], 0
        for m, p_res in zip(members, packed):
            r = m.args.forward_svd_rank
            bias = m.warmup_linear.bias
            if bias is not None:
                bias = m._bias_as(torch.float32 if (centre is not None and centre.dtype == torch.float32) else cd)
            calls.append((p_res, t_all[:, c0:c0 + r], m.ulinear.weight.to(cd), bias))      # a column slice: no copy
            c0 += r
        out_dtype = torch.float32 if F.compute_dtype == torch.float32 else torch.bfloat16
        # mean mode: every member also receives W^ me, inside the same launch (binary32)
        outs = ops.linear_fwd_grouped(px, calls, out_dtype=out_dtype, center=centre, reference_rounding=F.reference_rounding,
                                      a_operand=aop)
        lead = x.shape[:-1]
        return {id(m): y.reshape(*lead, y.shape[-1]).to(F.compute_dtype) for m, y in zip(members, outs)}

    def _bias_as(self, dtype: torch.dtype) -> torch.Tensor:
        """The residual branch's bias in `dtype`, converted once per parameter version (decode calls are launch-bound)."""
        b = self.warmup_linear.bias
        if b.dtype == dtype:
            return b
        key = (_pkey(b), b.device, dtype)
        cached = getattr(self, "_bias_cast_cache", None)
        if cached is None or cached[0] != key:
            cached = (key, b.detach().to(dtype))
            self._bias_cast_cache = cached
        return cached[1]

    # ------------------------------------------------------------------ forward (reference 736-769)
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        F = LinearLowbitFunction
        F.mean_cache = self.mean_cache
        if not self.is_svd_quant:
            return self.warmup_linear(x)
        group = self.activation_group
        if (BitLinear.grouped_inference and group is not None and not torch.is_grad_enabled() and len(group.get("members", ())) > 1
                and x.is_cuda and self._fusable()):
            ready = group.get("grouped_outputs")
            if ready is not None and ready[0]() is x and id(self) in ready[1]:
                return ready[1].pop(id(self))
            shared_input = self._get_shared_quantized_input(x)
            if isinstance(shared_input, (PackedNVFP4, CenteredNVFP4)):
                outs = self._forward_group(x, shared_input)
                if outs is not None:
                    mine = outs.pop(id(self))

                    def drop(ref, group=group):
                        if group.get("grouped_outputs") is not None and group["grouped_outputs"][0] is ref:
                            group["grouped_outputs"] = None
                    group["grouped_outputs"] = (weakref.ref(x, drop), outs)
                    return mine
        share_activation = (isinstance(self.vlinear, LinearLowbit) and isinstance(self.warmup_linear, LinearLowbit)
                            and self.args.forward_svd_rank > 0)
        if share_activation:
            r = self.args.forward_svd_rank
            fused = self._quantize_and_project(x) if (group is None and self._fusable()) else None
            shared_input = fused[0] if fused is not None else self._get_shared_quantized_input(x)
            if (isinstance(shared_input, (PackedNVFP4, CenteredNVFP4)) and r % 32 == 0 and self.ulinear.bias is None
                    and not BitLinear.quantized_lowrank_branch):
                # one fused launch for both branches; it already is the "merged" evaluation, so the
                # rollout switch changes nothing on this path
                p_res = self._packed_residual()
                if p_res is not None:
                    more = () if fused is None else fused[1:]
                    return _MetisFusedFunction.apply(x, self.vlinear.weight, self.s, self.ulinear.weight,
                                                     self.warmup_linear.weight, self.warmup_linear.bias, shared_input, p_res, *more)
            if BitLinear.rollout_merge_active and not torch.is_grad_enabled():
                return self._rollout_forward(shared_input, x.shape)
            y = self.vlinear(x, quantized_input=shared_input)
        else:
            F.mean_cache_key = f"{self.layer_name}.vlinear"
            y = self.vlinear(x)
        y = torch.mul(self.s, y)
        if y.dtype == self.ulinear.weight.dtype:
            y = self.ulinear(y)
        else:
            # the reference builds ulinear without a dtype (binary32, 872-876), so with compute_dtype=float32 this
            # matmul runs in binary32; here U is stored in the layer's dtype and widened for the product
            ub = self.ulinear.bias
            y = torch.nn.functional.linear(y, self.ulinear.weight.to(y.dtype), None if ub is None else ub.to(y.dtype))
        if self.args.forward_svd_rank > 0:
            if share_activation:
                y = y + self.warmup_linear(x, quantized_input=shared_input)
            else:
                F.mean_cache_key = f"{self.layer_name}.warmup"
                y = y + self.warmup_linear(x)
        return y

    # ------------------------------------------------------------------ factorisation (reference 776-924)
    @torch.no_grad()
    def split(self):
        if not self.args.enable_forward_svd:
            return
        if self.vlinear is not None:
            raise NotImplementedError("re-splitting an already factorised layer is not part of this build")
        if not self.args.enable_lowbit:
            raise NotImplementedError("enable_lowbit=False is not part of this build")
        w = self.warmup_linear.weight
        device, original_dtype = w.device, w.dtype
        u, s, v = torch.linalg.svd(w.to(torch.float32), full_matrices=False)
        u, s, v = u.to(original_dtype), s.to(original_dtype), v.to(original_dtype)
        bias = self.warmup_linear.bias
        rank = self.args.forward_svd_rank
        out_f, in_f = w.shape
        if rank > 0:
            residual = LinearLowbit(in_f, out_f, bias=bias is not None, args=self.args, device=device,
                                    storage_dtype=original_dtype, compute_dtype=self.compute_dtype)
            if bias is not None:
                residual.bias.copy_(bias)
            residual.weight.copy_(w - u[:, :rank] @ torch.diag(s[:rank]) @ v[:rank])
            self.warmup_linear = residual
            self.vlinear = LinearLowbit(in_f, rank, bias=False, args=self.args, device=device,
                                        storage_dtype=original_dtype, compute_dtype=self.compute_dtype)
            self.ulinear = nn.Linear(rank, out_f, bias=False, device=device, dtype=original_dtype)
            self.vlinear.weight.copy_(v[:rank, :])
            self.ulinear.weight.copy_(u[:, :rank])
            self.s = nn.Parameter(s[:rank].clone())
        else:
            self.vlinear = LinearLowbit(in_f, v.shape[0], bias=False, args=self.args, device=device,
                                        storage_dtype=original_dtype, compute_dtype=self.compute_dtype)
            self.ulinear = nn.Linear(u.shape[1], out_f, bias=False, device=device, dtype=original_dtype)
            self.vlinear.weight.copy_(v)
            self.ulinear.weight.copy_(u)
            self.s = nn.Parameter(s.clone())
            self.warmup_linear = None
        self.is_svd_quant = True

    @torch.no_grad()
    def lowrank_initialization(self, rank: int = 32):
        """Replace the weight by its best rank-r approximation (reference 926-940)."""
        W = self.warmup_linear.weight
        out_features, in_features = W.shape
        r = max(1, min(int(rank), min(out_features, in_features)))
        U, S, Vh = torch.linalg.svd(W.detach().to(torch.float32), full_matrices=False)
        W.copy_(((U[:, :r] * S[:r]) @ Vh[:r, :]).to(dtype=W.dtype, device=W.device))
