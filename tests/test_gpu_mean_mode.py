"""GPU parity of the pieces of the mean mode (column mean kept in high precision, centred residual in
NVFP4): centred quantizers bit-exact against the oracle on x - me, the packed matrix-vector product and
the binary32 bias of the GEMM against double precision."""
import dataclasses

import pytest
import torch

from helpers import rel_fro, synthetic_activation

pytestmark = pytest.mark.gpu


def _check(p, codes, scales, unit, what):
    torch.cuda.synchronize()
    assert torch.equal(p.codes.cpu(), codes), f"codes differ ({what}): {(p.codes.cpu() != codes).sum().item()}"
    assert torch.equal(p.scales.cpu(), scales), f"scales differ ({what})"
    assert float(p.unit.cpu()) == float(unit), f"unit differs ({what})"


def _offset_activation(seed, rows, cols):
    x = synthetic_activation(seed, rows, cols).float()
    g = torch.Generator().manual_seed(seed + 1)
    return (x + 3.0 * torch.randn(1, cols, generator=g)).bfloat16()        # a per-column offset worth removing


@pytest.mark.parametrize("col", [False, True])
@pytest.mark.parametrize("src", ["bf16", "f32"])
def test_centered_quant_binary32_arithmetic(col, src):
    """x - me in binary32 (one rounding, as the reference's `input_flat - me`), then the quantizer."""
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = _offset_activation(500, 256, 192)
    xin = x.float() if src == "bf16" else x.float() + 1e-3 * torch.randn(256, 192, generator=torch.Generator().manual_seed(3))
    me = xin.mean(dim=0)
    res = xin - me
    p = ops.quantize((x if src == "bf16" else xin).cuda(), 0, col=col, center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res)
    _check(p, codes, scales, unit, f"rne col={col} {src}")
    u = torch.rand(256, 192, generator=torch.Generator().manual_seed(4))
    p = ops.quantize((x if src == "bf16" else xin).cuda(), 0, col=col, sr=True, noise=u.cuda(), center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res, u)
    _check(p, codes, scales, unit, f"sr col={col} {src}")


@pytest.mark.parametrize("col", [False, True])
def test_centered_quant_bf16_arithmetic(col):
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = _offset_activation(510, 128, 256)
    me = x.mean(dim=0)                                             # bf16, as torch gives it for a bf16 tensor
    res = x - me                                                   # bf16 subtraction: one rounding
    p = ops.quantize(x.cuda(), 1, col=col, center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res)
    _check(p, codes, scales, unit, f"pb16 col={col}")
    u = torch.rand(128, 256, generator=torch.Generator().manual_seed(5)).bfloat16()
    p = ops.quantize(x.cuda(), 1, col=col, sr=True, noise=u.cuda(), center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res, u)
    _check(p, codes, scales, unit, f"pb16 sr col={col}")


def test_centered_quant_own_stream_and_errors():
    from metis_hip import _lib, ops
    x = _offset_activation(520, 64, 128).cuda()
    me = x.float().mean(dim=0)
    a = ops.quantize(x, 0, sr=True, seed=7, offset=3, center=me)
    b = ops.quantize(x, 0, sr=True, seed=7, offset=3, center=me)
    rne = ops.quantize(x, 0, center=me)
    assert torch.equal(a.codes, b.codes) and torch.equal(a.scales, rne.scales) and float(a.unit) == float(rne.unit)
    with pytest.raises(ValueError):
        ops.quantize(x, 0, center=me[:-1])


@pytest.mark.parametrize("rows,cols", [(192, 256), (1000, 48), (3584, 18944), (5, 16), (18944, 3584), (16387, 32), (1001, 4096)])
def test_packed_matvec(rows, cols):
    from metis_hip import ops
    g = torch.Generator().manual_seed(rows + cols)
    w = (torch.randn(rows, cols, generator=g) * 0.05).bfloat16().cuda()
    p = ops.quantize(w)
    v = torch.randn(cols, generator=g).cuda()
    deq = ops.dequantize(p, torch.float32).double()
    y = ops.matvec(p, v, alpha=0.5)
    want = 0.5 * (deq @ v.double())
    assert rel_fro(y.cpu().double(), want.cpu()) <= 1e-5
    ones = ops.matvec(p)
    assert rel_fro(ones.cpu().double(), deq.sum(dim=1).cpu()) <= 1e-5
    split = torch.zeros(rows, 32, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(rows, dtype=torch.float32, device="cuda")
    ops.matvec(p, v, out=out, split=split, split_col=4)
    torch.cuda.synchronize()
    back = split[:, 4].float() + split[:, 5].float() + split[:, 6].float()
    assert torch.equal(back, out) or float((back - out).abs().max()) <= 1e-7 * float(out.abs().max())
    assert int((split[:, :4] != 0).sum()) == 0 and int((split[:, 7:] != 0).sum()) == 0


@pytest.mark.parametrize("M,N,K", [(64, 512, 1024), (300, 260, 512), (512, 512, 2048), (128, 136, 96)])
def test_gemm_binary32_bias(M, N, K):
    """Every GEMM kernel (skinny, 256-tiles, split-K, 128-tiles) adds a binary32 bias at full precision."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + N)
    x = synthetic_activation(530 + M, M, K).cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 3.0).cuda()             # binary32, not bf16-valued
    px, pw = ops.quantize(x), ops.quantize(w)
    got = ops.linear_fwd(px, pw, bias=bias, out_dtype=torch.float32)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T + bias.double()
    torch.cuda.synchronize()
    assert rel_fro(got.cpu(), want.cpu()) <= 1e-6


# ---------------------------------------------------------------------------------------------
# module path: reference defaults (metis_mode="mean", activation and backward "svd" switches on)
# ---------------------------------------------------------------------------------------------
def _mean_args(rank=32):
    from metis_hip import MetisArgs
    args = MetisArgs(forward_svd_rank=rank, cache_quantized_weight=True)      # the reference's defaults: mean mode
    assert args.metis_mode == "mean" and args.enable_activation_svd and args.enable_backward_svd
    return args


def _oracle_mean_qdq(x32):
    from oracle import metis_oracle as O
    me = x32.mean(dim=0, keepdim=True)
    return me + O.nvfp4_qdq(x32 - me)


@pytest.mark.parametrize("M,K,Ns,r,one_pass", [(64, 3584, (3584, 512, 512), 64, True), (64, 18944, (3584,), 64, True),
                                               (1, 1024, (256, 96), 0, True), (40, 8192, (100,), 32, True),
                                               (200, 512, (260, 64), 32, True), (8, 8448, (8192,), 0, False),
                                               (16, 320, (128,), 0, False)])
def test_grouped_decode_gemm_with_the_centre_inside(M, K, Ns, r, one_pass):
    """Mean mode at decode size: out = R W^T + 1 (W^ me)^T + t u^T + bias with W^ me accumulated inside the GEMM
    launch.  Checked against double precision and against the two-pass form (packed matvec, then a binary32 bias);
    shapes whose centre slice does not fit the kernel (or K % 256 != 0) take the two-pass form by themselves."""
    import ctypes
    from metis_hip import _lib, ops
    g = torch.Generator().manual_seed(M + K)
    x = _offset_activation(600 + M, M, K).cuda()
    me = x.float().mean(dim=0) + 0.01 * torch.randn(K, generator=g).cuda()      # a running mean is not the batch mean
    px = ops.quantize(x, 0, center=me)
    members = []
    for i, N in enumerate(Ns):
        pw = ops.quantize((torch.randn(N, K, generator=g) * 0.05).bfloat16().cuda())
        t = u = None
        if r and i != 1:
            t = torch.randn(M, r, generator=g).bfloat16().cuda()
            u = (torch.randn(N, r, generator=g) * 0.1).bfloat16().cuda()
        bias = torch.randn(N, generator=g).cuda() if i % 2 == 0 else None
        members.append((pw, t, u, bias))
    arr = (_lib.LinearMember * len(Ns))()
    for i, N in enumerate(Ns):
        arr[i].N = N
    ap = ctypes.cast(arr, ctypes.c_void_p)
    L = _lib.load()
    has_ws = L.metis_linear_grouped_workspace_bytes(M, K, ap, len(Ns)) > 0
    assert bool(L.metis_linear_grouped_centered_supported(M, K, ap, len(Ns), int(has_ws))) == one_pass
    dr = ops.dequantize(px, torch.float32).double()
    for dt in (torch.float32, torch.bfloat16):
        got = ops.linear_fwd_grouped(px, members, out_dtype=dt, center=me)
        for (pw, t, u, b), y in zip(members, got):
            dw = ops.dequantize(pw, torch.float32).double()
            want = (dr + me.double()) @ dw.T
            if t is not None:
                want = want + t.double() @ u.double().T
            if b is not None:
                want = want + b.double()
            two_pass = ops.linear_fwd(px, pw, t=t, u=u, out_dtype=dt,
                                      bias=ops.matvec(pw, me) if b is None else ops.matvec(pw, me) + b)
            tol = 5e-5 if dt == torch.float32 else 2e-3
            assert rel_fro(y.cpu(), want.cpu().to(dt)) <= tol
            assert rel_fro(y.float().cpu(), two_pass.float().cpu()) <= (1e-5 if dt == torch.float32 else 2e-3)


def test_linear_lowbit_mean_mode_forward_runs_packed_and_matches_oracle(monkeypatch):
    """LinearLowbit under the reference's default arguments: mean + QDQ(x - mean) against QDQ(W), on the
    packed kernels (no dequantized activation or weight is ever formed)."""
    from metis_hip import BitLinear, LinearLowbitFunction as F, ops
    from oracle import metis_oracle as O
    K, N, L = 256, 192, 128
    args = _mean_args()
    args.enable_forward_svd = False                                # keep the plain quantized linear, no factorisation
    layer = BitLinear(K, N, args=args, bias=True, dtype=torch.bfloat16, compute_dtype=torch.float32).cuda()
    lin = layer.warmup_linear
    calls = []
    real = ops.dequantize
    monkeypatch.setattr(ops, "dequantize", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    x = _offset_activation(600, L, K).reshape(2, L // 2, K)
    y = lin(x.cuda())
    assert not calls and y.dtype == torch.float32
    w = lin.weight.detach().cpu().float()
    want = _oracle_mean_qdq(x.reshape(L, K).float()).double() @ O.nvfp4_qdq(w).double().T + lin.bias.detach().cpu().double()
    assert rel_fro(y.detach().cpu().reshape(L, N).double(), want) <= 1e-4
    # removing the mean matters on this input: plain quantization of x is visibly worse against the dense product
    dense = x.reshape(L, K).double() @ w.double().T + lin.bias.detach().cpu().double()
    plain = O.nvfp4_qdq(x.reshape(L, K).float()).double() @ O.nvfp4_qdq(w).double().T + lin.bias.detach().cpu().double()
    assert rel_fro(y.detach().cpu().reshape(L, N).double(), dense) < rel_fro(plain, dense)


@pytest.mark.parametrize("compute", [torch.float32, torch.bfloat16])
def test_packed_grads_mean_mode_decomposition(compute):
    """The rank-one bookkeeping of the mean mode, made deterministic with round-to-nearest quantizers:
    gX = (1 me_dy^T + R_dy) W^, gW = (1 me_dy^T + R_dy)^T (1 me_x^T + R_x), evaluated in double precision
    from the same packed residuals."""
    from metis_hip import LinearLowbitFunction as F, ops, quant_func
    L, N, K = 256, 192, 320
    g = torch.Generator().manual_seed(610)
    x = _offset_activation(611, L, K).cuda()
    dy = ((torch.randn(L, N, generator=g) + 0.7 * torch.randn(1, N, generator=g)) * 1e-2).bfloat16().cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    keep = (F.q_backward_outputgrad, F.q_backward_input, F.enable_backward_svd, F.compute_dtype, F.metis_mode,
            F.backward_lowrank_svd, F.tp_simulate, F.enable_nv_recipe)
    rne = quant_func["nvfp4e2m1bnosr"]
    try:
        F.q_backward_outputgrad, F.q_backward_input, F.enable_backward_svd, F.compute_dtype = rne, rne, True, compute
        F.metis_mode, F.backward_lowrank_svd, F.tp_simulate, F.enable_nv_recipe = "mean", 64, False, False
        me_x = F._token_mean(x)
        pw_col = rne.pack(w, col=True, arith=compute)
        gx, gw = F._packed_grads(dy, x, pw_col, me_x, torch.float32, torch.float32)
        me_dy = F._token_mean(dy)
        # exact operand values code * e4m3 * unit (what the GEMM multiplies), also for tensors packed in bf16 arithmetic
        d = lambda p: ops.dequantize(dataclasses.replace(p, mode=0), torch.float32).double()
        dy_hat = me_dy.double() + d(rne.pack(dy, arith=compute, center=me_dy))
        want_gx = dy_hat @ d(pw_col).t()                                   # [L, N] x [N, K]: pw_col is W^T packed as [K, N]
        dyt_hat = me_dy.double().unsqueeze(1) + d(rne.pack(dy, col=True, arith=compute, center=me_dy))     # [N, L]
        xt_hat = me_x.double().unsqueeze(1) + d(rne.pack(x, col=True, arith=compute, center=me_x))         # [K, L]
        want_gw = dyt_hat @ xt_hat.t()
    finally:
        (F.q_backward_outputgrad, F.q_backward_input, F.enable_backward_svd, F.compute_dtype, F.metis_mode,
         F.backward_lowrank_svd, F.tp_simulate, F.enable_nv_recipe) = keep
    torch.cuda.synchronize()
    assert rel_fro(gx.cpu().double(), want_gx.cpu()) <= 1e-5
    assert rel_fro(gw.cpu().double(), want_gw.cpu()) <= 1e-5


def test_bitlinear_mean_mode_forward_backward_and_decode_running_mean():
    """Split BitLinear under the reference's defaults: forward against the formula with mean-mode
    activations, gradients at FP4 noise level of the dense ones, and the single-token running mean."""
    from metis_hip import BitLinear, LinearLowbitFunction as F
    from oracle import metis_oracle as O
    K, N, r, L = 256, 192, 32, 128
    g = torch.Generator().manual_seed(620)
    w = torch.randn(N, K, generator=g) * 0.02 + (torch.linalg.qr(torch.randn(N, 8, generator=g))[0] * 3.0) @ torch.linalg.qr(torch.randn(K, 8, generator=g))[0].T
    layer = BitLinear(K, N, args=_mean_args(r), bias=True, dtype=torch.bfloat16, compute_dtype=torch.float32).cuda()
    with torch.no_grad():
        layer.warmup_linear.weight.copy_(w)
    layer.split()
    x = _offset_activation(621, L, K).reshape(2, L // 2, K).cuda().requires_grad_(True)
    y = layer(x)
    xf = x.detach().cpu().reshape(L, K).float()
    v, s, u = (t.detach().cpu().float() for t in (layer.vlinear.weight, layer.s, layer.ulinear.weight))
    res, b = layer.warmup_linear.weight.detach().cpu().float(), layer.warmup_linear.bias.detach().cpu().float()
    low = ((xf.bfloat16() @ v.bfloat16().T) * s.bfloat16()).float() @ u.bfloat16().float().T        # bf16 rank-r branch
    want = low.double() + _oracle_mean_qdq(xf).double() @ O.nvfp4_qdq(res).double().T + b.double()
    assert rel_fro(y.detach().cpu().reshape(L, N).double(), want) <= 2e-3
    dy = ((torch.randn(2, L // 2, N, generator=g) + 0.5) * 1e-2).bfloat16().cuda()
    y.backward(dy.to(y.dtype))
    dyf = dy.reshape(L, N).float().cpu()
    assert rel_fro(x.grad.reshape(L, K).float().cpu(), dyf @ w) < 0.1
    assert rel_fro(layer.warmup_linear.weight.grad.float().cpu(), dyf.T @ xf) < 0.3
    for p in (layer.vlinear.weight, layer.ulinear.weight, layer.s, layer.warmup_linear.weight, layer.warmup_linear.bias):
        assert p.grad is not None and bool(torch.isfinite(p.grad).all())
    # decode: single-token calls fold into the cached mean with their row counts (reference 316-323)
    key = f"{layer.layer_name}.shared"
    cached, count = layer.mean_cache[key]
    assert count == L
    step = _offset_activation(622, 4, K).reshape(4, 1, K).cuda()
    with torch.no_grad():
        y1 = layer(step)
    me2, count2 = layer.mean_cache[key]
    assert count2 == L + 4
    want_me = (cached * L + step.reshape(4, K).float().mean(dim=0, keepdim=True) * 4) / (L + 4)
    assert torch.allclose(me2, want_me, rtol=1e-6, atol=1e-7)
    sf = step.reshape(4, K).float().cpu()
    mec = want_me.cpu()
    low1 = ((sf.bfloat16() @ v.bfloat16().T) * s.bfloat16()).float() @ u.bfloat16().float().T
    want1 = low1.double() + (mec + O.nvfp4_qdq(sf - mec)).double() @ O.nvfp4_qdq(res).double().T + b.double()
    assert rel_fro(y1.cpu().reshape(4, N).double(), want1) <= 2e-3


@pytest.mark.parametrize("rows,cols,dtype", [(4096, 8960, torch.float32), (128, 256, torch.bfloat16), (1, 64, torch.float32),
                                             (1000, 1540, torch.bfloat16), (17, 4, torch.float32)])
def test_column_mean(rows, cols, dtype):
    from metis_hip import ops
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, cols, generator=g) + 2.0 * torch.randn(1, cols, generator=g)).to(dtype)
    want = x.double().mean(dim=0)
    got32 = ops.column_mean(x.cuda(), torch.float32).cpu()
    assert float((got32.double() - want).abs().max()) <= 1e-6 * float(want.abs().max() + 1)
    total = ops.column_sum(x.cuda(), torch.float32).cpu()
    assert float((total.double() - want * rows).abs().max()) <= 2e-6 * float((want * rows).abs().max() + rows)
    got16 = ops.column_mean(x.cuda(), torch.bfloat16).cpu()
    assert got16.dtype == torch.bfloat16 and float((got16.double() - want).abs().max()) <= 2 ** -8 * float(want.abs().max() + 1)
    # a strided view (row stride > cols)
    wide = torch.zeros(rows, cols + 8, dtype=dtype)
    wide[:, :cols] = x
    xs = wide.cuda()[:, :cols]
    if not xs.is_contiguous():
        again = ops.column_mean(xs, torch.float32).cpu()
        assert torch.equal(again, got32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_running_mean_update_matches_the_tensor_expression_bit_for_bit(dtype):
    """Decode calls: me = (cached * count + mean(x) * rows) / (count + rows) with every operation rounded to the
    arithmetic's dtype (reference bitlinear.py:316-323, evaluated on the CPU: true division), fused behind the
    column reduction; the float32 copy holds the same values."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(77)
    x = (torch.randn(64, 1, 3584, generator=g) + 0.5).to(dtype).cuda()
    cached = (torch.randn(3584, generator=g) * 0.3 + 0.5).to(dtype)
    this_mean = ops.column_mean(x, dtype).cpu()
    for count in (64, 4096, 1_000_003):
        me, me32 = ops.column_mean_running(x, cached.cuda(), count, dtype)
        want = (cached * count + this_mean * 64) / (count + 64)
        assert want.dtype == dtype
        assert torch.equal(me.cpu(), want), count
        assert me32.dtype == torch.float32 and torch.equal(me32.cpu(), want.float())
    me, me32 = ops.column_mean_running(x, None, 0, dtype)
    assert torch.equal(me.cpu(), this_mean) and torch.equal(me32.cpu(), this_mean.float())


def test_rank_one_operands_reach_binary32_precision():
    from metis_hip import ops
    g = torch.Generator().manual_seed(700)
    n, k = 300, 200
    a1, b1, a2, b2 = (torch.randn(m, generator=g).cuda() * s for m, s in ((n, 3.0), (k, 0.01), (n, 1e-3), (k, 50.0)))
    t, u = ops.rank_one_operands(n, k, (a1, b1), (a2, b2))
    got = t.double() @ u.double().T
    want = torch.outer(a1.double(), b1.double()) + torch.outer(a2.double(), b2.double())
    assert rel_fro(got.cpu(), want.cpu()) <= 2e-7
    t, u = ops.rank_one_operands(n, k, (a1, b1))
    assert rel_fro((t.double() @ u.double().T).cpu(), torch.outer(a1.double(), b1.double()).cpu()) <= 2e-7
    assert int((t[:, 6:] != 0).sum()) == 0 and int((u[:, 6:] != 0).sum()) == 0
    # the affine tail of the matrix-vector product
    w = (torch.randn(n, 64, generator=g) * 0.1).bfloat16().cuda()
    p = ops.quantize(w)
    y = ops.matvec(p, z=a1, beta=7.0)
    want = ops.dequantize(p, torch.float32).double().sum(dim=1) + 7.0 * a1.double()
    assert rel_fro(y.cpu().double(), want.cpu()) <= 1e-6


def test_qwen2_decoder_layer_under_the_reference_default_arguments(monkeypatch):
    """A Hugging Face Qwen2 decoder layer patched with MetisArgs() as the reference constructs it (mean mode for
    activations and output gradients): every projection runs on the packed kernels, and the result stays close to
    the same layer evaluated on dequantized tensors and torch matmuls (the generic path)."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import BitLinear, LinearLowbitFunction as F, MetisArgs, ops, replace_model_with_metis
    torch.manual_seed(0)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
    holder = torch.nn.ModuleDict({"layer": layer})
    x = (torch.randn(2, 64, 256, device="cuda") + 1.5 * torch.randn(1, 1, 256, device="cuda")).bfloat16()
    pos = torch.arange(64, device="cuda").unsqueeze(0).expand(2, -1)
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)

    def run(inp):
        out = holder["layer"](inp, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return out[0] if isinstance(out, tuple) else out

    args = MetisArgs(forward_svd_rank=32)
    assert args.metis_mode == "mean" and args.enable_activation_svd and args.enable_backward_svd
    replace_model_with_metis(holder, args)
    assert sum(isinstance(m, BitLinear) and m.is_svd_quant for m in holder.modules()) == 7
    centred = []
    real = ops.quantize
    monkeypatch.setattr(ops, "quantize", lambda *a, **k: (centred.append(k.get("center") is not None), real(*a, **k))[1])
    xr = x.clone().requires_grad_(True)
    out = run(xr)
    n_fwd = sum(centred)
    assert n_fwd == 4                                              # q/k/v share one, o, gate/up share one, down
    out.float().square().mean().backward()
    assert sum(centred) > n_fwd                                    # gradients are centred too
    gx_packed = xr.grad.detach().float().cpu()
    assert bool(torch.isfinite(gx_packed).all())
    # generic evaluation of the same modules
    monkeypatch.setattr(F, "_mean_mode_packable", staticmethod(lambda: False))
    for m in holder.modules():
        if isinstance(m, BitLinear):
            m.mean_cache.clear()
            if m.activation_group is not None:
                m.activation_group["mean_cache"].clear()
    xg = x.clone().requires_grad_(True)
    ref = run(xg)
    # not the same formula to the last bit: the fused launch feeds the rank-r branch the raw bf16 activation, the
    # generic evaluation feeds it the quantized one (both documented variants), so agreement is at FP4-noise level
    assert rel_fro(out.detach().float().cpu(), ref.detach().float().cpu()) <= 2e-2
    ref.float().square().mean().backward()
    assert rel_fro(gx_packed, xg.grad.detach().float().cpu()) < 0.2      # both carry independent stochastic rounding


@pytest.mark.parametrize("rows,cols", [(64, 512), (333, 1536), (4096, 3584), (16384, 4096), (7, 48), (1, 256)])
def test_rmsnorm_with_column_mean(rows, cols):
    """metis_rmsnorm_colmean: the normed tensor is that of the fused RMSNorm -> NVFP4 kernel, bit for bit; its column
    mean over tokens agrees with a double-precision mean of that tensor to binary32 / bf16 rounding; the running mean of
    decode calls follows the reference's tensor expression bit for bit given this call's mean; and the whole chain
    against the oracle: O.rmsnorm within the norm's tolerance, then me + QDQ(x - me) with codes and scale bytes
    bit-exact on the kernel's own normed tensor and mean."""
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = _offset_activation(900 + rows, rows, cols)
    gamma = (1 + 0.1 * torch.randn(cols, generator=torch.Generator().manual_seed(9))).bfloat16()
    ref_normed, _ = ops.rmsnorm_quantize(x.cuda(), gamma.cuda(), 1e-6, 0)
    normed, me, me32 = ops.rmsnorm_colmean(x.cuda(), gamma.cuda(), 1e-6, torch.float32)
    assert torch.equal(normed, ref_normed) and me32 is me
    assert rel_fro(normed.cpu(), O.rmsnorm(x, gamma, 1e-6)) <= 2e-3
    want = normed.cpu().double().mean(dim=0)
    assert float((me.cpu().double() - want).abs().max()) <= 1e-6 * float(want.abs().max() + 1)
    again = ops.rmsnorm_colmean(x.cuda(), gamma.cuda(), 1e-6, torch.float32)[1]
    assert torch.equal(again, me)                                  # fixed summation order: the same bits call after call
    # the same tensor OBJECTS with new contents (a serving loop's buffers): every call reads them afresh
    buf, gd = x.cuda(), gamma.cuda()
    first = ops.rmsnorm_colmean(buf, gd, 1e-6, torch.float32)
    buf.mul_(-0.5)
    buf[:, 0] += 3.0
    second = ops.rmsnorm_colmean(buf, gd, 1e-6, torch.float32)
    assert second[0].data_ptr() != first[0].data_ptr() and not torch.equal(second[1], first[1])
    assert torch.equal(second[0], ops.rmsnorm_quantize(buf, gd, 1e-6, 0)[0])
    # centred quantizer on the kernel's own outputs, against the oracle formula
    p = ops.quantize(normed, 0, center=me)
    codes, scales, unit, _ = O.nvfp4_pack(normed.cpu().float() - me.cpu())
    _check(p, codes, scales, unit, f"fused norm, mean mode {rows}x{cols}")
    # bf16 arithmetic: every operation of the mean rounded to bf16
    n16, me16, me16_32 = ops.rmsnorm_colmean(x.cuda(), gamma.cuda(), 1e-6, torch.bfloat16)
    assert torch.equal(n16, normed) and me16.dtype == torch.bfloat16 and torch.equal(me16_32, me16.float())
    assert float((me16.cpu().double() - want).abs().max()) <= 2 ** -8 * float(want.abs().max() + 1)
    p16 = ops.quantize(normed, 1, center=me16)
    codes, scales, unit, _ = O.nvfp4_pack(normed.cpu() - me16.cpu())
    _check(p16, codes, scales, unit, f"fused norm, mean mode, bf16 arithmetic {rows}x{cols}")
    # running mean (decode calls)
    for dtype, this_mean in ((torch.float32, me.cpu()), (torch.bfloat16, me16.cpu())):
        cached = (torch.randn(cols, generator=torch.Generator().manual_seed(11)) * 0.3).to(dtype)
        for count in (64, 1_000_003):
            _, run, run32 = ops.rmsnorm_colmean(x.cuda(), gamma.cuda(), 1e-6, dtype, cached.cuda(), count)
            wantr = (cached * count + this_mean * rows) / (count + rows)
            assert wantr.dtype == dtype and torch.equal(run.cpu(), wantr) and torch.equal(run32.cpu(), wantr.float())


@pytest.mark.parametrize("compute", [torch.float32, torch.bfloat16])
def test_fused_norm_feeds_the_projection_groups_under_the_reference_default_arguments(monkeypatch, compute):
    """MetisArgs() as the reference constructs it (mean mode) with the norms fused into the q/k/v and gate/up groups:
    no torch RMSNorm runs (the module's eager fallback is made to raise), the group's activation arrives as a
    CenteredNVFP4 whose mean is the column mean of the normed tensor, the running mean of decode calls lands in the
    group's cache, and the layer's output agrees with the same layer with unfused norms."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import BitLinear, LinearLowbitFunction as F, MetisArgs, replace_linear_with_metis
    from metis_hip.norm import FusedRMSNormQuant, fuse_rmsnorm_into_groups
    from metis_hip.ops import CenteredNVFP4
    torch.manual_seed(0)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"

    def build(fuse):
        torch.manual_seed(1)
        layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
        for p in layer.parameters():
            if p.dim() == 2:
                torch.nn.init.normal_(p, std=0.02)
        holder = torch.nn.ModuleDict({"layer": layer})
        args = MetisArgs(forward_svd_rank=32)
        replace_linear_with_metis(holder, torch.bfloat16, args, compute_dtype=compute)
        if fuse:
            assert fuse_rmsnorm_into_groups(holder) == 2
        return holder

    x = (torch.randn(2, 64, 256, device="cuda") + 1.5 * torch.randn(1, 1, 256, device="cuda")).bfloat16()
    pos = torch.arange(64, device="cuda").unsqueeze(0).expand(2, -1)
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)
    plain, fused = build(False), build(True)
    assert sum(isinstance(m, FusedRMSNormQuant) for m in fused.modules()) == 2
    real_plain = FusedRMSNormQuant._plain

    def plain_only_for_binary32(self, t):
        # with compute_dtype=float32 the residual stream after the first block is binary32 (the reference's forward returns
        # its compute dtype): that input keeps the eager norm; a bf16 input must never reach it
        assert t.dtype != torch.bfloat16, "eager RMSNorm ran on a bf16 tensor"
        return real_plain(self, t)
    monkeypatch.setattr(FusedRMSNormQuant, "_plain", plain_only_for_binary32)
    seen = []
    real = BitLinear._get_shared_quantized_input
    monkeypatch.setattr(BitLinear, "_get_shared_quantized_input", lambda self, t: (seen.append(real(self, t)), seen[-1])[1])
    with torch.no_grad():
        want = plain["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
        seen.clear()
        got = fused["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
    want, got = (t[0] if isinstance(t, tuple) else t for t in (want, got))
    assert all(isinstance(q, CenteredNVFP4) for q in seen) and len(seen) == 4     # q/k/v as one group call, o, gate/up, down
    # the rows' sums of squares are taken in another order than torch's: single roundings of the normed tensor may differ
    assert rel_fro(got.float().cpu(), want.float().cpu()) <= 2e-3
    group = fused["layer"].self_attn.q_proj.activation_group
    key = f"{group['name']}.shared"
    assert key in group["mean_cache"] and group["mean_cache"][key][1] == 128
    # a decode call updates the running mean through the same kernel
    xd = x[:, :1].contiguous()
    with torch.no_grad():
        fused["layer"](xd, position_embeddings=tuple(t[:, :1] for t in pe), attention_mask=None, position_ids=pos[:, :1])
    assert group["mean_cache"][key][1] == 130
    F.enable_activation_svd = False
    F.enable_backward_svd = False


def _mean_golden():
    import os
    import numpy as np
    return dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_mean_mode.npz")))


@pytest.mark.parametrize("tag,cd", [("p32", torch.float32), ("pb16", torch.bfloat16)])
def test_mean_mode_against_reference_vectors(tag, cd):
    """The reference's own svd_quant(metis_mode="mean") outputs (prefill, then a decode call on the same cache)
    against the packed path (centred quantizer + mean vector) and against the generic path."""
    from helpers import t
    from metis_hip import CenteredNVFP4, LinearLowbitFunction as F, quant_func
    g = _mean_golden()
    keep = (F.compute_dtype, F.enable_activation_svd, F.metis_mode, F.tp_simulate, F.enable_nv_recipe, F.q_forward_input)
    F.compute_dtype, F.enable_activation_svd, F.metis_mode, F.tp_simulate, F.enable_nv_recipe = cd, True, "mean", False, False
    F.q_forward_input = quant_func["nvfp4e2m1bnosr"]
    try:
        x, step = t(g["mean_x"]).cuda(), t(g["mean_step"]).cuda()
        for path in ("packed", "generic"):
            cache = {}
            if path == "packed":
                a = F._prepare_input(x, mean_cache=cache, cache_key="k")
                assert isinstance(a, CenteredNVFP4)
                got = a.dequantize(cd).reshape(x.shape)
                b = F._prepare_input(step, mean_cache=cache, cache_key="k")
                got_step = b.dequantize(cd).reshape(step.shape)
            else:
                got = F.svd_quant(x.to(cd), quant_func=F.q_forward_input, metis_mode="mean", mean_cache=cache, cache_key="k")
                got_step = F.svd_quant(step.to(cd), quant_func=F.q_forward_input, metis_mode="mean", mean_cache=cache, cache_key="k")
            want, want_step = t(g[f"mean_out_{tag}"]), t(g[f"mean_step_out_{tag}"])
            # the column mean is summed in another order than torch's CPU reduction; a last-bit difference of the mean
            # shifts every output by that much (and can move single codes), so the comparison is a tolerance: a few
            # binary32 ulps, or one bf16 ulp of the mean in bf16 arithmetic
            tol = 1e-6 if cd == torch.float32 else 4e-3
            assert rel_fro(got.cpu().float(), want.float()) <= tol, path
            assert rel_fro(got_step.cpu().float(), want_step.float()) <= tol, path
            assert cache["k"][1] == int(g[f"mean_step_count_{tag}"][0])
            torch.testing.assert_close(cache["k"][0].cpu().float().reshape(-1), t(g[f"mean_step_cache_{tag}"]).float().reshape(-1),
                                       rtol=1e-6 if cd == torch.float32 else 2 ** -7, atol=1e-7)
    finally:
        F.compute_dtype, F.enable_activation_svd, F.metis_mode, F.tp_simulate, F.enable_nv_recipe, F.q_forward_input = keep


def test_mean_mode_operands_in_bf16_arithmetic_hold_the_reference_tensor():
    """bf16 arithmetic: the reference multiplies with ONE bf16 tensor, me + QDQ(x - me) with the sum rounded to bf16.
    The tiled operand (prefill) and the ready decode operand built from the packed centred residual and the bf16 mean
    hold exactly that tensor: against the reference's own svd_quant output for the mean it computed, and bit for bit
    against the sum formed by torch from the same packed residual on larger shapes."""
    from helpers import from_decode_operand, t, untile
    from metis_hip import ops
    g = _mean_golden()
    x = t(g["mean_x"]).cuda().reshape(-1, 64)
    me = t(g["mean_cache_pb16"]).cuda().reshape(-1)                   # the reference's own bf16 mean of these tokens
    assert me.dtype == torch.bfloat16
    p = ops.quantize(x, 1, center=me)
    got = untile(ops.expand_tiled(p, cache=False, mode=1, center=me), x.shape[0], 64, torch.bfloat16)
    assert torch.equal(got.cpu(), t(g["mean_out_pb16"]).reshape(-1, 64))
    gen = torch.Generator().manual_seed(77)
    for rows, cols in ((300, 512), (64, 3584), (17, 256), (200, 1024)):
        xx = _offset_activation(rows + cols, rows, cols).cuda()
        mm = ops.column_mean(xx, torch.bfloat16)
        pp = ops.quantize(xx, 1, center=mm)
        want = mm.unsqueeze(0) + ops.dequantize(pp, torch.bfloat16)                  # bf16 add: the reference's expression
        assert torch.equal(untile(ops.expand_tiled(pp, cache=False, mode=1, center=mm), rows, cols, torch.bfloat16), want)
        # the same operands from a quantizer call that deferred its scale bytes (the consumers form them)
        lazy = ops.quantize(xx, 1, center=mm, deferred=True)
        assert lazy.deferred is not None and torch.equal(lazy.codes, pp.codes)
        assert torch.equal(untile(ops.expand_tiled(lazy, cache=False, mode=1, center=mm), rows, cols, torch.bfloat16), want)
        assert lazy.__dict__.get("_scales") is None and float(lazy.unit.cpu()) == float(pp.unit.cpu())
        if rows < 256:
            lazy = ops.quantize(xx, 1, center=mm, deferred=True)
            assert torch.equal(from_decode_operand(ops.decode_operand(lazy, 1, mm), rows, cols, torch.bfloat16), want)
            assert lazy.__dict__.get("_scales") is None and float(lazy.unit.cpu()) == float(pp.unit.cpu())
            assert torch.equal(lazy.scales, pp.scales)
            lazy0 = ops.quantize(xx, 0, deferred=True)
            assert torch.equal(from_decode_operand(ops.decode_operand(lazy0, 0), rows, cols, torch.float16), ops.expand(ops.quantize(xx, 0)))
            assert torch.equal(from_decode_operand(ops.decode_operand(pp, 1, mm), rows, cols, torch.bfloat16), want)
            assert torch.equal(from_decode_operand(ops.decode_operand(pp, 1), rows, cols, torch.bfloat16), ops.dequantize(pp, torch.bfloat16))
            exact = from_decode_operand(ops.decode_operand(pp, 0), rows, cols, torch.float16)
            assert torch.equal(exact, ops.expand(pp))


@pytest.mark.parametrize("L", [64, 512])
def test_mean_mode_forward_in_bf16_arithmetic_follows_the_all_bf16_evaluation(L):
    """The reference's default arguments under the GRPO caller's dtypes (mean mode, bf16 storage and arithmetic): the
    fused BitLinear forward against the oracle's evaluation in that arithmetic -- X^ = me + QDQ(x - me) as one bf16
    tensor, the residual product and the bias add rounded to bf16, the rank-r branch added before the final rounding --
    within the GEMM tolerance at decode and prefill sizes.  (Exact products with a separate binary32 mean term sit
    2-5e-3 from it.)"""
    from oracle import metis_oracle as O
    from metis_hip import BitLinear, LinearLowbitFunction as F, MetisArgs
    K, N, r = 1024, 768, 32
    g = torch.Generator().manual_seed(9)
    names = ("q_forward_input", "q_forward_weight", "q_backward_input", "q_backward_weight", "q_backward_outputgrad",
             "enable_backward_svd", "enable_activation_svd", "enable_nv_recipe", "compute_dtype", "metis_mode", "backward_lowrank_svd")
    saved = {k: getattr(F, k) for k in names}
    try:
        _mean_forward_bf16(L, K, N, r, g)
    finally:
        for k, val in saved.items():
            setattr(F, k, val)


def _mean_forward_bf16(L, K, N, r, g):
    from oracle import metis_oracle as O
    from metis_hip import BitLinear, LinearLowbitFunction as F, MetisArgs
    layer = BitLinear(K, N, args=MetisArgs(forward_svd_rank=r), bias=True, dtype=torch.bfloat16, compute_dtype=torch.bfloat16).cuda()
    with torch.no_grad():
        w = torch.randn(N, K, generator=g) * 0.02 + (torch.linalg.qr(torch.randn(N, 8, generator=g))[0] * 3.0) @ torch.linalg.qr(torch.randn(K, 8, generator=g))[0].T
        layer.warmup_linear.weight.copy_(w)
        layer.warmup_linear.bias.copy_(torch.randn(N, generator=g) * 0.1)
    layer.split()
    assert F.metis_mode == "mean" and F.enable_activation_svd and F.compute_dtype == torch.bfloat16
    x = _offset_activation(5, L, K)
    with torch.no_grad():
        y = layer(x.cuda().reshape(1, L, K)).reshape(L, N).cpu()
    want = O.metis_forward(x, layer.vlinear.weight.detach().cpu(), layer.s.detach().cpu(), layer.ulinear.weight.detach().cpu(),
                           layer.warmup_linear.weight.detach().cpu(), layer.warmup_linear.bias.detach().cpu(), p32=False, mean_mode=True)
    err = rel_fro(y.float(), want.float())
    assert err <= 3e-4, err                                         # tolerance of the task: 2e-3; measured 3e-5


def test_mean_mode_linear_against_reference_vectors(monkeypatch):
    """LinearLowbit with the mean mode on for activations and output gradients, round-to-nearest quantizers everywhere:
    forward against the reference's output on both paths; backward of the generic path (which follows the reference's
    operand choice: dY blocked along its last dimension, the saved forward activation) against the reference's gradients."""
    from helpers import t
    from metis_hip import BitLinear, LinearLowbitFunction as F, MetisArgs, quant_func
    g = _mean_golden()
    x, w, b, dy = (t(g[k]) for k in ("mean_lin_x", "mean_lin_w", "mean_lin_b", "mean_lin_dy"))
    args = MetisArgs(cache_quantized_weight=False)
    args.enable_forward_svd = False
    args.q_backward_input = args.q_backward_weight = args.q_backward_outputgrad = "nvfp4e2m1bnosr"
    lin = BitLinear(64, 48, args=args, bias=True, dtype=torch.float32, compute_dtype=torch.float32).cuda().warmup_linear
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    y = lin(x.cuda())                                             # packed path
    assert rel_fro(y.detach().cpu(), t(g["mean_lin_y"])) <= 1e-5
    monkeypatch.setattr(F, "_mean_mode_packable", staticmethod(lambda: False))
    xr = x.cuda().requires_grad_(True)
    y2 = lin(xr)                                                  # generic path
    assert rel_fro(y2.detach().cpu(), t(g["mean_lin_y"])) <= 1e-5
    y2.backward(dy.cuda())
    assert rel_fro(xr.grad.cpu(), t(g["mean_lin_gx"])) <= 1e-5
    assert rel_fro(lin.weight.grad.cpu(), t(g["mean_lin_gw"])) <= 1e-5
    assert rel_fro(lin.bias.grad.cpu(), t(g["mean_lin_gb"])) <= 1e-5
