"""GPU tests of the drop-in Python surface: registry classes against the reference's golden vectors
(bit-exact), LinearLowbit / BitLinear forward against the oracle (<= 2e-3 relative Frobenius, P32),
backward wiring, and patching of a Hugging Face Qwen2 decoder layer."""
import pytest
import torch

from helpers import rel_fro, same_bits, synthetic_activation, t

pytestmark = pytest.mark.gpu

TOL = 2e-3


@pytest.fixture(autouse=True)
def _config():
    from metis_hip import BitLinear, LinearLowbitFunction as F, quant_func
    F.q_forward_input = quant_func["nvfp4e2m1bnosr"]
    F.q_forward_weight = quant_func["nvfp4e2m1bnosr"]
    F.q_backward_input = quant_func["nvfp4e2m1b"]
    F.q_backward_weight = quant_func["nvfp4e2m1b"]
    F.q_backward_outputgrad = quant_func["nvfp4e2m1b"]
    F.enable_activation_svd = False
    F.enable_backward_svd = False
    F.enable_nv_recipe = False
    F.compute_dtype = torch.float32
    yield
    BitLinear.rollout_merge_active = False


@pytest.mark.parametrize("tag", ["p32", "pb16"])
def test_three_call_and_fused_against_reference_golden(golden, tag):
    from metis_hip import quant_func
    q = quant_func["nvfp4e2m1bnosr"]
    xb = t(golden["rne_x"])
    x = (xb.float() if tag == "p32" else xb).cuda()
    s = q.get_scalar(x)
    assert same_bits(s.cpu(), t(golden[f"rne_scalar_{tag}"]))
    xq = q.quant(x, s)
    assert same_bits(xq.cpu(), t(golden[f"rne_quant_{tag}"]))
    s_arg = s.clone()
    out = q.rquant(xq, s_arg)
    assert same_bits(out.cpu(), t(golden[f"rne_rquant_{tag}"]))
    assert same_bits(s_arg.cpu(), t(golden[f"rne_scalar_after_rquant_{tag}"]))      # in-place side effect
    fused = q.quantize_dequantize(x)
    assert same_bits(fused.cpu(), t(golden[f"rne_qdq_{tag}"])) and same_bits(fused.cpu(), out.cpu())
    x3 = t(golden["rne3d_x"])
    x3 = (x3.float() if tag == "p32" else x3).cuda()
    assert same_bits(q.quantize_dequantize(x3).cpu(), t(golden[f"rne3d_qdq_{tag}"]))


@pytest.mark.parametrize("tag", ["p32", "pb16"])
def test_stochastic_three_call_against_reference_golden(golden, tag):
    from metis_hip import quant_func
    q = quant_func["nvfp4e2m1b"]
    xb = t(golden["sr_x"])
    x = (xb.float() if tag == "p32" else xb).cuda()
    u = t(golden[f"sr_noise_{tag}"]).cuda()
    s = q.get_scalar(x)
    xq = q.quant(x, s, noise=u)
    assert same_bits(xq.cpu(), t(golden[f"sr_quant_{tag}"]))                        # incl. the off-grid +-8
    assert same_bits(q.rquant(xq, s.clone()).cpu(), t(golden[f"sr_rquant_{tag}"]))


def test_linear_lowbit_forward_backward_against_reference_golden(golden):
    """LinearLowbit (fp32 compute) on the reference's own input: forward within tolerance of its
    output; backward with the generic three-call path and the reference's recorded noise is exact
    up to the GEMM's summation order."""
    from types import SimpleNamespace
    from metis_hip import LinearLowbit, LinearLowbitFunction as F, quant_func
    x, w, b, dy = (t(golden[k]) for k in ("lin_x", "lin_w", "lin_b", "lin_dy"))
    args = SimpleNamespace(device="cuda", cache_quantized_weight=False)
    layer = LinearLowbit(64, 48, bias=True, args=args)
    with torch.no_grad():
        layer.weight.copy_(w)
        layer.bias.copy_(b)
    xr = x.cuda().requires_grad_(True)
    y = layer(xr)
    assert y.shape == (2, 16, 48) and y.dtype == torch.float32
    assert rel_fro(y.detach().cpu(), t(golden["lin_y"])) <= 1e-5
    y.backward(dy.cuda())
    # packed backward uses its own stochastic stream and token-blocked operands: FP4-noise level agreement
    assert rel_fro(xr.grad.cpu(), t(golden["lin_gx"])) < 0.2
    assert rel_fro(layer.weight.grad.cpu(), t(golden["lin_gw"])) < 0.35
    assert same_bits(layer.bias.grad.cpu(), t(golden["lin_gb"]))
    assert layer.weight.grad.dtype == torch.float32
    # reference-style backward: dY through the three-call SR quantizer with the reference's noise
    q = quant_func["nvfp4e2m1b"]
    dyd = dy.cuda()
    s = q.get_scalar(dyd)
    dyq = q.rquant(q.quant(dyd, s, noise=t(golden["lin_noise_dy"]).cuda()), s).reshape(-1, 48)
    xq = quant_func["nvfp4e2m1bnosr"].quantize_dequantize(x.cuda()).reshape(-1, 64)
    wq = quant_func["nvfp4e2m1bnosr"].quantize_dequantize(w.cuda())
    assert rel_fro((dyq.T @ xq).cpu(), t(golden["lin_gw"])) <= 1e-5
    assert rel_fro((dyq @ wq).reshape(2, 16, 64).cpu(), t(golden["lin_gx"])) <= 1e-5


def _make_bitlinear(K, N, r, bias, dtype, compute_dtype, seed=0):
    from metis_hip import BitLinear, MetisArgs
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(N, K, generator=g) * 0.02
    a = torch.linalg.qr(torch.randn(N, 8, generator=g))[0]
    b = torch.linalg.qr(torch.randn(K, 8, generator=g))[0]
    w = w + (a * 3.0) @ b.T
    args = MetisArgs.direct_fp4(forward_svd_rank=r)
    layer = BitLinear(K, N, args=args, bias=bias, dtype=dtype, compute_dtype=compute_dtype).cuda()
    with torch.no_grad():
        layer.warmup_linear.weight.copy_(w)
        if bias:
            layer.warmup_linear.bias.copy_(torch.randn(N, generator=g) * 0.1)
    layer.split()
    return layer, w


@pytest.mark.parametrize("bias", [False, True])
def test_bitlinear_fused_forward_against_oracle(bias):
    """P32 (compute_dtype=float32, the reference's default): <= 2e-3, bf16 vs bf16."""
    from oracle import metis_oracle as O
    K, N, r, L = 256, 192, 32, 128
    layer, w = _make_bitlinear(K, N, r, bias, torch.bfloat16, torch.float32)
    assert layer.is_svd_quant and layer.vlinear.weight.shape == (r, K)
    x = synthetic_activation(50, L, K).reshape(2, L // 2, K)
    y = layer(x.cuda())
    assert y.shape == (2, L // 2, N) and y.dtype == torch.float32
    want = O.metis_forward(x.reshape(L, K), layer.vlinear.weight.detach().cpu(), layer.s.detach().cpu(),
                           layer.ulinear.weight.detach().cpu(), layer.warmup_linear.weight.detach().cpu(),
                           None if not bias else layer.warmup_linear.bias.detach().cpu(), p32=True)
    assert rel_fro(y.detach().cpu().reshape(L, N).bfloat16(), want) <= TOL
    # and close to the unquantized layer it replaces (FP4 noise on the residual only)
    dense = x.reshape(L, K).float() @ w.T
    if bias:
        dense = dense + layer.warmup_linear.bias.detach().cpu().float()
    assert rel_fro(y.detach().cpu().reshape(L, N).float(), dense) < 0.05


def test_bitlinear_quantized_lowrank_branch_switch(monkeypatch):
    """BitLinear.quantized_lowrank_branch = True evaluates the reference's current formula, rank-r branch on
    Q(x) and Q(V) (bitlinear.py:752, 863-879), still on packed operands: <= 2e-3 against the oracle's variant."""
    from metis_hip import BitLinear
    from oracle import metis_oracle as O
    K, N, r, L = 256, 192, 32, 128
    layer, w = _make_bitlinear(K, N, r, True, torch.bfloat16, torch.float32)
    monkeypatch.setattr(BitLinear, "quantized_lowrank_branch", True)
    x = synthetic_activation(50, L, K).reshape(2, L // 2, K)
    y = layer(x.cuda())
    want = O.metis_forward(x.reshape(L, K), layer.vlinear.weight.detach().cpu(), layer.s.detach().cpu(),
                           layer.ulinear.weight.detach().cpu(), layer.warmup_linear.weight.detach().cpu(),
                           layer.warmup_linear.bias.detach().cpu(), p32=True, quantized_lowrank=True)
    assert rel_fro(y.detach().cpu().reshape(L, N).bfloat16(), want) <= TOL
    y.float().square().mean().backward()
    assert layer.vlinear.weight.grad is not None and layer.warmup_linear.weight.grad is not None


@pytest.mark.parametrize("L,bias", [(512, True), (1024, False), (128, True), (64, False), (16, True)])
def test_bitlinear_fused_forward_bf16_compute(L, bias):
    """compute_dtype=bfloat16, the configuration of the GRPO caller: operands are packed with the bf16-per-op arithmetic
    (bit-exact codes, see test_gpu_quant).  The GEMM multiplies the reference's own twice-rounded bf16 dequantized values
    and rounds the residual product and the bias add to bf16 as the reference's all-bf16 forward does -- the pipelined
    kernel from 256 rows on, the decode-sized kernel below: within 2e-3 of the oracle in that mode at every size."""
    from oracle import metis_oracle as O
    K, N, r = 256, 192, 32
    layer, w = _make_bitlinear(K, N, r, bias, torch.bfloat16, torch.bfloat16)
    x = synthetic_activation(50, L, K).reshape(2, L // 2, K)
    y = layer(x.cuda())
    assert y.dtype == torch.bfloat16
    want = O.metis_forward(x.reshape(L, K), layer.vlinear.weight.detach().cpu(), layer.s.detach().cpu(),
                           layer.ulinear.weight.detach().cpu(), layer.warmup_linear.weight.detach().cpu(),
                           None if not bias else layer.warmup_linear.bias.detach().cpu(), p32=False)
    err = rel_fro(y.detach().cpu().reshape(L, N), want)
    assert err <= 2e-3, err


def test_bitlinear_backward_reaches_every_parameter_and_matches_dense_gradients():
    K, N, r, L = 256, 192, 32, 128
    layer, w = _make_bitlinear(K, N, r, True, torch.bfloat16, torch.bfloat16, seed=3)
    x = synthetic_activation(51, L, K).reshape(2, L // 2, K).cuda().requires_grad_(True)
    g = torch.Generator().manual_seed(4)
    dy = (torch.randn(2, L // 2, N, generator=g) * 1e-2).bfloat16().cuda()
    layer(x).backward(dy)
    for p in (layer.vlinear.weight, layer.ulinear.weight, layer.s, layer.warmup_linear.weight, layer.warmup_linear.bias):
        assert p.grad is not None and bool(torch.isfinite(p.grad).all())
    # dense reference gradients of y = x W^T + b
    gx_dense = dy.reshape(L, N).float().cpu() @ w
    assert rel_fro(x.grad.reshape(L, K).float().cpu(), gx_dense) < 0.1
    gw_dense = dy.reshape(L, N).float().cpu().T @ x.detach().reshape(L, K).float().cpu()
    assert rel_fro(layer.warmup_linear.weight.grad.float().cpu(), gw_dense) < 0.3      # both operands in FP4 with SR
    assert rel_fro(layer.ulinear.weight.grad.float().cpu(),
                   gw_dense @ (layer.vlinear.weight.detach().float().cpu().T * layer.s.detach().float().cpu())) < 0.05
    torch.testing.assert_close(layer.warmup_linear.bias.grad.float().cpu(), dy.reshape(L, N).float().sum(0).cpu(),
                               rtol=2e-2, atol=1e-3)


def test_shared_activation_is_quantized_once_per_group():
    from metis_hip import LinearLowbitFunction as F, quant_func
    calls = {"n": 0}
    base = quant_func["nvfp4e2m1bnosr"]
    orig = base.pack.__func__

    def counting(cls, x, col=False, noise=None, arith=None, **more):
        if not col and tuple(x.shape) == (96, 256):      # the activation, not the [N, 256] weights
            calls["n"] += 1
        return orig(cls, x, col, noise, arith, **more)

    base.pack = classmethod(counting)
    try:
        q, _ = _make_bitlinear(256, 128, 32, False, torch.bfloat16, torch.bfloat16, seed=5)
        k, _ = _make_bitlinear(256, 64, 32, False, torch.bfloat16, torch.bfloat16, seed=6)
        group = {"name": "l0.qkv", "mean_cache": {}, "input_ref": None, "quantized_input": None}
        q.activation_group = k.activation_group = group
        calls["n"] = 0
        x = synthetic_activation(52, 96, 256).cuda()
        q(x), k(x)
        assert calls["n"] == 1                       # one activation quantization for the group
        q(synthetic_activation(53, 96, 256).cuda())
        assert calls["n"] == 2
    finally:
        base.pack = classmethod(orig)


def test_rollout_switch_on_the_fused_path_and_merged_weight_helper():
    """The fused launch already evaluates both branches at once, so the rollout switch leaves the
    output unchanged; the merged-weight helper keeps the reference's definition
    (U diag s) Q(V) + Q(W_res) and its cache semantics (reference 704-730)."""
    from metis_hip import BitLinear
    layer, _ = _make_bitlinear(256, 128, 32, True, torch.bfloat16, torch.float32, seed=7)
    x = synthetic_activation(54, 64, 256).float().cuda()
    with torch.no_grad():
        BitLinear.rollout_merge_active = False
        expected = layer(x)
        BitLinear.rollout_merge_active = True
        actual = layer(x)
        first = layer._get_merged_rollout_weight(torch.float32)
        second = layer._get_merged_rollout_weight(torch.float32)
        from metis_hip import quant_func
        q = quant_func["nvfp4e2m1bnosr"]
        want = (layer.ulinear.weight.float() * layer.s.float()) @ q.quantize_dequantize(layer.vlinear.weight.float()) \
            + q.quantize_dequantize(layer.warmup_linear.weight.float())
        layer.s.add_(0.1)
        updated = layer._get_merged_rollout_weight(torch.float32)
    assert torch.equal(actual, expected)
    assert first is second and updated is not first
    assert rel_fro(first.cpu(), want.cpu()) < 1e-6


def test_rollout_merged_weight_against_reference_vectors():
    """The merged rollout weight (U diag s) Q(V) + Q(W_res) and the one-matmul forward that uses it, against what the
    reference computed for the same hand-assembled layer (binary32 arithmetic): the two quantized weights are bit-exact,
    so only the order of the binary32 sums in the small products differs."""
    import os
    import numpy as np
    from metis_hip import BitLinear, LinearLowbit, MetisArgs
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_rollout.npz"))
    x, b = t(z["ro_x"]), t(z["ro_b"])
    v, u, s, res = t(z["ro_v"]), t(z["ro_u"]), t(z["ro_s"]), t(z["ro_res"])
    r, K = v.shape
    N = u.shape[0]
    args = MetisArgs.direct_fp4(forward_svd_rank=r)
    layer = BitLinear(K, N, args=args, bias=True, dtype=torch.float32, compute_dtype=torch.float32).cuda()
    layer.warmup_linear = LinearLowbit(K, N, bias=True, args=args, device="cuda")
    layer.vlinear = LinearLowbit(K, r, bias=False, args=args, device="cuda")
    layer.ulinear = torch.nn.Linear(r, N, bias=False, device="cuda")
    with torch.no_grad():
        layer.vlinear.weight.copy_(v)
        layer.ulinear.weight.copy_(u)
        layer.s = torch.nn.Parameter(s.clone().cuda())
        layer.warmup_linear.weight.copy_(res)
        layer.warmup_linear.bias.copy_(b)
    layer.is_svd_quant = True
    with torch.no_grad():
        merged = layer._get_merged_rollout_weight(torch.float32)
        assert rel_fro(merged.cpu(), t(z["ro_merged_weight"])) <= 1e-6
        # the reference's current file feeds the rank-r branch the quantized activation and the quantized V; with that
        # variant selected the rollout switch takes the merged-weight matmul exactly as the reference does
        BitLinear.quantized_lowrank_branch = True
        try:
            three = layer(x.cuda())
            BitLinear.rollout_merge_active = True
            one = layer(x.cuda())
        finally:
            BitLinear.rollout_merge_active = False
            BitLinear.quantized_lowrank_branch = False
    assert rel_fro(one.cpu(), t(z["ro_y_merged"])) <= 1e-5
    assert rel_fro(three.cpu(), t(z["ro_y_three_gemm"])) <= 1e-5


def test_rollout_in_bf16_arithmetic_runs_on_the_tiled_gemm_against_reference_vectors():
    """The rollout shortcut as GRPO runs it (bf16 tensors, bf16 arithmetic, rank 32, 256 tokens): the merged weight's
    rank-r product and the one-matmul forward run on the tiled GEMM with bf16 operands (no torch matmul), rounding
    where the reference's bf16 ops round.  Against vectors the reference wrote: the merged weight to a bf16 ulp of its
    largest entries, the output within 2e-3."""
    import os
    import numpy as np
    from metis_hip import BitLinear, LinearLowbit, LinearLowbitFunction as F, MetisArgs, ops
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_rollout_bf16.npz"))
    x, b = t(z["ro16_x"]), t(z["ro16_b"])
    v, u, s, res = t(z["ro16_v"]), t(z["ro16_u"]), t(z["ro16_s"]), t(z["ro16_res"])
    r, K = v.shape
    N = u.shape[0]
    dt = torch.bfloat16
    args = MetisArgs.direct_fp4(forward_svd_rank=r)
    args.cache_quantized_weight = True
    F.compute_dtype = dt
    layer = BitLinear(K, N, args=args, bias=True, dtype=dt, compute_dtype=dt).cuda()
    layer.warmup_linear = LinearLowbit(K, N, bias=True, args=args, device="cuda", storage_dtype=dt, compute_dtype=dt)
    layer.vlinear = LinearLowbit(K, r, bias=False, args=args, device="cuda", storage_dtype=dt, compute_dtype=dt)
    layer.ulinear = torch.nn.Linear(r, N, bias=False, device="cuda", dtype=dt)
    with torch.no_grad():
        layer.vlinear.weight.copy_(v)
        layer.ulinear.weight.copy_(u)
        layer.s = torch.nn.Parameter(s.clone().cuda())
        layer.warmup_linear.weight.copy_(res)
        layer.warmup_linear.bias.copy_(b)
    layer.is_svd_quant = True
    calls = []
    real, real_mm = ops.gemm_tiled, torch.matmul
    ops.gemm_tiled = lambda *a, **k: (calls.append("tiled"), real(*a, **k))[1]
    torch.matmul = lambda *a, **k: (calls.append("torch"), real_mm(*a, **k))[1]
    # the reference's current file feeds the rank-r branch the quantized activation and the quantized V; with that variant
    # selected the rollout switch takes the merged-weight matmul exactly as the reference does
    BitLinear.quantized_lowrank_branch = True
    try:
        with torch.no_grad():
            BitLinear.rollout_merge_active = True
            y = layer(x.cuda())
            y2 = layer(x.cuda())
            merged = layer._get_merged_rollout_weight(dt)
    finally:
        ops.gemm_tiled, torch.matmul = real, real_mm
        BitLinear.rollout_merge_active = False
        BitLinear.quantized_lowrank_branch = False
        F.compute_dtype = torch.float32
    assert layer._merged_rollout_tiled is not None
    assert calls == ["tiled", "tiled", "tiled"]                 # merged weight once (cached), one GEMM per forward
    want_w = t(z["ro16_merged_weight"]).float()
    assert float((merged.float().cpu() - want_w).abs().max()) <= float(want_w.abs().max()) * 2.0 ** -8
    assert rel_fro(merged.float().cpu(), want_w) <= 2e-3
    assert y.dtype == dt and torch.equal(y, y2)
    assert rel_fro(y.float().cpu(), t(z["ro16_y_merged"]).float()) <= 2e-3


def test_packed_weight_cache_reuses_then_invalidates_on_the_device():
    """The weight cache holds the PACKED weight (and what hangs off it: the column-blocked packing for dgrad, the tiled
    expansion of the pipelined GEMM), keyed on Parameter._version as the reference keys its dequantized cache
    (reference test_weight_cache_reuses_then_invalidates): one quantization before an update, a second one after
    `weight.add_`, with fresh derived layouts and a different result."""
    from metis_hip import LinearLowbit, MetisArgs, ops, quant_func
    from metis_hip.ops import PackedNVFP4
    args = MetisArgs.direct_fp4()
    lin = LinearLowbit(512, 512, bias=False, args=args, device="cuda", storage_dtype=torch.bfloat16, compute_dtype=torch.float32)
    x = synthetic_activation(91, 512, 512).cuda().requires_grad_(True)
    base = quant_func["nvfp4e2m1bnosr"]
    orig = base.pack.__func__
    packs = []

    def spy(cls, t_, col=False, noise=None, arith=None, center=None, **more):
        packs.append((tuple(t_.shape), bool(col)))
        return orig(cls, t_, col, noise, arith, center, **more)

    base.pack = classmethod(spy)
    try:
        y1 = lin(x)
        first = lin._quantized_weight_cache[1]
        assert isinstance(first, PackedNVFP4) and first.persistent
        y1.sum().backward()
        assert first.transposed is not None                       # dgrad packed the weight column-blocked, once
        assert first.tiled is not None                            # 512 rows: the pipelined GEMM kept its expansion
        n_weight_packs = sum(1 for shp, _ in packs if shp == (512, 512))
        y2 = lin(x)
        y2.sum().backward()
        assert lin._quantized_weight_cache[1] is first
        # the second step packed activations only: x row-wise, nothing of the weight (dgrad operands are not this class)
        assert sum(1 for shp, _ in packs if shp == (512, 512)) == n_weight_packs + 1
        assert torch.equal(y1, y2)
        with torch.no_grad():
            lin.weight.add_(0.01)
        y3 = lin(x)
        second = lin._quantized_weight_cache[1]
        assert second is not first and second.transposed is None                 # no backward yet on the new packing
        assert second.tiled is not None and second.tiled is not first.tiled       # this forward made its own expansion
        assert not torch.equal(y3, y1)
        want = ops.dequantize(ops.quantize(x.detach()), torch.float32).double() @ ops.dequantize(second, torch.float32).double().T
        assert rel_fro(y3.detach().cpu(), want.cpu()) <= 1e-5
    finally:
        base.pack = classmethod(orig)


def test_patch_qwen2_decoder_layer():
    """A randomly initialised Hugging Face Qwen2 decoder layer with every projection replaced."""
    transformers = pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import BitLinear, MetisArgs, replace_model_with_metis
    torch.manual_seed(0)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
    holder = torch.nn.ModuleDict({"layer": layer})
    x = torch.randn(2, 64, 256, device="cuda", dtype=torch.bfloat16)
    pos = torch.arange(64, device="cuda").unsqueeze(0).expand(2, -1)
    rope = Qwen2RotaryEmbedding(cfg).cuda()
    pe = rope(x, pos)

    def run(m, inp):
        out = m(inp, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return out[0] if isinstance(out, tuple) else out

    with torch.no_grad():
        ref = run(layer, x)
    replace_model_with_metis(holder, MetisArgs.direct_fp4(forward_svd_rank=32))
    names = [n for n, m in holder.named_modules() if isinstance(m, BitLinear)]
    assert len(names) == 7
    attn = holder["layer"].self_attn
    assert attn.q_proj.activation_group is attn.k_proj.activation_group is attn.v_proj.activation_group
    xr = x.clone().requires_grad_(True)
    out = run(holder["layer"], xr)
    assert out.shape == ref.shape and bool(torch.isfinite(out).all())
    assert rel_fro(out.detach().float().cpu(), ref.float().cpu()) < 0.1
    out.float().square().mean().backward()
    assert xr.grad is not None and bool(torch.isfinite(xr.grad).all())
    assert attn.q_proj.warmup_linear.weight.grad is not None


def test_nv_recipe_against_reference_vectors():
    """NV recipe (tiled random Hadamard rotation around the wgrad operands and the weight QDQ), all
    quantizers round-to-nearest: rotated wgrad operand, LinearLowbit forward and both gradients against
    what the reference computed on CPU.  The rotation is a 16-term binary32 GEMM whose summation order
    differs between devices, so an element now and then lands on the other side of an FP4 rounding
    boundary: agreement is checked in the Frobenius norm and as a fraction of identical elements."""
    import os
    from types import SimpleNamespace

    import numpy as np

    from metis_hip import LinearLowbit, LinearLowbitFunction as F, quant_func
    g = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_hadamard.npz")))
    nosr = quant_func["nvfp4e2m1bnosr"]
    F.q_backward_input = F.q_backward_weight = F.q_backward_outputgrad = nosr
    F.hadamard_tile_size, F.hadamard_backend = 16, "torch_gemm"
    F.enable_nv_recipe = True
    try:
        x = t(g["had_x"]).cuda()
        torch.testing.assert_close(F._apply_hadamard_blocks(x).cpu(), t(g["had_fwd"]), rtol=1e-6, atol=1e-6)
        got = F._quantize_wgrad_operand(x.clone(), nosr).cpu()
        want = t(g["had_wgrad_operand_p32"])
        assert rel_fro(got, want) <= 2e-2
        assert float((got - want).abs().le(1e-6).float().mean()) > 0.9

        layer = LinearLowbit(64, 48, bias=False, args=SimpleNamespace(device="cuda", cache_quantized_weight=False))
        with torch.no_grad():
            layer.weight.copy_(t(g["had_lin_w"]))
        xr = t(g["had_lin_x"]).cuda().requires_grad_(True)
        y = layer(xr)
        y.backward(t(g["had_lin_dy"]).cuda())
        assert rel_fro(y.detach().cpu(), t(g["had_lin_y"])) <= 2e-2
        assert rel_fro(xr.grad.cpu(), t(g["had_lin_gx"])) <= 2e-2
        assert rel_fro(layer.weight.grad.cpu(), t(g["had_lin_gw"])) <= 2e-2
        assert layer.weight.grad.dtype == torch.float32
    finally:
        F.enable_nv_recipe = False


def test_svd_activation_mode_beats_plain_quantization_on_low_rank_plus_noise():
    """metis_mode="svd" (reference bitlinear.py:243-309): the dominant low-rank part is carried by
    quantized factors with S in high precision and only the residual sees FP4, so on an input with a
    strong rank-16 component the error is well below that of quantizing the input directly."""
    from metis_hip import LinearLowbitFunction as F, quant_func
    q = quant_func["nvfp4e2m1bnosr"]
    g = torch.Generator().manual_seed(9)
    a = torch.linalg.qr(torch.randn(512, 16, generator=g))[0]
    b = torch.linalg.qr(torch.randn(256, 16, generator=g))[0]
    x = ((a * (40.0 * 0.8 ** torch.arange(16))) @ b.T + 0.05 * torch.randn(512, 256, generator=g)).cuda()
    torch.manual_seed(10)                                       # svd_lowrank draws its test matrix from the global stream
    out = F.svd_quant(x, q, rank=16, niter=2, metis_mode="svd")
    plain = q.quantize_dequantize(x)
    assert out.shape == x.shape and out.dtype == x.dtype
    e_svd, e_plain = rel_fro(out.cpu(), x.cpu()), rel_fro(plain.cpu(), x.cpu())
    assert e_svd < 0.5 * e_plain, (e_svd, e_plain)
    out3 = F.svd_quant(x.reshape(2, 256, 256), q, rank=16, niter=2, tp_simulate=True, tp_parts=2, metis_mode="svd")
    assert out3.shape == (2, 256, 256) and rel_fro(out3.cpu().reshape(512, 256), x.cpu()) < e_plain


def test_hot_path_replays_from_a_captured_graph():
    """Serving loops capture quantize -> GEMM once and replay it: the library launches only kernels (no
    memset nodes, no allocation, no synchronisation), so every replay on fresh input contents must equal
    the eager result bit for bit."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(12)
    w = (torch.randn(384, 512, generator=g) * 0.02).bfloat16().cuda()
    pw = ops.quantize(w)
    x_static = torch.zeros(64, 512, dtype=torch.bfloat16, device="cuda")
    gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16().cuda()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        _, p = ops.rmsnorm_quantize(x_static, gamma, 1e-6)     # warm-up allocates the stream's workspace
        ops.linear_fwd(p, pw)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            normed, p = ops.rmsnorm_quantize(x_static, gamma, 1e-6)
            y_static = ops.linear_fwd(p, pw)
    for seed in (21, 22, 23):
        x = synthetic_activation(seed, 64, 512).cuda()
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        got, got_normed = y_static.clone(), normed.clone()
        want_normed, pe = ops.rmsnorm_quantize(x, gamma, 1e-6)    # eager work between replays
        want = ops.linear_fwd(pe, pw)
        torch.cuda.synchronize()
        assert torch.equal(got_normed, want_normed), seed
        assert torch.equal(got, want), seed


def test_decode_path_replays_from_a_captured_graph():
    """The decode-sized chain (column mean with running update, centred quantizer, rank-r projection, grouped GEMM with
    K split through scratch taken from the allocator inside the capture, centre inside the launch) captured once and
    replayed on fresh inputs, with eager work between the replays: every replay equals the eager result bit for bit."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(14)
    M, K, r = 8, 8192, 32
    pws = [ops.quantize((torch.randn(n, K, generator=g) * 0.02).bfloat16().cuda()) for n in (64, 36)]
    us = [(torch.randn(n, r, generator=g) * 0.1).bfloat16().cuda() for n in (64, 36)]
    v = (torch.randn(2 * r, K, generator=g) / K ** 0.5).bfloat16().cuda()
    sv = torch.rand(2 * r, generator=g).bfloat16().cuda()
    bias = torch.randn(64, generator=g).cuda()
    cached = (torch.randn(K, generator=g) * 0.1).cuda()
    x_static = torch.zeros(M, K, dtype=torch.bfloat16, device="cuda")

    def chain(x):
        me, me32 = ops.column_mean_running(x, cached, 40, torch.float32)
        px = ops.quantize(x, 0, center=me)
        _, t = ops.lowrank_project(x, v, sv)
        members = [(pws[0], t[:, :r], us[0], bias), (pws[1], t[:, r:], us[1], None)]
        return ops.linear_fwd_grouped(px, members, out_dtype=torch.float32, center=me32)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        chain(x_static)                                          # warm-up allocates the stream's workspace
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs_static = chain(x_static)
    for seed in (31, 32, 33):
        x = (synthetic_activation(seed, M, K).float() + 0.5).bfloat16().cuda()
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs_static]
        want = chain(x)                                          # eager work between replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), seed


def test_compile_flag_is_accepted_and_changes_nothing():
    """Reference tests/test_metis_quant_cache.py:30-42: the flag that selects the torch.compile'd QDQ there
    selects the same kernel here; results are identical at atol 0 and the status helper says so."""
    from metis_hip import nvfp4_nosr_qdq_compile_status, quant_func
    q = quant_func["nvfp4e2m1bnosr"]
    x = synthetic_activation(90, 8 * 16, 128).reshape(8, 16, 128).cuda()
    q.compile_quantize_dequantize = False
    expected = q.quantize_dequantize(x)
    q.compile_quantize_dequantize = True
    try:
        actual = q.quantize_dequantize(x)
    finally:
        q.compile_quantize_dequantize = False
    assert same_bits(actual, expected)
    assert nvfp4_nosr_qdq_compile_status() == "validated"


def test_fused_rmsnorm_feeds_the_projection_groups_of_a_qwen2_layer():
    """The RMSNorm in front of {q,k,v} and {gate,up} is replaced by the fused norm+quant module: the
    groups find their packed activation already cached (no quantizer launch for the normed tensors),
    the layer output and the gradients agree with the unfused patched layer, and norm weights get
    gradients."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import FusedRMSNormQuant, MetisArgs, fuse_rmsnorm_into_groups, quant_func, replace_model_with_metis
    torch.manual_seed(0)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
        else:
            torch.nn.init.normal_(p, mean=1.0, std=0.1)
    holder = torch.nn.ModuleDict({"layer": layer})
    replace_model_with_metis(holder, MetisArgs.direct_fp4(forward_svd_rank=32))
    x = torch.randn(2, 64, 256, device="cuda", dtype=torch.bfloat16)
    pos = torch.arange(64, device="cuda").unsqueeze(0).expand(2, -1)
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)

    def run(inp):
        out = holder["layer"](inp, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return out[0] if isinstance(out, tuple) else out

    def grads():
        xr = x.clone().requires_grad_(True)
        for p in holder.parameters():
            p.grad = None
        out = run(xr)
        out.float().square().mean().backward()
        lyr = holder["layer"]
        return (out.detach().float().cpu(), xr.grad.float().cpu(), lyr.input_layernorm.weight.grad.float().cpu(),
                lyr.post_attention_layernorm.weight.grad.float().cpu())

    plain = grads()
    assert fuse_rmsnorm_into_groups(holder) == 2
    lyr = holder["layer"]
    assert isinstance(lyr.input_layernorm, FusedRMSNormQuant) and isinstance(lyr.post_attention_layernorm, FusedRMSNormQuant)
    assert lyr.input_layernorm.group is lyr.self_attn.q_proj.activation_group
    assert lyr.post_attention_layernorm.group is lyr.mlp.gate_proj.activation_group
    assert fuse_rmsnorm_into_groups(holder) == 0                       # idempotent
    fused = grads()
    assert rel_fro(fused[0], plain[0]) < 2e-2                              # a bf16 ulp of the norm here and there
    assert rel_fro(fused[1], plain[1]) < 0.25                              # backward re-draws its stochastic rounding
    assert rel_fro(fused[2], plain[2]) < 0.25 and rel_fro(fused[3], plain[3]) < 0.25
    # the normed tensors are never quantized by the projections: only o_proj's and down_proj's inputs are
    base = quant_func["nvfp4e2m1bnosr"]
    orig = base.pack.__func__
    seen = []

    def spy(cls, t_, col=False, noise=None, arith=None, **more):
        if not col:
            seen.append(tuple(t_.shape))
        return orig(cls, t_, col, noise, arith, **more)

    # (a decode-sized activation that no sibling shares is quantized by the launch that also starts its projection)
    from metis_hip import ops
    orig_qpd = ops.quantize_project_decode

    def spy_qpd(x2, *a, **k):
        seen.append(tuple(x2.shape))
        return orig_qpd(x2, *a, **k)

    base.pack = classmethod(spy)
    ops.quantize_project_decode = spy_qpd
    try:
        with torch.no_grad():
            run(x)
    finally:
        base.pack = classmethod(orig)
        ops.quantize_project_decode = orig_qpd
    # q/k/v and gate/up inputs came packed from the norms: the only row quantizations left are o_proj's input
    # (attention output, also [128, 256]) and down_proj's (the MLP activation)
    assert sorted(seen) == [(128, 256), (128, 512)], seen


@pytest.mark.parametrize("mean_mode", [False, True])
def test_projection_groups_run_as_one_launch_without_autograd(mean_mode, monkeypatch):
    """Decode-sized batch through a patched Qwen2 decoder layer with autograd off: q/k/v and gate/up each take one
    grouped GEMM call (the first member evaluates the group, its siblings pick their results up), o and down one
    plain call each; the layer output equals the member-by-member evaluation up to bf16 roundings of the stacked
    rank-r product."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import BitLinear, MetisArgs, ops, replace_model_with_metis
    torch.manual_seed(0)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
    holder = torch.nn.ModuleDict({"layer": layer})
    args = MetisArgs(forward_svd_rank=32, cache_quantized_weight=True) if mean_mode else MetisArgs.direct_fp4(forward_svd_rank=32)
    replace_model_with_metis(holder, args)
    x = (torch.randn(64, 1, 256, device="cuda") + 0.5).bfloat16()
    pos = torch.zeros(64, 1, dtype=torch.long, device="cuda")
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)

    def run():
        with torch.no_grad():
            out = holder["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return out[0] if isinstance(out, tuple) else out

    def reset_means():
        for m in holder.modules():
            if isinstance(m, BitLinear):
                m.mean_cache.clear()
                if m.activation_group is not None:
                    m.activation_group["mean_cache"].clear()

    calls = {"grouped": 0, "plain": 0}
    real_g, real_p = ops.linear_fwd_grouped, ops.linear_fwd
    # a one-member call of the grouped entry (mean mode at decode size: the centre rides inside the launch) is a plain call
    def spy_grouped(a, members, *rest, **k):
        kind = "grouped" if len(members) > 1 else "plain"
        calls[kind] += 1
        return real_g(a, members, *rest, **k)
    monkeypatch.setattr(ops, "linear_fwd_grouped", spy_grouped)
    monkeypatch.setattr(ops, "linear_fwd", lambda *a, **k: (calls.__setitem__("plain", calls["plain"] + 1), real_p(*a, **k))[1])
    reset_means()
    got = run()
    assert calls == {"grouped": 2, "plain": 2}
    monkeypatch.setattr(BitLinear, "grouped_inference", False)
    calls.update(grouped=0, plain=0)
    reset_means()
    want = run()
    assert calls == {"grouped": 0, "plain": 7}
    assert rel_fro(got.float().cpu(), want.float().cpu()) <= 2e-3
    # with autograd on the group is evaluated member by member (each needs its own graph)
    monkeypatch.setattr(BitLinear, "grouped_inference", True)
    calls.update(grouped=0, plain=0)
    out = holder["layer"](x.clone().requires_grad_(True), position_embeddings=pe, attention_mask=None, position_ids=pos)
    assert calls["grouped"] == 0


def test_grouped_decode_sees_replaced_parameters():
    """The per-group caches of the decode path (stacked V and s of the members, converted biases, packed weights) key on
    the parameters' identity as well as their version: a member whose `s`, `vlinear.weight` or residual weight is
    REPLACED by a fresh Parameter with the same version counter changes the grouped result exactly as it changes the
    member-by-member evaluation."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import BitLinear, MetisArgs, replace_model_with_metis
    torch.manual_seed(0)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
    holder = torch.nn.ModuleDict({"layer": layer})
    replace_model_with_metis(holder, MetisArgs.direct_fp4(forward_svd_rank=32))
    x = (torch.randn(64, 1, 256, device="cuda") + 0.5).bfloat16()
    pos = torch.zeros(64, 1, dtype=torch.long, device="cuda")
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)

    def run():
        with torch.no_grad():
            out = holder["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return (out[0] if isinstance(out, tuple) else out).float().cpu()

    def same_version(old, new):
        with torch.no_grad():
            while new._version < old._version:
                new.add_(0.0)
        assert new._version == old._version
        return new

    base = run()
    gate = holder["layer"].mlp.gate_proj
    assert isinstance(gate, BitLinear)
    for name, owner in (("s", gate), ("weight", gate.vlinear), ("weight", gate.warmup_linear)):
        old = getattr(owner, name)
        fresh = same_version(old, torch.nn.Parameter((old.detach() * 1.5 + 0.01).clone()))
        setattr(owner, name, fresh)
        grouped = run()
        BitLinear.grouped_inference = False
        try:
            single = run()
        finally:
            BitLinear.grouped_inference = True
        assert not torch.equal(grouped, base), name
        assert rel_fro(grouped, single) <= 2e-3, name
        base = grouped


@pytest.mark.parametrize("compute", [torch.bfloat16, torch.float32])
def test_an_unshared_activation_is_quantized_and_projected_in_one_pass(compute, monkeypatch):
    """A BitLinear whose activation no sibling shares (o_proj, down_proj) quantizes it and forms x V^T in one kernel from
    256 rows on: same output and gradients as with the two separate passes, bit for bit in the forward (the packed
    activation and the projection are the same bytes)."""
    from metis_hip import BitLinear, ops
    layer, _ = _make_bitlinear(512, 384, 64, True, torch.bfloat16, compute, seed=41)
    x = synthetic_activation(77, 512, 512).reshape(4, 128, 512).cuda()
    calls = {"n": 0}
    orig = ops.quantize_project

    def counting(*a, **k):
        calls["n"] += 1
        return orig(*a, **k)

    monkeypatch.setattr(ops, "quantize_project", counting)

    def run():
        xi = x.clone().requires_grad_(True)
        for p_ in layer.parameters():
            p_.grad = None
        from metis_hip.quant import _NVFP4Base
        _NVFP4Base.sr_offset = 0                                      # the same stochastic draws in both runs
        y = layer(xi)
        y.backward(torch.ones_like(y) * 1e-2)
        return y.detach(), xi.grad, layer.vlinear.weight.grad.clone(), layer.warmup_linear.weight.grad.clone()

    fused = run()
    assert calls["n"] == 1
    monkeypatch.setattr(BitLinear, "_quantize_and_project", lambda self, x_: None)
    plain = run()
    assert calls["n"] == 1
    torch.cuda.synchronize()
    for a, b in zip(fused, plain):
        assert torch.equal(a, b)
    # fewer than 256 rows: the decode-sized kernels, no fused pass
    monkeypatch.undo()
    monkeypatch.setattr(ops, "quantize_project", counting)
    with torch.no_grad():
        layer(x[:1])
    assert calls["n"] == 1


def test_decode_step_in_bf16_arithmetic_never_writes_the_activation_scale_bytes(monkeypatch):
    """A decode-sized forward in bf16 arithmetic feeds the GEMM ready operands built straight from the codes and the parked
    block maxima: the quantizer's second launch (scale bytes of the row-major packing) must not run at all."""
    from metis_hip import ops
    layer, _ = _make_bitlinear(512, 768, 64, True, torch.bfloat16, torch.bfloat16, seed=43)
    x = synthetic_activation(78, 64, 512).reshape(64, 1, 512).cuda()
    calls = {"n": 0}
    orig = ops.PackedNVFP4._materialize

    def counting(self):
        calls["n"] += 1
        return orig(self)

    with torch.no_grad():
        want = layer(x)
    monkeypatch.setattr(ops.PackedNVFP4, "_materialize", counting)
    with torch.no_grad():
        got = layer(x)
    torch.cuda.synchronize()
    assert calls["n"] == 0
    assert torch.equal(got, want)


@pytest.mark.parametrize("mean_mode,fuse_norms,rows", [(False, True, 64), (False, False, 48), (True, False, 64), (False, True, 1)])
def test_merged_decode_launches_leave_the_layer_output_unchanged(mean_mode, fuse_norms, rows, monkeypatch):
    """The decode step of a patched Qwen2 layer with the small launches merged (the projection's finishing step inside
    the operand build, the projection's first step inside an unshared activation's quantizer launch) against the same
    step with the merged calls switched off: the same bits, and the merged calls are the ones that ran."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import BitLinear, MetisArgs, ops, replace_model_with_metis
    torch.manual_seed(3)
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
    holder = torch.nn.ModuleDict({"layer": layer})
    args = MetisArgs(forward_svd_rank=32, cache_quantized_weight=True) if mean_mode else MetisArgs.direct_fp4(forward_svd_rank=32)
    replace_model_with_metis(holder, args, fuse_norms=fuse_norms)
    x = (torch.randn(rows, 1, 256, device="cuda") + 0.5).bfloat16()
    pos = torch.zeros(rows, 1, dtype=torch.long, device="cuda")
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)

    def run():
        for m in holder.modules():
            if isinstance(m, BitLinear):
                m.mean_cache.clear()
                if m.activation_group is not None:
                    m.activation_group["mean_cache"].clear()
        with torch.no_grad():
            out = holder["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return out[0] if isinstance(out, tuple) else out

    seen = {"prepare": 0, "quant_project": 0}
    real_pao, real_qpd = ops.project_and_operand, ops.quantize_project_decode
    monkeypatch.setattr(ops, "project_and_operand", lambda *a, **k: (seen.__setitem__("prepare", seen["prepare"] + 1), real_pao(*a, **k))[1])
    monkeypatch.setattr(ops, "quantize_project_decode",
                        lambda *a, **k: (seen.__setitem__("quant_project", seen["quant_project"] + 1), real_qpd(*a, **k))[1])
    merged = run()
    # q/k/v, o, gate/up, down each prepare once; o and down quantize their own activation (direct mode only)
    assert seen == {"prepare": 4, "quant_project": 0 if mean_mode else 2}, seen
    monkeypatch.setattr(ops, "project_and_operand_applies", lambda *a, **k: False)
    monkeypatch.setattr(ops, "quantize_project_decode_applies", lambda *a, **k: False)
    seen.update(prepare=0, quant_project=0)
    separate = run()
    assert seen == {"prepare": 0, "quant_project": 0}
    assert torch.equal(merged, separate)
