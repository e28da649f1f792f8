"""GPU tests of the NV recipe (tiled random Hadamard rotation, reference bitlinear.py:75-211, 395-405, 495-501,
577-585) on the library's kernels: the rotation itself, rotation + quantizer in one pass, the tiled GEMM operands that
rotate a packed block back (plain and transposed), and LinearLowbit forward + both gradients against vectors the
reference wrote (tests/golden/metis_reference_hadamard*.npz)."""
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from helpers import rel_fro, same_bits, synthetic_activation, t

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(autouse=True)
def _config():
    from metis_hip import LinearLowbitFunction as F, quant_func
    nosr = quant_func["nvfp4e2m1bnosr"]
    F.q_forward_input = F.q_forward_weight = nosr
    F.q_backward_input = F.q_backward_weight = F.q_backward_outputgrad = nosr
    F.enable_activation_svd = False
    F.enable_backward_svd = False
    F.enable_nv_recipe = False
    F.hadamard_tile_size, F.hadamard_backend = 16, "auto"
    F.compute_dtype = torch.float32
    keep = F.reference_rounding
    yield
    F.enable_nv_recipe = False
    F.compute_dtype = torch.float32
    F.reference_rounding = keep


def _mask():
    from metis_hip import LinearLowbitFunction as F
    return F._hadamard_mask()


def _signs():
    m = _mask()
    return torch.tensor([-1.0 if (m >> j) & 1 else 1.0 for j in range(16)], dtype=torch.float64)


def _h16():
    h = torch.ones(1, 1, dtype=torch.float64)
    while h.shape[0] < 16:
        h = torch.cat((torch.cat((h, h), 1), torch.cat((h, -h), 1)), 0)
    return h


def _rot(x64, inverse=False):
    tiles = x64.reshape(-1, 16)
    out = (tiles @ _h16()) / 16 * _signs() if inverse else (tiles * _signs()) @ _h16()
    return out.reshape(x64.shape)


def test_rotation_kernel_against_reference_vectors_and_closed_form():
    from metis_hip import LinearLowbitFunction as F, ops
    g = dict(np.load(os.path.join(GOLDEN, "metis_reference_hadamard.npz")))
    assert torch.equal(F._get_hadamard_sign(16, torch.device("cpu"), torch.float32), t(g["had_sign16"]))
    x = t(g["had_x"]).cuda()
    torch.testing.assert_close(ops.hadamard16(x, _mask()).cpu(), t(g["had_fwd"]), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(ops.hadamard16(x, _mask(), inverse=True).cpu(), t(g["had_inv"]), rtol=1e-6, atol=1e-6)
    got = ops.hadamard16(x.bfloat16(), _mask()).cpu()
    want = t(g["had_fwd_bf16"])
    assert float((got.view(torch.int16).int() - want.view(torch.int16).int()).abs().max()) <= 1   # one rounding of a binary32 sum
    # the module's rotation now runs on that kernel
    F.hadamard_backend = "auto"
    assert torch.equal(F._apply_hadamard_blocks(x), ops.hadamard16(x, _mask()))
    # closed form on a larger tensor, and the round trip
    big = synthetic_activation(5, 300, 1024).cuda()
    rot = ops.hadamard16(big, _mask())
    want = _rot(big.double().cpu())
    assert float((rot.double().cpu() - want).abs().max()) <= float(want.abs().max()) * 2.0 ** -8
    f = big.float()
    back = ops.hadamard16(ops.hadamard16(f, _mask()), _mask(), inverse=True)
    torch.testing.assert_close(back, f, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("mode", [0, 1])
def test_rotation_and_quantizer_in_one_pass_equal_the_two_steps(mode):
    """quantize_rht(x) packs exactly what quantizing the rotated tensor packs: binary32 arithmetic quantizes the
    binary32 rotated values, bf16 arithmetic their bf16 roundings."""
    from metis_hip import ops
    x = synthetic_activation(21 + mode, 512, 1024).cuda()
    p = ops.quantize_rht(x, mode, _mask())
    if mode == 0:
        two = ops.quantize(ops.hadamard16(x.float(), _mask()), 0)          # binary32 input path
    else:
        two = ops.quantize(ops.hadamard16(x, _mask()), 1)
    assert torch.equal(p.codes, two.codes) and torch.equal(p.scales, two.scales) and torch.equal(p.unit, two.unit)
    assert p.rht == _mask()
    # dequantize() returns to the tensor's own domain: close to x, and equal to rotating the plain dequantization back
    plain = ops.PackedNVFP4(p.codes, p.scales, p.unit, p.rows, p.cols, p.mode)
    want = ops.hadamard16(plain.dequantize(torch.float32), _mask(), inverse=True)
    assert torch.equal(p.dequantize(torch.float32), want)
    assert rel_fro(p.dequantize(torch.float32).cpu(), x.float().cpu()) < 0.15
    # stochastic rounding on the library's stream: reproducible, and a different stream gives different codes
    a = ops.quantize_rht(x, mode, _mask(), sr=True, seed=7, offset=0)
    b = ops.quantize_rht(x, mode, _mask(), sr=True, seed=7, offset=0)
    c = ops.quantize_rht(x, mode, _mask(), sr=True, seed=8, offset=0)
    assert torch.equal(a.codes, b.codes) and not torch.equal(a.codes, c.codes)
    assert torch.equal(a.scales, p.scales) and torch.equal(a.unit, p.unit)


def test_wgrad_operand_against_reference_vector():
    """rot -> QDQ -> rot^-1 of the reference's test tensor (binary32 arithmetic, round to nearest)."""
    from metis_hip import ops
    g = dict(np.load(os.path.join(GOLDEN, "metis_reference_hadamard.npz")))
    x = t(g["had_x"]).cuda()
    got = ops.quantize_rht(x, 0, _mask()).dequantize(torch.float32).cpu()
    want = t(g["had_wgrad_operand_p32"])
    assert rel_fro(got, want) <= 1e-6
    assert float((got - want).abs().le(1e-6).float().mean()) == 1.0


@pytest.mark.parametrize("mode", [0, 1])
def test_tiled_operands_rotate_a_packed_block_back(mode):
    """GEMMs on the tiled expansions of a rotated packed tensor (plain and transposed) equal the product of its
    dequantized, rotated-back values: within the one binary16 rounding per operand element (2^-12) in binary32
    arithmetic, within the bf16 roundings of the reference's evaluation in bf16 arithmetic."""
    from metis_hip import ops
    L, N, K = 512, 384, 640
    a = synthetic_activation(31, L, K).cuda()
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(32)) * 0.05).bfloat16().cuda()
    pa = ops.quantize(a, mode)                                  # plain activation
    pw = ops.quantize_rht(w, mode, _mask())                     # rotated weight
    # dense references in the arithmetic's own dtype: in bf16 arithmetic the rotated-back values are bf16 tensors, and
    # the GEMM rounds its product to bf16 once more (2^-9 relative at worst)
    dt = torch.float32 if mode == 0 else torch.bfloat16
    da, dw = pa.dequantize(dt).double(), pw.dequantize(dt).double()
    tol = 2e-4 if mode == 0 else 2.5e-3
    # forward shape: A [L, K] . W~[N, K]^T
    y = ops.gemm_tiled(ops.expand_tiled(pa, cache=False, mode=mode), pa.unit, ops.expand_tiled(pw, cache=False, mode=mode), pw.unit,
                       L, N, K, mode=mode, out_dtype=torch.float32)
    assert rel_fro(y.double().cpu(), (da @ dw.T).cpu()) <= tol
    # the same through linear_fwd, which routes a rotated operand to the tiled kernel by itself
    y2 = ops.linear_fwd(pa, pw, out_dtype=torch.float32, reference_rounding=mode == 1)
    assert torch.equal(y2, y)
    # transposed operands: contraction over the packed tensors' rows.  dY~ [L, N] rotated, against W~^T [K, N] and X~^T
    dy = (torch.randn(L, N, generator=torch.Generator().manual_seed(33)) * 1e-3).bfloat16().cuda()
    pdy = ops.quantize_rht(dy, mode, _mask())
    px = ops.quantize_rht(a, mode, _mask())
    ddy, dx = pdy.dequantize(dt).double(), px.dequantize(dt).double()
    gx = ops.gemm_tiled(ops.expand_tiled(pdy, cache=False, mode=mode), pdy.unit, ops.expand_tiled_transposed(pw, mode=mode), pw.unit,
                        L, K, N, mode=mode, out_dtype=torch.float32)
    assert rel_fro(gx.double().cpu(), (ddy @ dw).cpu()) <= tol
    gw = ops.gemm_tiled(ops.expand_tiled_transposed(pdy, mode=mode), pdy.unit, ops.expand_tiled_transposed(px, mode=mode), px.unit,
                        N, K, L, mode=mode, out_dtype=torch.float32)
    assert rel_fro(gw.double().cpu(), (ddy.T @ dx).cpu()) <= tol
    # a transposed expansion without rotation: plain packed tensors
    gw2 = ops.gemm_tiled(ops.expand_tiled_transposed(pa, mode=mode), pa.unit, ops.expand_tiled_transposed(pa, mode=mode), pa.unit,
                         K, K, L, mode=mode, out_dtype=torch.float32)
    assert rel_fro(gw2.double().cpu(), (da.T @ da).cpu()) <= tol


@pytest.mark.parametrize("tag", ["p32", "pb16"])
def test_linear_lowbit_nv_recipe_on_the_packed_kernels_against_reference_vectors(tag):
    """LinearLowbit with enable_nv_recipe, 64 tokens, 96 -> 64 features: forward, grad_input and grad_weight against
    what the reference computed, with no torch matmul on the way (the generic path would warn)."""
    import warnings

    from metis_hip import LinearLowbit, LinearLowbitFunction as F, bitlinear, ops
    g = dict(np.load(os.path.join(GOLDEN, "metis_reference_hadamard_wide.npz")))
    dtype = torch.float32 if tag == "p32" else torch.bfloat16
    F.enable_nv_recipe = True
    F.compute_dtype = dtype
    layer = LinearLowbit(96, 64, bias=False, args=SimpleNamespace(device="cuda", cache_quantized_weight=True),
                         storage_dtype=dtype, compute_dtype=dtype)
    with torch.no_grad():
        layer.weight.copy_(t(g["hw_w"]).to(dtype))
    xr = t(g["hw_x"]).to(dtype).cuda().requires_grad_(True)
    bitlinear._generic_path_warned.clear()
    calls = []
    real = ops.gemm_tiled
    ops.gemm_tiled = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            y = layer(xr)
            y.backward(t(g["hw_dy"]).to(dtype).cuda())
    finally:
        ops.gemm_tiled = real
    assert len(calls) == 3                                      # forward, input gradient, weight gradient
    pw = layer._get_quantized_weight(layer.weight, arith=dtype)
    assert isinstance(pw, ops.PackedNVFP4) and pw.rht == F._hadamard_mask() and (pw.tiled_t is not None or pw.tiled_t_pb16 is not None)
    # the quantized weight the reference multiplied with
    wq = pw.dequantize(dtype).float().cpu()
    assert rel_fro(wq, t(g[f"hw_{tag}_wq"]).float()) <= (1e-6 if tag == "p32" else 2e-3)
    tol = 2e-3
    assert rel_fro(y.detach().float().cpu(), t(g[f"hw_{tag}_y"]).float()) <= tol
    assert rel_fro(xr.grad.float().cpu(), t(g[f"hw_{tag}_gx"]).float()) <= tol
    # The weight gradient's second operand is the ALREADY quantized input, rotated and quantized again (495-501).  Its
    # rotated values are small-integer combinations of one block scale, so their quotients by the new block scalar sit
    # exactly on FP4 rounding boundaries far more often than those of ordinary data, and which side such a value lands
    # on hangs on the last bit of a 16-term binary32 sum.  The kernels add the sixteen terms in the order the reference's
    # matrix product adds them (k = 0 .. 15), which reproduces its operand bit for bit (test_oracle_pins.py shows on the
    # CPU that a butterfly network or a double-precision sum would each leave 5 % of the elements different).
    x_op = F.q_backward_input.pack(t(g[f"hw_{tag}_xq"]).to(dtype).cuda().reshape(-1, 96), arith=dtype, rht=F._hadamard_mask())
    got, want = x_op.dequantize(dtype).float().cpu(), t(g[f"hw_{tag}_wgrad_x"]).float().reshape(-1, 96)
    assert rel_fro(got, want) <= (1e-6 if tag == "p32" else 2e-3)
    assert float((got - want).abs().le(1e-6 * float(want.abs().max())).float().mean()) > (0.9999 if tag == "p32" else 0.99)
    dy_op = F.q_backward_outputgrad.pack(t(g["hw_dy"]).to(dtype).cuda().reshape(-1, 64), arith=dtype, rht=F._hadamard_mask())
    assert rel_fro(dy_op.dequantize(dtype).float().cpu(), t(g[f"hw_{tag}_wgrad_dy"]).float().reshape(-1, 64)) <= (1e-6 if tag == "p32" else 2e-3)
    assert rel_fro(layer.weight.grad.float().cpu(), t(g[f"hw_{tag}_gw"]).float()) <= tol
    # and against the product of the operands as this library formed them: the GEMM itself is exact to its tolerance
    dense = dy_op.dequantize(dtype).double().T @ x_op.dequantize(dtype).double()
    assert rel_fro(layer.weight.grad.double().cpu(), dense.cpu()) <= (2e-4 if tag == "p32" else 2.5e-3)


def test_nv_recipe_at_a_training_shape_keeps_the_packed_kernels_and_matches_the_generic_path():
    """4096 tokens, 1536 -> 8960 (the QAT projection): kernel path against the module's own generic path
    (rotation kernel + three-call QDQ + torch matmuls, `hadamard_backend="torch_gemm"` switches the kernels off)."""
    from metis_hip import LinearLowbit, LinearLowbitFunction as F
    F.enable_nv_recipe = True
    args = SimpleNamespace(device="cuda", cache_quantized_weight=True)
    layer = LinearLowbit(1536, 8960, bias=False, args=args, storage_dtype=torch.bfloat16, compute_dtype=torch.float32)
    x = synthetic_activation(41, 4096, 1536).cuda().reshape(2, 2048, 1536)
    dy = (torch.randn(2, 2048, 8960, generator=torch.Generator().manual_seed(42)) * 1e-3).bfloat16().cuda()
    outs = {}
    for backend in ("auto", "torch_gemm"):
        F.hadamard_backend = backend
        layer._quantized_weight_cache = None
        layer.weight.grad = None
        xr = x.clone().requires_grad_(True)
        y = layer(xr)
        y.backward(dy.to(y.dtype))
        outs[backend] = (y.detach().float(), xr.grad.float(), layer.weight.grad.float())
    # output and input gradient agree to the GEMM tolerance; the weight gradient's re-quantized input operand is the one
    # whose codes hang on the last bit of the rotation's sums (see the test above), and the two paths sum in different orders
    for (a, b), tol in zip(zip(outs["auto"], outs["torch_gemm"]), (2e-3, 2e-3, 3e-2)):
        assert rel_fro(a.cpu(), b.cpu()) <= tol


def test_bitlinear_under_the_nv_recipe_is_the_rotated_residual_plus_the_rank_r_branch():
    """BitLinear (rank 32) with enable_nv_recipe: the fused launch multiplies the quantized activation with the rotated,
    quantized, rotated-back residual weight and adds the rank-r branch; its gradients are LinearLowbit's (pinned above
    against the reference's vectors) plus the branch's share.  Checked against the pieces computed separately."""
    from metis_hip import BitLinear, LinearLowbitFunction as F, MetisArgs, ops
    F.enable_nv_recipe = True
    K, N, r, L = 256, 192, 32, 320
    args = MetisArgs.direct_fp4(forward_svd_rank=r)
    args.enable_nv_recipe = True
    args.q_backward_input = args.q_backward_weight = args.q_backward_outputgrad = "nvfp4e2m1bnosr"   # round to nearest: deterministic
    layer = BitLinear(K, N, args=args, bias=False, dtype=torch.float32, compute_dtype=torch.float32).cuda()
    with torch.no_grad():
        layer.warmup_linear.weight.copy_(torch.randn(N, K, generator=torch.Generator().manual_seed(61)) * 0.05)
    layer.split()
    assert F.enable_nv_recipe and F._nv_on_kernels()
    x = synthetic_activation(62, L, K).float().cuda().requires_grad_(True)
    dy = (torch.randn(L, N, generator=torch.Generator().manual_seed(63)) * 1e-2).cuda()
    calls = []
    real = ops.gemm_tiled
    ops.gemm_tiled = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        y = layer(x)
        y.backward(dy)
    finally:
        ops.gemm_tiled = real
    assert len(calls) == 3
    mask = F._hadamard_mask()
    v, u, s_ = layer.vlinear.weight.detach(), layer.ulinear.weight.detach(), layer.s.detach()
    res = layer.warmup_linear.weight.detach()
    pw = ops.quantize_rht(res, 0, mask)
    w_back = pw.dequantize(torch.float32).double()
    xq = ops.quantize(x.detach(), 0).dequantize(torch.float32).double()
    tt = ((x.detach().bfloat16() @ v.bfloat16().T) * s_.bfloat16()).double()              # bf16 rank-r branch
    want_y = xq @ w_back.T + tt @ u.bfloat16().double().T
    assert rel_fro(y.detach().double().cpu(), want_y.cpu()) <= 2e-3
    dy_back = ops.quantize_rht(dy, 0, mask).dequantize(torch.float32).double()
    x_back = ops.quantize_rht(xq.float(), 0, mask).dequantize(torch.float32).double()
    assert rel_fro(layer.warmup_linear.weight.grad.double().cpu(), (dy_back.T @ x_back).cpu()) <= 2e-3
    g_xv = (dy.bfloat16() @ u.bfloat16()) * s_.bfloat16()                                   # [L, r]
    want_gx = dy_back @ w_back + g_xv.double() @ v.bfloat16().double()
    assert rel_fro(x.grad.double().cpu(), want_gx.cpu()) <= 2e-3


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("M,N,K,r", [(64, 384, 1024, 32), (1, 132, 256, 0), (200, 64, 2048, 64), (48, 512, 18944, 0)])
@pytest.mark.parametrize("deferred", [False, True])
def test_decode_sized_call_against_a_rotated_weight_rotates_the_activation(mode, M, N, K, r, deferred, monkeypatch):
    """NV recipe at decode size: the packed rotated weight is streamed as it is by the decode-sized kernel and the
    activation's operand carries the rotation (every dequantized block rotated forward, / 16): x^ W~^T = a' Q^T.
    Against the product of the dequantized tensors (the weight rotated back) in double precision, within the one
    rounding of the rotated operand to its 16-bit format; the tiled GEMM (which rounds the rotated-back weight
    instead) gives the same to that accuracy; and no tiled expansion is built."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + N + K)
    x = synthetic_activation(41 + M, M, K).cuda()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().cuda()
    tt = uu = None
    if r:
        tt, uu = (torch.randn(M, r, generator=g) * 0.1).bfloat16().cuda(), (torch.randn(N, r, generator=g) * 0.1).bfloat16().cuda()
    bias = torch.randn(N, generator=g).bfloat16().cuda()
    pw = ops.quantize_rht(w, mode, _mask())
    pw.persistent = True
    px = ops.quantize(x, mode, deferred=deferred)
    tiled = ops.linear_fwd(ops.quantize(x, mode), pw, t=tt, u=uu, bias=bias, out_dtype=torch.float32, reference_rounding=mode == 1, tiled=True)
    assert ops.nv_decode_applies(px, [pw], [r])
    monkeypatch.setattr(ops, "expand_tiled", lambda *a, **k: (_ for _ in ()).throw(AssertionError("the tiled expansion ran")))
    got = ops.linear_fwd(px, pw, t=tt, u=uu, bias=bias, out_dtype=torch.float32, reference_rounding=mode == 1)
    monkeypatch.undo()
    dt = torch.float32 if mode == 0 else torch.bfloat16
    want = ops.quantize(x, mode).dequantize(dt).double() @ pw.dequantize(dt).double().T + bias.double()
    if r:
        want = want + tt.double() @ uu.double().T
    tol = 4e-4 if mode == 0 else 4e-3                     # binary16 / bf16 rounding of one operand (and of the bf16 product)
    assert rel_fro(got.double().cpu(), want.cpu()) <= tol
    assert rel_fro(tiled.double().cpu(), want.cpu()) <= tol
    assert torch.equal(px.unit, ops.quantize(x, mode).unit)
    # grouped: two rotated members on one activation, one launch
    outs = ops.linear_fwd_grouped(ops.quantize(x, mode, deferred=deferred), [(pw, tt, uu, bias), (pw, None, None, None)],
                                  out_dtype=torch.float32, reference_rounding=mode == 1)
    assert torch.equal(outs[0], got)
    # a rotated activation, or mixed rotations, are not this call's business
    assert not ops.nv_decode_applies(ops.quantize_rht(x, mode, _mask()), [pw], [r])
    assert not ops.nv_decode_applies(px, [pw, ops.quantize(w, mode)], [r, r])


@pytest.mark.parametrize("compute,fuse_norms", [(torch.bfloat16, False), (torch.float32, False), (torch.bfloat16, True)])
def test_decode_step_of_a_layer_under_the_nv_recipe_stays_on_the_decode_sized_kernel(compute, fuse_norms, monkeypatch):
    """A patched Qwen2 decoder layer under the NV recipe, 64 sequences x 1 token, no autograd: every projection runs on the
    decode-sized kernel against its packed rotated weight (q/k/v and gate/up as grouped launches), no tiled expansion
    and no tiled GEMM; the output agrees with the member-by-member evaluation on the tiled GEMM."""
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
    args = MetisArgs.direct_fp4(forward_svd_rank=32)
    args.enable_nv_recipe = True
    if compute == torch.float32:
        from metis_hip.patch import DEFAULT_TARGETS, replace_linear_with_metis
        replace_linear_with_metis(model=holder, dtype=torch.bfloat16, metis_args=args, target_modules=list(DEFAULT_TARGETS),
                                  compute_dtype=torch.float32)
    else:
        replace_model_with_metis(holder, args, fuse_norms=fuse_norms)
    assert F.enable_nv_recipe and F._nv_on_kernels()
    if fuse_norms:
        from metis_hip import FusedRMSNormQuant
        fused_calls = []
        real_rq = ops.rmsnorm_quantize
        monkeypatch.setattr(ops, "rmsnorm_quantize", lambda *a, **k: (fused_calls.append(1), real_rq(*a, **k))[1])
        assert isinstance(layer.input_layernorm, FusedRMSNormQuant)
    x = (torch.randn(64, 1, 256, device="cuda") + 0.5).bfloat16()
    pos = torch.zeros(64, 1, dtype=torch.long, device="cuda")
    pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)

    def run():
        with torch.no_grad():
            out = holder["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
        return (out[0] if isinstance(out, tuple) else out).float()

    seen = {"rotated_operand": 0, "tiled": 0}
    real_do, real_gt = ops.decode_operand, ops.gemm_tiled
    monkeypatch.setattr(ops, "decode_operand", lambda p, mode=0, center=None, rotate=None:
                        (seen.__setitem__("rotated_operand", seen["rotated_operand"] + (rotate is not None)), real_do(p, mode, center, rotate))[1])
    monkeypatch.setattr(ops, "gemm_tiled", lambda *a, **k: (seen.__setitem__("tiled", seen["tiled"] + 1), real_gt(*a, **k))[1])
    # (the rotated operand usually comes from the launch that also finishes the rank-r projection)
    real_pao = ops.project_and_operand
    monkeypatch.setattr(ops, "project_and_operand", lambda *a, **k:
                        (seen.__setitem__("rotated_operand", seen["rotated_operand"] + (k.get("rotate") is not None)), real_pao(*a, **k))[1])
    got = run()
    assert seen == {"rotated_operand": 4, "tiled": 0}, seen          # q/k/v, o, gate/up, down
    if fuse_norms:
        assert len(fused_calls) == 2                                 # both norms quantize for their groups under the recipe too
    monkeypatch.setattr(ops, "nv_decode_applies", lambda *a, **k: False)
    seen.update(rotated_operand=0, tiled=0)
    want = run()
    assert seen == {"rotated_operand": 0, "tiled": 7}, seen
    assert rel_fro(got.cpu(), want.cpu()) <= 1e-2


def test_fused_norm_feeds_the_groups_under_the_nv_recipe_with_autograd():
    """Training step of a patched Qwen2 layer under the NV recipe (round-to-nearest backward quantizers, so that two
    runs can be compared): with the norms fused into the groups' quantizer the output and every gradient agree with
    the unfused layer up to a bf16 ulp of the normed tensor here and there."""
    pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
    from metis_hip import FusedRMSNormQuant, LinearLowbitFunction as F, MetisArgs, replace_model_with_metis
    cfg = Qwen2Config(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=128, max_position_embeddings=256)
    cfg._attn_implementation = "eager"
    results = {}
    for fuse in (False, True):
        torch.manual_seed(0)
        layer = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16).cuda()
        for p in layer.parameters():
            if p.dim() == 2:
                torch.nn.init.normal_(p, std=0.02)
        holder = torch.nn.ModuleDict({"layer": layer})
        args = MetisArgs.direct_fp4(forward_svd_rank=32)
        args.enable_nv_recipe = True
        args.q_backward_input = args.q_backward_weight = args.q_backward_outputgrad = "nvfp4e2m1bnosr"
        replace_model_with_metis(holder, args, fuse_norms=fuse)
        assert F.enable_nv_recipe and F._nv_on_kernels() and isinstance(layer.input_layernorm, FusedRMSNormQuant) == fuse
        g = torch.Generator().manual_seed(5)
        x = (torch.randn(2, 160, 256, generator=g) + 0.5).bfloat16().cuda().requires_grad_(True)
        pos = torch.arange(160, device="cuda").unsqueeze(0).expand(2, -1)
        pe = Qwen2RotaryEmbedding(cfg).cuda()(x, pos)
        out = holder["layer"](x, position_embeddings=pe, attention_mask=None, position_ids=pos)
        out = out[0] if isinstance(out, tuple) else out
        dy = (torch.randn(out.shape, generator=g) * 1e-2).bfloat16().cuda()
        out.backward(dy)
        results[fuse] = (out.detach().float().cpu(), x.grad.float().cpu(),
                         layer.mlp.down_proj.warmup_linear.weight.grad.float().cpu(),
                         layer.self_attn.q_proj.warmup_linear.weight.grad.float().cpu(),
                         layer.input_layernorm.weight.grad.float().cpu())
    for a, b in zip(results[True], results[False]):
        assert rel_fro(a, b) <= 3e-2


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("M,K,R", [(64, 3584, 192), (1, 256, 32), (200, 2048, 64)])
def test_merged_prepare_launch_builds_the_rotated_operand_too(mode, M, K, R):
    """metis_decode_prepare_deferred with rotate: the projection's finishing step and the rotated operand in one launch
    equal metis_lowrank_project and metis_nvfp4_decode_operand_rht bit for bit, also after the quantizer's launch has
    carried the projection's first step."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + K + R)
    x = (torch.randn(M, K, generator=g) * 2).bfloat16().cuda()
    v = (torch.randn(R, K, generator=g) * 0.05).bfloat16().cuda()
    s = torch.rand(R, generator=g).bfloat16().cuda()
    want_xv, want_t = ops.lowrank_project(x, v, s)
    p1 = ops.quantize(x, mode, deferred=True)
    want_op = ops.decode_operand(p1, mode, rotate=_mask())
    plain_op = ops.decode_operand(ops.quantize(x, mode, deferred=True), mode)
    assert not torch.equal(want_op, plain_op)
    p2 = ops.quantize(x, mode, deferred=True)
    xv, t, op = ops.project_and_operand(x, v, s, p2, mode, rotate=_mask())
    assert torch.equal(xv, want_xv) and torch.equal(t, want_t) and torch.equal(op, want_op) and torch.equal(p2.unit, p1.unit)
    if R <= 128:
        p3, pending = ops.quantize_project_decode(x, v, mode)
        xv3, t3, op3 = ops.project_and_operand(x, v, s, p3, mode, pending=pending, rotate=_mask())
        assert torch.equal(xv3, want_xv) and torch.equal(t3, want_t) and torch.equal(op3, want_op)
