"""Module wiring of the drop-in classes, mirroring the reference's own tests
(tests/test_metis_quant_cache.py) with counting quantizer subclasses of Cast2Fp32 as spies.
These run on CPU: identity quantizers take the generic (torch matmul) path, no NVFP4 arithmetic.
"""
from collections import OrderedDict as OrderedDictCompat
from types import SimpleNamespace

import pytest
import torch

from metis_hip import (BitLinear, Cast2Fp32, LinearLowbit, LinearLowbitFunction, MetisArgs, MetisHipError,
                       quant_func, replace_linear_with_metis)


@pytest.fixture(autouse=True)
def _reset_function_config():
    F = LinearLowbitFunction
    keep = {k: getattr(F, k) for k in ("q_forward_input", "q_forward_weight", "q_backward_input", "q_backward_weight",
                                       "q_backward_outputgrad", "enable_activation_svd", "enable_backward_svd",
                                       "enable_nv_recipe", "compute_dtype", "metis_mode")}
    yield
    for k, v in keep.items():
        setattr(F, k, v)
    BitLinear.rollout_merge_active = False


def _identity_config():
    F = LinearLowbitFunction
    F.compute_dtype = torch.float32
    F.q_forward_input = Cast2Fp32
    F.q_forward_weight = Cast2Fp32
    F.q_backward_input = Cast2Fp32
    F.q_backward_outputgrad = Cast2Fp32
    F.enable_activation_svd = False
    F.enable_backward_svd = False
    F.enable_nv_recipe = False


def test_registry_surface():
    assert {"nvfp4e2m1bnosr", "nvfp4e2m1b", "fp32"} <= set(quant_func)
    for q in quant_func.values():
        for m in ("get_scalar", "quant", "rquant", "quantize_dequantize"):
            assert callable(getattr(q, m))
        assert hasattr(q, "compile_quantize_dequantize")
    assert quant_func["nvfp4e2m1bnosr"].block_shape == (1, 16)
    with pytest.raises(KeyError):
        quant_func["no_such_format"]


def test_nvfp4_has_no_cpu_path():
    with pytest.raises(MetisHipError):
        quant_func["nvfp4e2m1bnosr"].quantize_dequantize(torch.zeros(4, 32))
    with pytest.raises(ValueError):       # reference quant.py:400-403
        quant_func["nvfp4e2m1bnosr"].quantize_dequantize(torch.zeros(4, 24))


def test_weight_cache_reuses_then_invalidates_after_parameter_update():
    class CountingQuant(Cast2Fp32):
        calls = 0

        @classmethod
        def quantize_dequantize(cls, value):
            cls.calls += 1
            return value.detach().clone()

    args = SimpleNamespace(device="cpu", cache_quantized_weight=True)
    layer = LinearLowbit(16, 8, bias=False, args=args)
    _identity_config()
    LinearLowbitFunction.q_forward_weight = CountingQuant
    x = torch.randn(2, 3, 16, requires_grad=True)
    layer(x).sum().backward()
    assert layer.weight.grad is not None
    layer(x.detach())
    assert CountingQuant.calls == 1
    with torch.no_grad():
        layer.weight.add_(0.1)
    layer(x.detach())
    assert CountingQuant.calls == 2


def test_mean_activation_path_uses_quantize_dequantize():
    class CountingQuant(Cast2Fp32):
        calls = 0

        @classmethod
        def quantize_dequantize(cls, value):
            cls.calls += 1
            return value

        @classmethod
        def get_scalar(cls, value):
            raise AssertionError("mean activation path must use fused QDQ")

    x = torch.randn(2, 3, 16)
    cache = {}
    out = LinearLowbitFunction.svd_quant(x, quant_func=CountingQuant, metis_mode="mean", mean_cache=cache, cache_key="t")
    assert out.shape == x.shape and CountingQuant.calls == 1
    torch.testing.assert_close(out, x)
    assert cache["t"][1] == 6
    # single-token decode updates the running mean with weights (reference 315-322)
    step = torch.randn(4, 1, 16)
    LinearLowbitFunction.svd_quant(step, quant_func=CountingQuant, metis_mode="mean", mean_cache=cache, cache_key="t")
    assert cache["t"][1] == 10
    with pytest.raises(ValueError):
        LinearLowbitFunction.svd_quant(x, quant_func=CountingQuant, metis_mode="bogus")


@pytest.mark.parametrize("cd", [torch.float32, torch.bfloat16])
def test_token_mean_of_the_packed_mean_mode_follows_the_reference_bookkeeping(cd):
    """The helper the packed mean mode uses gives the generic path's mean and cache entries: plain mean and
    row count for a prefill call, weighted running mean for single-token calls (reference 311-329)."""
    F = LinearLowbitFunction
    keep = F.compute_dtype
    F.compute_dtype = cd
    try:
        g = torch.Generator().manual_seed(1)
        x = (torch.randn(2, 3, 16, generator=g) + 2.0).to(cd)
        a, b = {}, {}
        me = F._token_mean(x, mean_cache=a, cache_key="k")
        F.svd_quant(x, quant_func=Cast2Fp32, metis_mode="mean", mean_cache=b, cache_key="k")
        assert me.shape == (16,) and me.dtype == cd and a["k"][1] == b["k"][1] == 6
        torch.testing.assert_close(a["k"][0], b["k"][0])
        step = (torch.randn(4, 1, 16, generator=g) - 1.0).to(cd)
        me2 = F._token_mean(step, mean_cache=a, cache_key="k")
        F.svd_quant(step, quant_func=Cast2Fp32, metis_mode="mean", mean_cache=b, cache_key="k")
        assert a["k"][1] == b["k"][1] == 10
        torch.testing.assert_close(a["k"][0], b["k"][0])
        torch.testing.assert_close(me2, a["k"][0].reshape(-1))
        # without a cache: the plain mean, nothing stored
        torch.testing.assert_close(F._token_mean(x.reshape(6, 16)), x.reshape(6, 16).float().mean(dim=0).to(cd))
    finally:
        F.compute_dtype = keep


def test_identity_quantizers_give_plain_linear_gradients():
    args = SimpleNamespace(device="cpu", cache_quantized_weight=False)
    layer = LinearLowbit(16, 16, bias=True, args=args)
    _identity_config()
    x = torch.randn(2, 3, 16, requires_grad=True)
    layer(x).sum().backward()
    want_w = torch.ones(16, 1) @ x.detach().reshape(-1, 16).sum(dim=0, keepdim=True)
    torch.testing.assert_close(layer.weight.grad, want_w, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(layer.bias.grad, torch.full((16,), 6.0))
    torch.testing.assert_close(x.grad, layer.weight.detach().sum(0).expand(2, 3, 16), rtol=1e-5, atol=1e-5)
    assert layer.weight.grad.dtype == torch.float32


def test_replace_linear_does_not_split_when_forward_svd_disabled():
    model = torch.nn.Sequential(torch.nn.Linear(16, 8, bias=False))
    args = MetisArgs(enable_forward_svd=False)
    args.device = "cpu"
    replaced = replace_linear_with_metis(model, dtype=torch.float32, metis_args=args, target_modules=["0"],
                                         compute_dtype=torch.float32)
    layer = replaced[0]
    assert isinstance(layer.warmup_linear, LinearLowbit)
    assert layer.vlinear is None and layer.ulinear is None and layer.s is None and not layer.is_svd_quant


def test_replace_linear_splits_and_keeps_state_dict_keys():
    torch.manual_seed(0)
    model = torch.nn.ModuleDict({"attn": torch.nn.ModuleDict({"q_proj": torch.nn.Linear(32, 24, bias=True),
                                                              "k_proj": torch.nn.Linear(32, 16, bias=True)}),
                                 "mlp": torch.nn.ModuleDict({"down_proj": torch.nn.Linear(24, 32, bias=False)})})
    w_q = model["attn"]["q_proj"].weight.detach().clone()
    args = MetisArgs(forward_svd_rank=8)
    args.device = "cpu"
    replace_linear_with_metis(model, dtype=torch.float32, metis_args=args, compute_dtype=torch.float32)
    q, k, d = model["attn"]["q_proj"], model["attn"]["k_proj"], model["mlp"]["down_proj"]
    assert all(isinstance(m, BitLinear) and m.is_svd_quant for m in (q, k, d))
    assert q.activation_group is k.activation_group and q.activation_group["name"] == "attn.qkv"
    assert d.activation_group is None and q.layer_name == "attn.q_proj"
    keys = set(model.state_dict())
    assert {"attn.q_proj.ulinear.weight", "attn.q_proj.vlinear.weight", "attn.q_proj.s",
            "attn.q_proj.warmup_linear.weight", "attn.q_proj.warmup_linear.bias"} <= keys
    assert "mlp.down_proj.warmup_linear.bias" not in keys
    # U diag(s) V + residual reconstructs the original weight
    rec = (q.ulinear.weight * q.s) @ q.vlinear.weight + q.warmup_linear.weight
    torch.testing.assert_close(rec, w_q, rtol=1e-5, atol=1e-5)
    assert q.vlinear.weight.shape == (8, 32) and q.ulinear.weight.shape == (24, 8) and q.s.shape == (8,)


def _hand_assembled(args, group=None, name="test.layer", bias=False):
    layer = BitLinear.__new__(BitLinear)
    torch.nn.Module.__init__(layer)
    layer.args = args
    layer.is_svd_quant = True
    layer.mean_cache = {}
    layer.activation_group = group
    layer._merged_rollout_weight_cache = None
    layer.layer_name = name
    layer.compute_dtype = torch.float32
    layer.vlinear = LinearLowbit(16, 4, bias=False, args=args)
    layer.ulinear = torch.nn.Linear(4, 8, bias=False)
    layer.warmup_linear = LinearLowbit(16, 8, bias=bias, args=args)
    layer.s = torch.nn.Parameter(torch.ones(4))
    return layer


class _CountingActivationQuant(Cast2Fp32):
    calls = 0

    @classmethod
    def quantize_dequantize(cls, value):
        cls.calls += 1
        return value


def _mean_config(q):
    _identity_config()
    F = LinearLowbitFunction
    F.q_forward_input = q
    F.enable_activation_svd = True
    F.activation_lowrank_svd = 4
    F.activation_broadcast_dim = -1
    F.tp_simulate = False
    F.metis_mode = "mean"


def test_bitlinear_svd_branches_share_one_quantized_activation():
    args = SimpleNamespace(device="cpu", cache_quantized_weight=False, forward_svd_rank=4)
    layer = _hand_assembled(args)
    _CountingActivationQuant.calls = 0
    _mean_config(_CountingActivationQuant)
    x = torch.randn(2, 3, 16, requires_grad=True)
    layer(x).sum().backward()
    assert _CountingActivationQuant.calls == 1
    assert x.grad is not None and layer.vlinear.weight.grad is not None and layer.warmup_linear.weight.grad is not None


def test_projection_group_reuses_quantized_activation():
    args = SimpleNamespace(device="cpu", cache_quantized_weight=False, forward_svd_rank=4)
    group = {"name": "test.attention.qkv", "mean_cache": {}, "input_ref": None, "quantized_input": None}
    q_proj = _hand_assembled(args, group, "test.attention.q_proj")
    k_proj = _hand_assembled(args, group, "test.attention.k_proj")
    _CountingActivationQuant.calls = 0
    _mean_config(_CountingActivationQuant)
    x = torch.randn(2, 3, 16, requires_grad=True)
    (q_proj(x).sum() + k_proj(x).sum()).backward()
    assert _CountingActivationQuant.calls == 1
    assert x.grad is not None and q_proj.vlinear.weight.grad is not None and k_proj.vlinear.weight.grad is not None
    # a different tensor object is quantized again
    q_proj(torch.randn(2, 3, 16))
    assert _CountingActivationQuant.calls == 2


def test_rollout_merged_weight_cache_reuses_and_invalidates():
    args = SimpleNamespace(device="cpu", cache_quantized_weight=True, forward_svd_rank=4)
    layer = _hand_assembled(args, bias=True)
    _mean_config(Cast2Fp32)
    x = torch.randn(2, 3, 16)
    with torch.no_grad():
        BitLinear.rollout_merge_active = False
        expected = layer(x)
        BitLinear.rollout_merge_active = True
        actual = layer(x)
        first = layer._get_merged_rollout_weight(torch.float32)
        second = layer._get_merged_rollout_weight(torch.float32)
        layer.s.add_(0.1)
        updated = layer._get_merged_rollout_weight(torch.float32)
    torch.testing.assert_close(actual, expected)
    assert first is second and updated is not first


def test_weight_cache_sees_a_replaced_parameter():
    """A Parameter that is replaced by a fresh one (load_state_dict(assign=True), `layer.weight = nn.Parameter(...)`) starts
    at the same version counter as the one it replaces: the caches key on the parameter's identity and storage as well."""
    class CountingQuant(Cast2Fp32):
        calls = 0

        @classmethod
        def quantize_dequantize(cls, value):
            cls.calls += 1
            return value.detach().clone()

    layer = LinearLowbit(16, 8, bias=False, args=SimpleNamespace(device="cpu", cache_quantized_weight=True))
    _identity_config()
    LinearLowbitFunction.q_forward_weight = CountingQuant
    x = torch.randn(2, 3, 16)
    first = layer(x)
    layer(x)
    assert CountingQuant.calls == 1
    fresh = torch.nn.Parameter(torch.randn(8, 16))
    with torch.no_grad():
        while fresh._version < layer.weight._version:            # the same version counter as the parameter it replaces
            fresh.add_(0.0)
    assert fresh._version == layer.weight._version
    layer.weight = fresh
    second = layer(x)
    assert CountingQuant.calls == 2 and not torch.equal(first, second)
    layer.load_state_dict({"weight": torch.randn(8, 16)}, assign=True)
    third = layer(x)
    assert CountingQuant.calls == 3 and not torch.equal(second, third)


def test_full_svd_backward_branch_is_refused():
    """enable_backward_svd with backward_lowrank_svd <= 0 is the reference's full-SVD branch (bitlinear.py:476-486), which
    this library does not implement: it says so instead of quantizing the gradient with another method."""
    layer = LinearLowbit(16, 8, bias=False, args=SimpleNamespace(device="cpu", cache_quantized_weight=False))
    _identity_config()
    F = LinearLowbitFunction
    F.enable_backward_svd, F.backward_lowrank_svd = True, 0
    try:
        y = layer(torch.randn(2, 3, 16, requires_grad=True))
        with pytest.raises(NotImplementedError):
            y.sum().backward()
    finally:
        F.enable_backward_svd, F.backward_lowrank_svd = False, 32


def test_unsupported_options_fail_loudly():
    args = MetisArgs()
    args.device = "cpu"
    with pytest.raises(ValueError):
        BitLinear(16, 8, args=args, dtype=torch.float32, compute_dtype=torch.int8)
    with pytest.raises(ValueError):                             # reference bitlinear.py:368
        LinearLowbitFunction.svd_quant(torch.zeros(2, 16), Cast2Fp32, metis_mode="no_such_mode")
    LinearLowbitFunction.hadamard_backend = "dao_cuda"          # the optional CUDA extension is not part of this build
    try:
        with pytest.raises(RuntimeError):
            LinearLowbitFunction._apply_hadamard_blocks(torch.zeros(2, 16))
    finally:
        LinearLowbitFunction.hadamard_backend = "auto"


# ----------------------------------------------------------------------------- NV recipe: tiled random Hadamard rotation
def _hadamard_golden():
    import os
    import numpy as np
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_hadamard.npz")
    return np.load(path)


def test_hadamard_rotation_matches_the_reference_vectors():
    g = _hadamard_golden()
    F = LinearLowbitFunction
    x = torch.from_numpy(g["had_x"])
    assert torch.equal(F._get_hadamard_sign(16, torch.device("cpu"), torch.float32), torch.from_numpy(g["had_sign16"]))
    torch.testing.assert_close(F._apply_hadamard_blocks(x), torch.from_numpy(g["had_fwd"]), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(F._apply_hadamard_blocks(x, inverse=True), torch.from_numpy(g["had_inv"]), rtol=1e-6, atol=1e-6)
    want_bf16 = torch.from_numpy(g["had_fwd_bf16"].view("int16")).view(torch.bfloat16)
    got_bf16 = F._apply_hadamard_blocks(x.bfloat16())
    assert got_bf16.dtype == torch.bfloat16
    torch.testing.assert_close(got_bf16.float(), want_bf16.float(), rtol=1e-2, atol=1e-2)
    with pytest.raises(ValueError):
        F._apply_hadamard_blocks(torch.zeros(2, 24))              # 16 does not divide 24 (reference 143-147)


def test_hadamard_roundtrip_non_power_of_two_hidden_size_and_small_workspace():
    """Reference tests/test_metis_quant_cache.py:101-122."""
    F = LinearLowbitFunction
    x = torch.randn(2, 3, 1536, generator=torch.Generator().manual_seed(3))
    torch.testing.assert_close(F._apply_hadamard_blocks(F._apply_hadamard_blocks(x), inverse=True), x, rtol=1e-5, atol=1e-5)
    x = torch.randn(64, 1536, generator=torch.Generator().manual_seed(4))
    keep = F.hadamard_workspace_mb
    F.hadamard_workspace_mb = 1
    try:
        back = F._apply_hadamard_blocks(F._apply_hadamard_blocks(x), inverse=True)
    finally:
        F.hadamard_workspace_mb = keep
    torch.testing.assert_close(back, x, rtol=1e-5, atol=1e-5)


def test_direct_forward_path_is_untouched_by_the_nv_recipe():
    """Reference tests/test_metis_quant_cache.py:125-135."""
    _identity_config()
    LinearLowbitFunction.enable_nv_recipe = True
    x = torch.randn(2, 3, 1536, generator=torch.Generator().manual_seed(5))
    torch.testing.assert_close(LinearLowbitFunction.quantize_input(x), x, rtol=1e-5, atol=1e-5)


def test_nv_recipe_rotates_only_the_wgrad_operands():
    """Reference tests/test_metis_quant_cache.py:138-160: with identity quantizers the rotations cancel
    and the weight gradient is the plain one."""
    _identity_config()
    layer = LinearLowbit(16, 16, bias=False, args=SimpleNamespace(device="cpu", cache_quantized_weight=False))
    LinearLowbitFunction.enable_nv_recipe = True
    LinearLowbitFunction.hadamard_backend = "torch_gemm"
    LinearLowbitFunction.hadamard_tile_size = 16
    x = torch.randn(2, 3, 16, generator=torch.Generator().manual_seed(6), requires_grad=True)
    layer(x).sum().backward()
    expected = torch.ones(16, 1) @ x.detach().reshape(-1, 16).sum(dim=0, keepdim=True)
    torch.testing.assert_close(layer.weight.grad, expected, rtol=1e-5, atol=1e-5)


def test_svd_mode_and_tp_simulation_reassemble_the_input_with_identity_quantizers():
    """With identity quantizers, low-rank part + residual is the input again, whatever the rank, for 2-D
    and 3-D inputs, with a broadcast slice, and chunk by chunk under the TP simulation (reference 243-360)."""
    F = LinearLowbitFunction
    g = torch.Generator().manual_seed(8)
    x2 = torch.randn(48, 64, generator=g)
    x3 = torch.randn(2, 24, 64, generator=g)
    for x in (x2, x3):
        out = F.svd_quant(x, Cast2Fp32, rank=16, niter=1, metis_mode="svd")
        assert out.shape == x.shape
        torch.testing.assert_close(out, x, rtol=1e-5, atol=1e-5)
        out = F.svd_quant(x, Cast2Fp32, rank=16, niter=1, tp_simulate=True, tp_parts=3, metis_mode="svd")
        assert out.shape == x.shape
        torch.testing.assert_close(out, x, rtol=1e-5, atol=1e-5)
    out = F.svd_quant(x3, Cast2Fp32, rank=8, niter=0, broadcast_dim=0, metis_mode="svd")
    torch.testing.assert_close(out, x3, rtol=1e-5, atol=1e-5)


def test_merge_tool_restores_plain_linear_weights(tmp_path):
    """Patched-and-split model -> state dict -> merge tool -> loads into the unpatched architecture with
    the original weights (reference tools/convert_bitlinear_to_standard.py:80-172)."""
    from metis_hip.tools.merge_state_dict import main as merge_main, merge_bitlinear_state_dict
    torch.manual_seed(11)

    def make():
        return torch.nn.Sequential(OrderedDictCompat([("q_proj", torch.nn.Linear(64, 48, bias=True)),
                                                     ("act", torch.nn.ReLU()),
                                                     ("o_proj", torch.nn.Linear(48, 32, bias=False))]))
    plain = make()
    reference_weights = {k: v.clone() for k, v in plain.state_dict().items()}
    args = MetisArgs(forward_svd_rank=16)
    args.device = "cpu"
    replace_linear_with_metis(plain, dtype=torch.float32, metis_args=args, target_modules=["q_proj", "o_proj"],
                              compute_dtype=torch.float32)
    sd = plain.state_dict()
    assert "q_proj.ulinear.weight" in sd and "o_proj.s" in sd and "q_proj.warmup_linear.bias" in sd
    merged = merge_bitlinear_state_dict(sd)
    assert set(merged) == set(reference_weights)
    for k, w in reference_weights.items():
        torch.testing.assert_close(merged[k], w, rtol=1e-5, atol=1e-5)
    fresh = make()
    fresh.load_state_dict(merged)                                # strict: exactly the plain architecture's keys
    # file round trip and dtype cast
    from safetensors.torch import load_file, save_file
    src, dst = tmp_path / "in.safetensors", tmp_path / "out.safetensors"
    save_file({k: v.contiguous() for k, v in sd.items()}, str(src))
    merge_main([str(src), str(dst), "--dtype", "bf16"])
    back = load_file(str(dst))
    assert set(back) == set(reference_weights) and all(t.dtype == torch.bfloat16 for t in back.values())


def test_scale_bytes_are_deferred_only_when_the_consumer_forms_them(monkeypatch):
    """The quantizer may stop after its first launch when the GEMM that follows forms the scale bytes itself: the tiled
    expansion (256 rows or more, cached weights, tiled copies kept) or any consumer under bf16 arithmetic with the
    reference's roundings.  Row count alone does not decide."""
    from metis_hip import ops
    from metis_hip.bitlinear import LinearLowbitFunction as F
    monkeypatch.setattr(F, "compute_dtype", torch.float32)
    monkeypatch.setattr(F, "reference_rounding", True)
    assert F._scales_formed_by_consumer(4096, True) and not F._scales_formed_by_consumer(4096, False)
    assert not F._scales_formed_by_consumer(64, True)
    monkeypatch.setattr(ops, "tiled_weight_copies", False)
    assert not F._scales_formed_by_consumer(4096, True)
    monkeypatch.setattr(F, "compute_dtype", torch.bfloat16)
    assert F._scales_formed_by_consumer(4096, False) and F._scales_formed_by_consumer(1, False)
    monkeypatch.setattr(F, "reference_rounding", False)
    assert not F._scales_formed_by_consumer(1, False)
