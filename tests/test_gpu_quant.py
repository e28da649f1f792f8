"""GPU parity of the NVFP4 quantizer kernels, called through the C ABI, against the CPU oracle.

Bar: bit-exact codes, E4M3 scale bytes and unit in both parity modes; dequantized output equal
to the reference's own golden QDQ output.
"""
import math

import numpy as np
import pytest
import torch

from helpers import same_bits, synthetic_activation, t

pytestmark = pytest.mark.gpu

MODES = [("p32", 0), ("pb16", 1)]


@pytest.fixture(scope="module")
def ops():
    from metis_hip import ops as _ops
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    return _ops


def _oracle_in(x_bf16, mode):
    return x_bf16.float() if mode == 0 else x_bf16


def _check_packed(p, codes, scales, unit, what=""):
    torch.cuda.synchronize()
    assert torch.equal(p.codes.cpu(), codes), f"codes differ {what}: {(p.codes.cpu() != codes).sum().item()} bytes"
    assert torch.equal(p.scales.cpu(), scales), f"scales differ {what}: {(p.scales.cpu() != scales).sum().item()} bytes"
    assert float(p.unit.cpu()) == float(unit), f"unit differs {what}: {float(p.unit.cpu())} vs {float(unit)}"


@pytest.mark.parametrize("tag,mode", MODES)
@pytest.mark.parametrize("case", ["rne", "rne3d", "rnew"])
def test_rne_against_reference_golden(ops, golden, case, tag, mode):
    """deq(pack(x)) == the reference's quantize_dequantize(x) on the reference's own vectors."""
    from oracle import metis_oracle as O
    x = t(golden[f"{case}_x"])
    want = t(golden[f"{case}_qdq_{tag}"])
    p = ops.quantize(x.cuda(), mode)
    codes, scales, unit, _ = O.nvfp4_pack(_oracle_in(x, mode))
    _check_packed(p, codes, scales, unit, case)
    got = ops.dequantize(p, want.dtype).cpu().reshape(want.shape)
    assert same_bits(got, want)
    if mode == 0:   # "stored as bf16": one rounding of the binary32 result
        assert same_bits(ops.dequantize(p, torch.bfloat16).cpu().reshape(want.shape), want.bfloat16())


@pytest.mark.parametrize("tag,mode", MODES)
@pytest.mark.parametrize("shape", [(256, 512), (1, 16), (37, 48), (3, 5, 64), (1000, 1536)])
def test_rne_row_seeded(ops, shape, tag, mode):
    from oracle import metis_oracle as O
    x = synthetic_activation(100 + sum(shape), int(np.prod(shape[:-1])), shape[-1]).reshape(shape)
    x.view(-1)[::97] = 0
    p = ops.quantize(x.cuda(), mode)
    codes, scales, unit, _ = O.nvfp4_pack(_oracle_in(x, mode))
    _check_packed(p, codes, scales, unit, str(shape))


@pytest.mark.parametrize("tag,mode", MODES)
def test_rne_all_bf16_magnitudes_and_exact_ties(ops, tag, mode):
    """Every finite bf16 magnitude against block scalars that make ties exact."""
    from oracle import c_oracle as C
    pat = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    n = (pat.numel() // 15) * 15
    for amax in (6.0, 3.0, 0.75, 448.0, 0.0283203125, 3.0e-5, 2.984375, 1.5e30):
        am = torch.tensor(amax).bfloat16()
        body = pat[:n].reshape(-1, 15)
        body = torch.where(body.float() <= am.float(), body, torch.zeros_like(body))
        x = torch.cat([am.expand(body.shape[0], 1), body], dim=1).contiguous()
        x[1::2] = -x[1::2]
        p = ops.quantize(x.cuda(), mode)
        cc, cs, cu, _ = C.nvfp4_pack(x, mode)
        _check_packed(p, cc, cs, cu, f"amax={amax}")


def test_rne_p32_exception_quotients(ops):
    """Blocks built so that |x| / (scalar/2) rounds to 5+1ulp, 7-1ulp, 10+1ulp: the three quotients
    where the reference's compress/round sequence differs from a plain RNE conversion."""
    from oracle import c_oracle as C
    import struct
    rows = []
    g = torch.Generator().manual_seed(9)
    found = 0
    # search block maxima whose scalar h = s/2 puts a bf16 value right next to 5h / 7h / 10h
    cand = torch.arange(0x3C00, 0x4400, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    s = cand / 6 + 1e-9
    h = s / 2
    for mult, delta in ((5.0, 1), (7.0, -1), (10.0, 1)):
        tgt = torch.tensor(mult)
        tq = torch.nextafter(tgt, tgt + delta)                       # the exceptional quotient
        xs = (tq * h).bfloat16()                                     # nearest bf16 to q*h
        q = xs.float() / h
        hit = (q == tq) & (xs.float() <= cand)
        for i in hit.nonzero().flatten().tolist()[:8]:
            blk = torch.zeros(16)
            blk[0] = cand[i]
            blk[1] = xs[i].float()
            blk[2] = -xs[i].float()
            rows.append(blk)
            found += 1
    assert found >= 3, "test construction failed to reach the exceptional quotients"
    x = torch.stack(rows).bfloat16().contiguous()
    p = ops.quantize(x.cuda(), 0)
    cc, cs, cu, _ = C.nvfp4_pack(x, 0)
    _check_packed(p, cc, cs, cu, "exception quotients")


@pytest.mark.parametrize("tag,mode", MODES)
@pytest.mark.parametrize("shape", [(64, 96), (256, 512), (48, 1000)])
def test_rne_col(ops, shape, tag, mode):
    from oracle import metis_oracle as O
    x = synthetic_activation(200 + shape[0], *shape)
    p = ops.quantize(x.cuda(), mode, col=True)
    codes, scales, unit, _ = O.nvfp4_pack_col(_oracle_in(x, mode))
    assert (p.rows, p.cols) == (shape[1], shape[0])
    _check_packed(p, codes, scales, unit, str(shape))


@pytest.mark.parametrize("tag,mode", MODES)
@pytest.mark.parametrize("col", [False, True])
def test_sr_explicit_noise(ops, golden, tag, mode, col):
    from oracle import metis_oracle as O
    x = t(golden["sr_x"])
    u = t(golden[f"sr_noise_{tag}"])
    p = ops.quantize(x.cuda(), mode, col=col, sr=True, noise=u.cuda())
    xin = _oracle_in(x, mode)
    codes, scales, unit, ncl = (O.nvfp4_pack_col if col else O.nvfp4_pack)(xin, u)
    _check_packed(p, codes, scales, unit, f"sr col={col}")
    if not col:
        # against the reference's own SR output wherever it stayed on the E2M1 grid
        want = t(golden[f"sr_rquant_{tag}"])
        on_grid = t(golden[f"sr_quant_{tag}"]).abs() <= 6
        got = ops.dequantize(p, want.dtype).cpu()
        assert torch.equal(got[on_grid], want[on_grid]) and int((~on_grid).sum()) == ncl


@pytest.mark.parametrize("tag,mode", MODES)
@pytest.mark.parametrize("col", [False, True])
def test_sr_internal_stream_properties(ops, tag, mode, col):
    """With its own random stream the library rounds stochastically in hardware, one Philox draw per
    output block.  What must hold whatever the draws: scale bytes and unit are those of the
    round-to-nearest pack (bit-exact against the oracle); every code is one of the two grid neighbours
    of the exact quotient with the sign of x; the result is a function of (seed, offset) only; and since
    the stream is indexed by output block, column packing equals row packing of the transpose."""
    from oracle import metis_oracle as O
    x = synthetic_activation(300, 64, 128)
    x.view(-1)[::53] = 0
    seed, offset = 0x1234_5678_9ABC_DEF0, 77
    xd = x.cuda()
    p = ops.quantize(xd, mode, col=col, sr=True, seed=seed, offset=offset)
    xin = _oracle_in(x, mode)
    xt = xin.t().contiguous() if col else xin
    _, scales, unit, _ = O.nvfp4_pack(xt)
    torch.cuda.synchronize()
    assert torch.equal(p.scales.cpu(), scales) and float(p.unit.cpu()) == float(unit)
    # bracket: code magnitude in {floor, ceil} of the quotient on the grid {0,1,2,3,4,6,8,12} (units of s/2)
    scalar = O.block_scalars(xt).double().reshape(xt.shape[0], -1, 1)
    q = (xt.double().abs().reshape(xt.shape[0], -1, 16) / (scalar / 2)).reshape(xt.shape)
    grid = torch.tensor([0, 1, 2, 3, 4, 6, 8, 12], dtype=torch.float64)
    nib = torch.stack((p.codes.cpu() & 0xF, p.codes.cpu() >> 4), dim=-1).reshape(xt.shape)
    mag = grid[(nib & 7).long()]
    lo = grid[(torch.bucketize(q * (1 - 1e-2), grid, right=True) - 1).clamp(0, 7)]
    hi = grid[torch.bucketize(q * (1 + 1e-2), grid).clamp(0, 7)]
    assert bool(((mag >= lo) & (mag <= hi)).all())
    nonzero = xt.float() != 0
    assert bool((((nib & 8) != 0) == (xt.float() < 0))[nonzero].all())
    assert bool((nib[~nonzero] == 0).all())
    assert float((mag != grid[(torch.bucketize(q, grid) - 0).clamp(0, 7)]).double().mean()) > 0.05   # it does round both ways
    # determinism and sensitivity
    again = ops.quantize(xd, mode, col=col, sr=True, seed=seed, offset=offset)
    other_seed = ops.quantize(xd, mode, col=col, sr=True, seed=seed + 1, offset=offset)
    other_off = ops.quantize(xd, mode, col=col, sr=True, seed=seed, offset=offset + 1)
    assert torch.equal(p.codes, again.codes)
    assert not torch.equal(p.codes, other_seed.codes) and not torch.equal(p.codes, other_off.codes)
    if col:
        as_rows = ops.quantize(xd.t().contiguous(), mode, sr=True, seed=seed, offset=offset)
        assert torch.equal(p.codes, as_rows.codes) and torch.equal(p.scales, as_rows.scales)


@pytest.mark.parametrize("tag,mode", MODES)
def test_three_call_quant_draws_the_documented_philox_stream(tag, mode):
    """quant() without caller noise draws Philox4x32-10(counter = offset + e/4, key = seed), word e % 4, for
    element e; with the same draws fed to the oracle as explicit noise the values agree bit for bit.  This
    pins the device generator to the host implementation checked against the published known answers."""
    from metis_hip import quant_func
    from metis_hip.quant import _NVFP4Base
    from oracle import metis_oracle as O
    from philox_ref import uniform_for_elements
    q = quant_func["nvfp4e2m1b"]
    x = synthetic_activation(301, 32, 128)
    xin = _oracle_in(x, mode)
    keep = (_NVFP4Base.sr_seed, _NVFP4Base.sr_offset)
    _NVFP4Base.sr_seed, _NVFP4Base.sr_offset = 0x0BAD_CAFE_1234_5678, 1000
    try:
        xd = xin.cuda()
        s = q.get_scalar(xd)
        got = q.quant(xd, s)
    finally:
        _NVFP4Base.sr_seed, _NVFP4Base.sr_offset = keep
    u = torch.from_numpy(uniform_for_elements(x.numel(), 0x0BAD_CAFE_1234_5678, 1000, bf16=(mode == 1))).reshape(32, 128)
    want = O.quant(xin, O.get_scalar(xin), noise=u.to(xin.dtype))
    torch.cuda.synchronize()
    clamped = want.abs() > 6                                       # the reference's off-grid 8: kept by quant()
    assert same_bits(got.cpu(), want) or bool((got.cpu() == want)[~clamped].all())


@pytest.mark.parametrize("tag,mode", MODES)
def test_sr_is_unbiased(ops, tag, mode):
    """E[deq(SR(x))] = x for values inside the grid: mean over 4096 independent draws."""
    vals = torch.tensor([0.1, 0.3, 0.6, 0.9, 1.2, 1.7, 2.3, 2.9, 3.4, 4.4, 5.1, 5.8, -0.2, -1.1, -2.6, 6.0])
    x = vals.bfloat16().repeat(4096, 1).contiguous()              # block max 6 -> scalar 1 + 1e-9
    p = ops.quantize(x.cuda(), mode, sr=True, seed=42)
    deq = ops.dequantize(p, torch.float32).cpu()
    mean = deq.mean(0)
    step = torch.tensor([0.5] * 4 + [0.5] * 3 + [1.0] * 2 + [2.0] * 3 + [0.5, 0.5, 1.0, 2.0])
    sigma = step / 2 / (4096 ** 0.5)
    assert bool(((mean - x[0].float()).abs() <= 5 * sigma + 1e-6).all()), (mean, x[0])
    assert bool((deq[:, :15].std(0) > 0).all())                      # every off-grid value rounds both ways
    assert float(deq[:, 15].std()) == 0.0                            # the block maximum sits on the grid
    # different seeds give different streams, same seed the same codes
    p2 = ops.quantize(x.cuda(), mode, sr=True, seed=42)
    p3 = ops.quantize(x.cuda(), mode, sr=True, seed=43)
    assert torch.equal(p.codes, p2.codes) and not torch.equal(p.codes, p3.codes)


def test_errors_and_edges(ops):
    with pytest.raises(ValueError):
        ops.quantize(torch.zeros(4, 24, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        ops.quantize(torch.zeros(24, 32, dtype=torch.bfloat16, device="cuda"), col=True)
    p = ops.quantize(torch.zeros(0, 32, dtype=torch.bfloat16, device="cuda"))
    assert p.codes.shape == (0, 16) and p.scales.shape == (0, 2)
    # all-zero tensor: scalar = 1e-9 everywhere, scale byte 0x7E, codes 0
    z = ops.quantize(torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda"))
    torch.cuda.synchronize()
    assert int(z.codes.sum()) == 0 and bool((z.scales == 0x7E).all())
    assert float(z.unit.cpu()) == float(torch.tensor(1e-9) / 448)
    # strided rows (ld > cols)
    from oracle import metis_oracle as O
    base = synthetic_activation(5, 32, 256)
    view = base[:, 64:192]
    from metis_hip import _lib
    L = _lib.load()
    xd = base.cuda()
    codes = torch.empty(32, 64, dtype=torch.uint8, device="cuda")
    scales = torch.empty(32, 8, dtype=torch.uint8, device="cuda")
    unit = torch.empty(1, dtype=torch.float32, device="cuda")
    ws = torch.zeros(L.metis_nvfp4_workspace_bytes(32, 128), dtype=torch.uint8, device="cuda")
    rc = L.metis_nvfp4_quant_row(xd.data_ptr() + 64 * 2, 32, 128, 256, 0, codes.data_ptr(), scales.data_ptr(),
                                 unit.data_ptr(), ws.data_ptr(), ws.numel(), None)
    assert rc == 0
    oc, os_, ou, _ = O.nvfp4_pack(view.float().contiguous())
    torch.cuda.synchronize()
    assert torch.equal(codes.cpu(), oc) and torch.equal(scales.cpu(), os_) and float(unit.cpu()) == float(ou)
    # error codes straight from the C ABI
    assert L.metis_nvfp4_quant_row(None, 1, 16, 16, 0, codes.data_ptr(), scales.data_ptr(), unit.data_ptr(),
                                   ws.data_ptr(), ws.numel(), None) == _lib.E_ARG
    assert L.metis_nvfp4_quant_row(xd.data_ptr(), 32, 128, 256, 0, codes.data_ptr(), scales.data_ptr(),
                                   unit.data_ptr(), ws.data_ptr(), 16, None) == _lib.E_WORKSPACE
    assert L.metis_nvfp4_quant_row(xd.data_ptr(), 32, 24, 256, 0, codes.data_ptr(), scales.data_ptr(),
                                   unit.data_ptr(), ws.data_ptr(), ws.numel(), None) == _lib.E_SHAPE


@pytest.mark.parametrize("tag,mode", MODES)
def test_full_size_config1(ops, tag, mode):
    """bf16 [8192, 4096], 0.1 % outlier channels: bit-exact against the C restatement, plus the
    size-independent properties (idempotence of QDQ on its own output, odd symmetry)."""
    from oracle import c_oracle as C
    x = synthetic_activation(1001, 8192, 4096)
    xd = x.cuda()
    p = ops.quantize(xd, mode)
    cc, cs, cu, _ = C.nvfp4_pack(x, mode)
    _check_packed(p, cc, cs, cu, "config 1")
    deq = ops.dequantize(p, torch.bfloat16)
    ob, of = C.nvfp4_dequant(cc, cs, cu, mode)
    assert same_bits(deq.cpu(), ob)
    pn = ops.quantize(-xd, mode)
    torch.cuda.synchronize()
    assert torch.equal(pn.scales, p.scales) and torch.equal(pn.unit, p.unit)
    nz = (xd != 0)
    flip = torch.where(nz, 8, 0).to(torch.uint8)
    flip = flip[:, 0::2] | (flip[:, 1::2] << 4)
    assert torch.equal(pn.codes, p.codes ^ flip)


@pytest.mark.parametrize("tag,mode", MODES)
def test_round_trip_from_one_call(ops, tag, mode):
    """metis_nvfp4_quant_dequant_row: codes, scale bytes, unit and the dequantized bf16 tensor of quant.py:6-36 from one
    call whose second launch forms bytes and dequantized values together.  Config 1 at full size bit for bit against
    the C restatement; ragged and tiny shapes against the separate calls (block counts that are not multiples of four,
    signed zeros, an all-zero tensor)."""
    from oracle import c_oracle as C
    x = synthetic_activation(1001, 8192, 4096)
    p, deq = ops.quantize_dequantize(x.cuda(), mode)
    cc, cs, cu, _ = C.nvfp4_pack(x, mode)
    _check_packed(p, cc, cs, cu, "config 1 round trip")
    ob, _ = C.nvfp4_dequant(cc, cs, cu, mode)
    assert same_bits(deq.cpu(), ob)
    for k, (r, c) in enumerate([(1, 16), (3, 48), (7, 80), (64, 256), (1000, 96), (300, 7168), (5, 16)]):
        y = synthetic_activation(4100 + k, r, c)
        y[0, ::5] = -0.0
        y[-1, 1::3] = -1e-5
        if k == 6:
            y.zero_()
        y = y.cuda()
        ref = ops.quantize(y, mode)
        want = ops.dequantize(ref, torch.bfloat16)
        got_p, got = ops.quantize_dequantize(y, mode)
        _check_packed(got_p, ref.codes.cpu(), ref.scales.cpu(), ref.unit.cpu(), f"round trip {r}x{c} {tag}")
        assert same_bits(got.cpu(), want.cpu()), (r, c, tag)
    # the quantizer class takes this path for bf16 tensors
    from metis_hip import quant_func
    if mode == 1:
        z = synthetic_activation(4200, 24, 64).reshape(8, 3, 64).cuda()
        q = quant_func["nvfp4e2m1bnosr"].quantize_dequantize(z)
        assert q.shape == z.shape and same_bits(q.reshape(24, 64).cpu(), ops.dequantize(ops.quantize(z, 1), torch.bfloat16).cpu())


@pytest.mark.parametrize("tag,mode", MODES)
def test_deferred_scale_bytes_give_the_same_packed_tensor(ops, tag, mode):
    """deferred=True runs the first launch only and parks the block maxima with the packed tensor.  Whoever reads
    `scales` / `unit` later gets the bytes of the two-launch path; the tiled expansion forms them itself (it never
    materialises them) and is bit-equal to the expansion of the eager tensor, in both operand formats; and a parked
    buffer that is all garbage beforehand changes nothing (every entry a reader folds is written by the call)."""
    from helpers import untile
    shapes = [(8192, 4096), (16, 32), (64, 256), (4096, 1536), (1000, 96), (3, 32), (16384, 4096), (300, 7168)]
    for k, (r, c) in enumerate(shapes):
        x = synthetic_activation(700 + k, r, c).cuda()
        ref = ops.quantize(x, mode)
        got = ops.quantize(x, mode, deferred=True)
        assert got.deferred is not None and got.__dict__.get("_scales") is None
        for fmt in (0, 1):
            if fmt == 1 and mode == 0:
                continue                                          # bf16 operands belong to tensors packed in bf16 arithmetic
            lazy = ops.quantize(x, mode, deferred=True)
            a = ops.expand_tiled(lazy, cache=False, mode=fmt)
            b = ops.expand_tiled(ref, cache=False, mode=fmt)
            assert torch.equal(a, b), f"tiled operand differs, shape {r}x{c} {tag} format {fmt}"
            assert lazy.__dict__.get("_scales") is None and lazy.__dict__["_unit_ready"]
            assert float(lazy.unit.cpu()) == float(ref.unit.cpu())
            assert lazy.__dict__.get("_scales") is None               # reading the unit after the expansion launches nothing
            _check_packed(lazy, ref.codes.cpu(), ref.scales.cpu(), ref.unit.cpu(), f"after expansion, shape {r}x{c} {tag}")
        _check_packed(got, ref.codes.cpu(), ref.scales.cpu(), ref.unit.cpu(), f"shape {r}x{c} {tag}")
        assert torch.equal(ops.dequantize(got, torch.bfloat16), ops.dequantize(ref, torch.bfloat16))
    # through the C ABI with a poisoned parked buffer
    from metis_hip import _lib
    L = _lib.load()
    x = synthetic_activation(777, 48, 64).cuda()
    ref = ops.quantize(x, mode)
    parked = torch.full((L.metis_nvfp4_deferred_bytes(48, 64),), 0x7f, dtype=torch.uint8, device="cuda")
    codes = torch.empty(48, 32, dtype=torch.uint8, device="cuda")
    scales = torch.empty(48, 4, dtype=torch.uint8, device="cuda")
    unit = torch.empty(1, dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert L.metis_nvfp4_quant_row_deferred(x.data_ptr(), 48, 64, mode, None, codes.data_ptr(), parked.data_ptr(), parked.numel(), st) == 0
    assert L.metis_nvfp4_deferred_scales(parked.data_ptr(), 48, 64, mode, scales.data_ptr(), unit.data_ptr(), st) == 0
    torch.cuda.synchronize()
    assert torch.equal(codes, ref.codes) and torch.equal(scales, ref.scales) and float(unit.cpu()) == float(ref.unit.cpu())
    assert L.metis_nvfp4_quant_row_deferred(x.data_ptr(), 48, 64, mode, None, codes.data_ptr(), parked.data_ptr(), 16, st) == _lib.E_WORKSPACE


@pytest.mark.parametrize("tag,mode", MODES)
def test_single_launch_variant_matches_two_launch_path(ops, tag, mode):
    """The single-launch kernel (grid-wide maximum through a tree of device-scope atomics) gives the same
    bytes as the two-launch path, call after call on one workspace (the generation tag
    advances each time) and across sizes that change the number of groups and members."""
    shapes = [(8192, 4096), (16, 16), (64, 256), (4096, 1536), (16384, 4096), (1000, 48), (8192, 4096), (2, 32)]
    for k, (r, c) in enumerate(shapes):
        x = synthetic_activation(300 + k, r, c).cuda()
        ref = ops.quantize(x, mode)
        for rep in range(3):
            got = ops.quantize(x, mode, resident=True)
            _check_packed(got, ref.codes.cpu(), ref.scales.cpu(), ref.unit.cpu(), f"shape {r}x{c} rep {rep} {tag}")


@pytest.mark.parametrize("tag,mode", MODES)
def test_single_launch_workgroups_that_give_up_are_finished_by_the_last_one(ops, tag, mode):
    """The grid-wide wait is bounded, and giving up loses nothing: with a spin limit of one poll most workgroups stop
    waiting before the last one has arrived, park their block maxima and leave; the last workgroup writes their scale
    bytes.  Same bytes as the two-launch path, call after call on one workspace, and the workspace stays usable."""
    from metis_hip import _lib
    L = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    for k, (rows, cols) in enumerate([(16384, 4096), (8192, 4096), (4096, 1536), (64, 256), (16384, 4096)]):
        x = synthetic_activation(777 + k, rows, cols).cuda()
        ref = ops.quantize(x, mode)
        ws = torch.zeros(L.metis_nvfp4_workspace_bytes(rows, cols), dtype=torch.uint8, device="cuda")
        for limit in (1, 0, 1, 1, 0):
            codes, scales = torch.zeros_like(ref.codes), torch.full_like(ref.scales, 0xAA)
            unit = torch.zeros(1, device="cuda")
            rc = L.metis_nvfp4_quant_row_resident(x.data_ptr(), rows, cols, mode, codes.data_ptr(), scales.data_ptr(), unit.data_ptr(),
                                                  ws.data_ptr(), ws.numel(), limit, st)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(unit, ref.unit) and torch.equal(codes, ref.codes), (rows, cols, limit, tag)
            assert torch.equal(scales, ref.scales), (rows, cols, limit, tag, int((scales != ref.scales).sum()))
        # counters and maxima of the tree are clean again; the generation counter has advanced once per call (what
        # stays behind are tagged words -- published results, flags of workgroups that gave up -- which a later call ignores)
        sync = ws[16384:16384 + 260 * 256].view(torch.int32)
        assert int(sync[0]) == 5 and int(sync[4:6].abs().sum()) == 0 and int(sync[64:2176].abs().sum()) == 0
        # (whether any workgroup actually left depends on timing: flags at sync[4224:] tell, typically most of them at
        # the large shapes; the assertions above hold either way)


@pytest.mark.parametrize("tag,mode", MODES)
def test_signed_zeros_and_negatives_that_round_to_zero(ops, tag, mode):
    """The reference's sign comes from sign(x): -0.0 has no sign (nibble 0), a negative value whose
    magnitude rounds to zero keeps it (nibble 8).  Both sit next to ordinary values in every block."""
    from oracle import metis_oracle as O
    x = synthetic_activation(61, 64, 256)
    x[:, 0::7] = -0.0
    x[:, 1::7] = 0.0
    x[:, 2::7] = -1e-4
    x[:, 3::7] = 1e-4
    x[3] = 0.0
    x[4] = -0.0
    codes, scales, unit, _ = O.nvfp4_pack(_oracle_in(x, mode))
    _check_packed(ops.quantize(x.cuda(), mode), codes, scales, unit, tag)
    ct, st, ut, _ = O.nvfp4_pack_col(_oracle_in(x, mode))
    _check_packed(ops.quantize(x.cuda(), mode, col=True), ct, st, ut, tag + " col")


def test_offsets_beyond_32_bits(ops):
    """2.4 GB input, 75 M blocks: byte offsets pass 2^31 and 2^32.  The tensor is a 1024-row pattern
    repeated 36 times, so every repetition must carry the pattern's own codes and scale bytes (the
    tensor-wide unit is the same) -- checked against the oracle on the pattern."""
    from oracle import metis_oracle as O
    pat = synthetic_activation(71, 1024, 32768)
    codes, scales, unit, _ = O.nvfp4_pack(pat.float())
    x = pat.cuda().repeat(36, 1)
    assert x.numel() * 2 > 2 ** 31
    p = ops.quantize(x, 0)
    torch.cuda.synchronize()
    assert float(p.unit.cpu()) == float(unit)
    cd, sd = codes.cuda(), scales.cuda()
    for rep in (0, 17, 35):
        assert torch.equal(p.codes[rep * 1024:(rep + 1) * 1024], cd), rep
        assert torch.equal(p.scales[rep * 1024:(rep + 1) * 1024], sd), rep
    assert torch.equal(p.codes.view(36, -1), cd.view(1, -1).expand(36, -1))
    del p
    pc = ops.quantize(x, 0, col=True)                         # [32768, 36864 / 2]: blocks run down the repeated rows
    ct, st, ut, _ = O.nvfp4_pack_col(pat.float())
    torch.cuda.synchronize()
    assert float(pc.unit.cpu()) == float(ut)
    assert torch.equal(pc.codes.view(32768, 36, -1), ct.cuda().view(32768, 1, -1).expand(-1, 36, -1))
    assert torch.equal(pc.scales.view(32768, 36, -1), st.cuda().view(32768, 1, -1).expand(-1, 36, -1))


# ---------------------------------------------------------------------------------------------
# binary32 tensors whose values are not bf16 values (binary32 arithmetic only): gradients and
# activations downstream of a layer that ran with compute_dtype=float32
# ---------------------------------------------------------------------------------------------
def _f32_valued(seed, rows, cols):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g))
    x.view(-1)[::211] *= 37.0                                    # outliers
    x.view(-1)[::97] = 0
    x.view(-1)[5::389] = -0.0
    assert not torch.equal(x, x.bfloat16().float())
    return x


@pytest.mark.parametrize("shape", [(256, 512), (1, 16), (37, 48), (1000, 1536)])
def test_f32_input_rne_row(ops, shape):
    from oracle import c_oracle as C, metis_oracle as O
    x = _f32_valued(400 + shape[0], *shape)
    p = ops.quantize(x.cuda(), 0)
    codes, scales, unit, _ = O.nvfp4_pack(x)                    # torch restatement of the reference
    _check_packed(p, codes, scales, unit, str(shape))
    cc, cs, cu, _ = C.nvfp4_pack(x, 2)                          # C restatement
    _check_packed(p, cc, cs, cu, f"C {shape}")
    assert p.mode == 0
    want = O.nvfp4_qdq(x)
    assert same_bits(ops.dequantize(p, torch.float32).cpu(), want)


@pytest.mark.parametrize("shape", [(64, 96), (256, 512), (48, 1000)])
def test_f32_input_rne_col(ops, shape):
    from oracle import metis_oracle as O
    x = _f32_valued(410 + shape[0], *shape)
    p = ops.quantize(x.cuda(), 0, col=True)
    codes, scales, unit, _ = O.nvfp4_pack_col(x)
    assert (p.rows, p.cols) == (shape[1], shape[0])
    _check_packed(p, codes, scales, unit, str(shape))


def test_f32_input_ties_and_their_neighbours(ops):
    """Block scalar 1 (maximum 6; 1e-9 is below half an ulp), so |x| / 0.5 is exact: every rounding
    threshold of the element rule, its binary32 neighbours on both sides, and the three quotients where
    the rule's second rounding matters (5, 7, 10 and their neighbours)."""
    from oracle import c_oracle as C, metis_oracle as O
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0])
    vals = torch.cat([ties, torch.nextafter(ties, torch.zeros(())), torch.nextafter(ties, torch.full((), 9.0))])
    vals = torch.cat([vals, -vals])
    rows = []
    for i in range(0, vals.numel(), 15):
        chunk = vals[i:i + 15]
        rows.append(torch.cat([torch.tensor([6.0]), chunk, torch.zeros(15 - chunk.numel())]))
    x = torch.stack(rows).contiguous()
    p = ops.quantize(x.cuda(), 0)
    codes, scales, unit, _ = O.nvfp4_pack(x)
    _check_packed(p, codes, scales, unit, "ties")
    cc, cs, cu, _ = C.nvfp4_pack(x, 2)
    _check_packed(p, cc, cs, cu, "ties C")


@pytest.mark.parametrize("col", [False, True])
def test_f32_input_sr_explicit_noise(ops, col):
    from oracle import metis_oracle as O
    x = _f32_valued(420, 128, 256)
    u = torch.rand(128, 256, generator=torch.Generator().manual_seed(421))
    p = ops.quantize(x.cuda(), 0, col=col, sr=True, noise=u.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(x, u)
    _check_packed(p, codes, scales, unit, f"sr col={col}")


@pytest.mark.parametrize("col", [False, True])
def test_f32_input_sr_internal_stream(ops, col):
    """Own random stream: scale bytes and unit bit-exact, every code a grid neighbour of the exact quotient,
    a function of (seed, offset) only, unbiased in the mean."""
    from oracle import metis_oracle as O
    x = _f32_valued(430, 64, 128)
    xd = x.cuda()
    p = ops.quantize(xd, 0, col=col, sr=True, seed=99, offset=5)
    xt = x.t().contiguous() if col else x
    _, scales, unit, _ = O.nvfp4_pack(xt)
    torch.cuda.synchronize()
    assert torch.equal(p.scales.cpu(), scales) and float(p.unit.cpu()) == float(unit)
    scalar = O.block_scalars(xt).double().reshape(xt.shape[0], -1, 1)
    q = (xt.double().abs().reshape(xt.shape[0], -1, 16) / (scalar / 2)).reshape(xt.shape)
    grid = torch.tensor([0, 1, 2, 3, 4, 6, 8, 12], dtype=torch.float64)
    nib = torch.stack((p.codes.cpu() & 0xF, p.codes.cpu() >> 4), dim=-1).reshape(xt.shape)
    mag = grid[(nib & 7).long()]
    lo = grid[(torch.bucketize(q * (1 - 1e-6), grid, right=True) - 1).clamp(0, 7)]
    hi = grid[torch.bucketize(q * (1 + 1e-6), grid).clamp(0, 7)]
    assert bool(((mag >= lo) & (mag <= hi)).all())
    assert bool((((nib & 8) != 0) == (xt < 0))[xt != 0].all())
    assert bool((nib[xt == 0] == 0).all())                          # +0.0 and -0.0 both give the all-zero nibble
    again = ops.quantize(xd, 0, col=col, sr=True, seed=99, offset=5)
    assert torch.equal(p.codes, again.codes)
    # unbiased: mean over many seeds of the dequantized value approaches x
    acc = torch.zeros_like(xt, dtype=torch.float64)
    n = 256
    for sd in range(n):
        acc += ops.dequantize(ops.quantize(xd, 0, col=col, sr=True, seed=1000 + sd), torch.float32).cpu().double()
    step = (scalar / 2 * 4).expand(-1, -1, 16).reshape(xt.shape)     # widest grid interval in units of x
    assert float(((acc / n - xt.double()).abs() / step).max()) < 0.2


def test_f32_input_argument_checks():
    from metis_hip import _lib
    lib = _lib.load()
    x = torch.zeros(16, 64, dtype=torch.float32, device="cuda")
    codes = torch.empty(16, 32, dtype=torch.uint8, device="cuda")
    scales = torch.empty(16, 4, dtype=torch.uint8, device="cuda")
    unit = torch.empty(1, dtype=torch.float32, device="cuda")
    need = lib.metis_nvfp4_workspace_bytes(16, 64)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    call = lambda ptr, ld, mode: lib.metis_nvfp4_quant_row(ptr, 16, 64, ld, mode, codes.data_ptr(), scales.data_ptr(),
                                                           unit.data_ptr(), ws.data_ptr(), need, st)
    assert call(x.data_ptr(), 64, 2) == 0
    assert call(x.data_ptr(), 66, 2) == _lib.E_ARG               # rows must stay 16-byte aligned
    assert call(x.data_ptr() + 4, 64, 2) == _lib.E_ARG
    assert call(x.data_ptr(), 64, 3) == _lib.E_ARG               # unknown mode
    torch.cuda.synchronize()


@pytest.mark.parametrize("tag,mode", MODES + [("f32", 2)])
def test_col_quant_large_ragged_tensors(ops, tag, mode):
    """A tensor of many tiles, ragged in both directions (rows not a multiple of the 256-row tile, columns not a
    multiple of the 64-column tile), plain, centred and with the library's own stochastic rounding."""
    from oracle import metis_oracle as O
    rows, cols = 4096 + 48, 8192 + 6
    g = torch.Generator().manual_seed(77)
    x = torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g))
    x.view(-1)[::101] = 0
    xin = x if mode == 2 else x.bfloat16()
    arith = xin if mode == 1 else xin.float()
    p = ops.quantize(xin.cuda(), 1 if mode == 1 else 0, col=True)
    codes, scales, unit, _ = O.nvfp4_pack_col(arith)
    _check_packed(p, codes, scales, unit, f"wide col {tag}")
    me = arith.mean(dim=0)
    p = ops.quantize(xin.cuda(), 1 if mode == 1 else 0, col=True, center=me.cuda())
    codes, scales, unit, _ = O.nvfp4_pack_col(arith - me)
    _check_packed(p, codes, scales, unit, f"wide col centred {tag}")
    # own-stream stochastic rounding is indexed by output block: equal to row packing of the transpose
    a = ops.quantize(xin.cuda(), 1 if mode == 1 else 0, col=True, sr=True, seed=5, offset=9)
    b = ops.quantize(xin.cuda().t().contiguous(), 1 if mode == 1 else 0, sr=True, seed=5, offset=9)
    assert torch.equal(a.codes, b.codes) and torch.equal(a.scales, b.scales)


@pytest.mark.parametrize("tag,mode", MODES + [("f32", 2)])
@pytest.mark.parametrize("shape", [(16, 16), (48, 80), (256, 64), (1008, 1552), (4096 + 48, 2048 + 16), (4096, 8960)])
def test_both_packings_in_one_pass_equal_the_two_calls(ops, tag, mode, shape):
    """Row-blocked and column-blocked stochastic packings of one tensor from one kernel: the same bytes as the row call
    and the column call with the same seed and offsets (tiles ragged in both directions, single block, one tile, and the
    output gradient of the config-4 projection at full size)."""
    rows, cols = shape
    g = torch.Generator().manual_seed(1234 + rows)
    x = torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g))
    x.view(-1)[::53] = 0
    xin = (x if mode == 2 else x.bfloat16()).cuda()
    km = 1 if mode == 1 else 0
    seed, o_row, o_col = 0x9E3779B97F4A7C15, (1 << 33) + 7, 12345
    pr, pc = ops.quantize_both_sr(xin, km, seed=seed, offset_row=o_row, offset_col=o_col)
    want_r = ops.quantize(xin, km, sr=True, seed=seed, offset=o_row)
    want_c = ops.quantize(xin, km, col=True, sr=True, seed=seed, offset=o_col)
    torch.cuda.synchronize()
    for got, want, what in ((pr, want_r, "rows"), (pc, want_c, "columns")):
        assert (got.rows, got.cols) == (want.rows, want.cols)
        assert torch.equal(got.codes, want.codes), f"{what} codes {tag} {shape}: {(got.codes != want.codes).sum().item()} bytes"
        assert torch.equal(got.scales, want.scales), f"{what} scale bytes {tag} {shape}"
        assert torch.equal(got.unit, want.unit), f"{what} unit {tag} {shape}"
    # a strided view (row stride larger than the width) reads the same values
    if cols >= 32:
        wide = torch.zeros(rows, cols + 64, dtype=xin.dtype, device="cuda")
        wide[:, :cols] = xin
        x2, kmode = wide[:, :cols], (2 if mode == 2 else km)
        from metis_hip import _lib
        L = _lib.load()
        outs = [torch.empty_like(t_) for t_ in (pr.codes, pr.scales, pr.unit, pc.codes, pc.scales, pc.unit)]
        ws = torch.zeros(2 * L.metis_nvfp4_workspace_bytes(rows, cols), dtype=torch.uint8, device="cuda")
        rc = L.metis_nvfp4_quant_sr_both(x2.data_ptr(), rows, cols, x2.stride(0), kmode, seed, o_row, o_col, *[o.data_ptr() for o in outs],
                                         ws.data_ptr(), ws.numel(), None)
        assert rc == 0
        torch.cuda.synchronize()
        for o, w in zip(outs, (pr.codes, pr.scales, pr.unit, pc.codes, pc.scales, pc.unit)):
            assert torch.equal(o, w)


def test_both_packings_argument_checks(ops):
    from metis_hip import _lib
    L = _lib.load()
    x = torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda")
    o = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    u = torch.zeros(2, dtype=torch.float32, device="cuda")
    ws = torch.zeros(2 * L.metis_nvfp4_workspace_bytes(64, 64), dtype=torch.uint8, device="cuda")

    def call(rows, cols, ld, mode=0, ptr=None, wsn=None):
        return L.metis_nvfp4_quant_sr_both(x.data_ptr() if ptr is None else ptr, rows, cols, ld, mode, 1, 0, 0, o.data_ptr(), o.data_ptr() + 8192,
                                           u.data_ptr(), o.data_ptr() + 16384, o.data_ptr() + 32768, u.data_ptr() + 4, ws.data_ptr(),
                                           ws.numel() if wsn is None else wsn, None)

    assert call(64, 64, 64) == 0
    assert call(0, 64, 64) == 0 and call(64, 0, 64) == 0           # nothing to do
    assert call(40, 64, 64) == _lib.E_SHAPE and call(64, 40, 64) == _lib.E_SHAPE
    assert call(64, 64, 60) == _lib.E_ARG                          # row stride below the width
    assert call(32, 32, 36) == _lib.E_ARG                          # rows not 16-byte aligned
    assert call(64, 64, 64, ptr=x.data_ptr() + 2) == _lib.E_ARG
    assert call(64, 64, 64, mode=7) == _lib.E_ARG
    assert call(64, 64, 64, wsn=ws.numel() // 2) == _lib.E_WORKSPACE  # one workspace is not enough for two sets of maxima
    torch.cuda.synchronize()
