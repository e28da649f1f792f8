"""GPU parity of the block-scaled NVFP4 GEMM (forward with low-rank extension, dgrad, wgrad).

Bar (P32): relative Frobenius error <= 2e-3 between bf16(ours) and bf16(oracle); the oracle is
the reference formula evaluated in fp64 on operands dequantized from the (bit-exact) packed
tensors, plus the op-for-op torch restatement on small shapes.
"""
import pytest
import torch

from helpers import rel_fro, synthetic_activation

pytestmark = pytest.mark.gpu

TOL = 2e-3


def _weights(seed, n, k, scale=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, k, generator=g) * scale).bfloat16()


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 512), (100, 132, 96), (1, 64, 32), (64, 3584, 1536),
                                   (300, 260, 4096),
                                   # skinny path (M <= 64): narrow and wide runs, ragged N, one and two row tiles
                                   (7, 100, 64), (33, 96, 320), (32, 2052, 768), (1, 3584, 3584), (64, 4736, 3584),
                                   (16, 1536, 8960)])
def test_gemm_against_fp64_of_dequantized_operands(M, N, K):
    from metis_hip import ops
    x = synthetic_activation(10 + M, M, K)
    w = _weights(11 + N, N, K)
    px, pw = ops.quantize(x.cuda()), ops.quantize(w.cuda())
    out = ops.linear_fwd(px, pw)
    xq = ops.dequantize(px, torch.float32).double()
    wq = ops.dequantize(pw, torch.float32).double()
    want = (xq @ wq.T)
    torch.cuda.synchronize()
    assert rel_fro(out.cpu(), want.cpu().bfloat16()) <= TOL
    out32 = ops.linear_fwd(px, pw, out_dtype=torch.float32)
    assert rel_fro(out32.cpu(), want.cpu()) <= 1e-5           # binary32 accumulation only


def test_gemm_tiny_blocks_with_subnormal_scales():
    """Blocks 2^-12 below the tensor maximum get subnormal E4M3 scale bytes (1..7)."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 128, generator=g)
    x[:, 32:64] *= 2.0 ** -14
    x[:, 64:80] *= 2.0 ** -11
    w = torch.randn(64, 128, generator=g)
    w[:, 32:48] *= 2.0 ** -13
    px, pw = ops.quantize(x.bfloat16().cuda()), ops.quantize(w.bfloat16().cuda())
    torch.cuda.synchronize()
    assert int(((px.scales > 0) & (px.scales < 8)).sum()) > 0
    out = ops.linear_fwd(px, pw, out_dtype=torch.float32)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T
    assert rel_fro(out.cpu(), want.cpu()) <= 1e-5


@pytest.mark.parametrize("M,N,K,r", [(128, 256, 256, 32), (200, 192, 512, 64), (48, 260, 256, 64), (5, 96, 192, 32),
                                     (64, 512, 1024, 320)])
def test_metis_forward_with_lowrank_extension_and_bias(M, N, K, r):
    """out = (X V^T * s) U^T + QDQ(X) QDQ(R)^T + b against the op-for-op oracle (P32)."""
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = synthetic_activation(20 + M, M, K)
    w = _weights(21, N, K) .float()
    g = torch.Generator().manual_seed(22)
    a = torch.linalg.qr(torch.randn(N, 8, generator=g))[0]
    b = torch.linalg.qr(torch.randn(K, 8, generator=g))[0]
    w = w + (a * 5.0) @ b.T
    U, S, Vh = torch.linalg.svd(w, full_matrices=False)
    u, s, v = U[:, :r].bfloat16(), S[:r].bfloat16(), Vh[:r].bfloat16()
    res = (w - (U[:, :r] * S[:r]) @ Vh[:r]).bfloat16()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16()
    want = O.metis_forward(x, v, s, u, res, bias, p32=True)
    xd = x.cuda()
    t = (torch.matmul(xd, v.cuda().T) * s.cuda())             # bf16 low-rank projection (library GEMM)
    out = ops.linear_fwd(ops.quantize(xd), ops.quantize(res.cuda()), t=t, u=u.cuda(), bias=bias.cuda())
    torch.cuda.synchronize()
    assert rel_fro(out.cpu(), want) <= TOL


def test_dgrad_and_wgrad():
    """gX = deq(dY) deq(W); gW = deq(dY)^T deq(X) with operands blocked along the contraction."""
    from metis_hip import ops
    L, N, K = 256, 192, 320
    x = synthetic_activation(30, L, K)
    w = _weights(31, N, K)
    g = torch.Generator().manual_seed(32)
    dy = (torch.randn(L, N, generator=g) * 1e-3).bfloat16()
    dyd, wd, xd = dy.cuda(), w.cuda(), x.cuda()
    p_dy = ops.quantize(dyd, sr=True, seed=1)                 # blocks along N
    p_wt = ops.quantize(wd, col=True)                         # W^T [K, N], blocks along N
    gx = ops.linear_dgrad(p_dy, p_wt, out_dtype=torch.float32)
    want_gx = ops.dequantize(p_dy, torch.float32).double() @ ops.dequantize(p_wt, torch.float32).double().T
    assert gx.shape == (L, K) and rel_fro(gx.cpu(), want_gx.cpu()) <= 1e-5
    p_dyt = ops.quantize(dyd, col=True, sr=True, seed=2)      # dY^T [N, L], blocks along L
    p_xt = ops.quantize(xd, col=True, sr=True, seed=3)        # X^T [K, L]
    gw = ops.linear_wgrad(p_dyt, p_xt)
    want_gw = ops.dequantize(p_dyt, torch.float32).double() @ ops.dequantize(p_xt, torch.float32).double().T
    assert gw.shape == (N, K) and gw.dtype == torch.float32 and rel_fro(gw.cpu(), want_gw.cpu()) <= 1e-5
    # and both stay close to the unquantized gradients (FP4 noise level, not a parity bar)
    assert rel_fro(gx.cpu(), dy.double() @ w.double()) < 0.25
    assert rel_fro(gw.cpu(), dy.double().T @ x.double()) < 0.25


def test_expanded_path_is_bit_identical_to_packed_path():
    """metis_linear_fwd_expanded on exact f16 expansions == metis_linear_fwd on packed operands
    (with K unsplit: splitting changes the order of the binary32 additions)."""
    from metis_hip import ops
    M, N, K, r = 512, 768, 1024, 64
    x = synthetic_activation(40, M, K)
    w = _weights(41, N, K)
    g = torch.Generator().manual_seed(42)
    t = torch.randn(M, r, generator=g).bfloat16().cuda()
    u = torch.randn(N, r, generator=g).bfloat16().cuda()
    bias = torch.randn(N, generator=g).bfloat16().cuda()
    px, pw = ops.quantize(x.cuda()), ops.quantize(w.cuda())
    a = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, expanded=False, split_k=False)
    b = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, expanded=True)
    assert torch.equal(a, b)
    # the expansion itself: e2m1 * e4m3 * 2^-8, exact
    e = ops.expand(px).float() * 256.0 * px.unit
    assert rel_fro(e.cpu(), ops.dequantize(px, torch.float32).cpu()) < 1e-6


@pytest.mark.parametrize("M,N,K,r,bias_f32", [(512, 768, 1024, 64, False), (300, 260, 32, 0, False), (256, 256, 96, 32, True),
                                              (1000, 516, 2112, 64, True), (2048, 1024, 4096, 0, False)])
def test_tiled_pipelined_path_is_bit_identical_to_packed_path(M, N, K, r, bias_f32):
    """metis_linear_fwd_tiled (operands expanded once into the tiled binary16 layout, direct-to-LDS ring) against
    metis_linear_fwd on the packed operands, unsplit: the same exact products summed in the same order.  Covers
    ragged M and N (tile rows padded with zeros, rows clamped), K shorter than the ring, and both bias and output
    types; and against the double-precision product of the dequantized operands."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(4000 + M)
    x = synthetic_activation(60 + M, M, K).cuda()
    w = _weights(61 + N, N, K).cuda()
    t = u = None
    if r:
        t = torch.randn(M, r, generator=g).bfloat16().cuda()
        u = torch.randn(N, r, generator=g).bfloat16().cuda()
    bias = torch.randn(N, generator=g)
    bias = bias.cuda() if bias_f32 else bias.bfloat16().cuda()
    px, pw = ops.quantize(x), ops.quantize(w)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T + bias.double()
    if r:
        want = want + t.double() @ u.double().T
    for dt in (torch.float32, torch.bfloat16):
        a = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=dt, split_k=False)
        b = ops.linear_fwd_tiled(px, pw, t=t, u=u, bias=bias, out_dtype=dt, split_k=False)
        c = ops.linear_fwd_tiled(px, pw, t=t, u=u, bias=bias, out_dtype=dt)                # K split where the shape has few tiles
        torch.cuda.synchronize()
        assert rel_fro(b.cpu(), want.cpu().to(dt)) <= (1e-5 if dt == torch.float32 else TOL)
        assert rel_fro(c.cpu(), want.cpu().to(dt)) <= (1e-5 if dt == torch.float32 else TOL)
        assert torch.equal(a, b), f"{(a != b).sum().item()} of {a.numel()} elements differ ({dt})"
    # the tiled expansion holds exactly the values of the row-major one
    e = ops.expand(px)
    tiles = ops.expand_tiled(px, cache=False).view(torch.float16).reshape(-1, K // 32, 16, 4, 8)
    rows = torch.arange(16, device="cuda")
    swz = ((rows >> 2) & 1) | ((((rows >> 1) ^ (rows >> 3)) & 1) << 1)
    slot = torch.arange(4, device="cuda")[None, :] ^ swz[:, None]                  # [16 rows, 4 chunks] -> slot
    unswz = torch.gather(tiles, 3, slot[None, None, :, :, None].expand(tiles.shape[0], tiles.shape[1], 16, 4, 8))
    flat = unswz.permute(0, 2, 1, 3, 4).reshape(-1, K)[:M]
    assert torch.equal(flat, e)


@pytest.mark.parametrize("M,N,K,r,with_bias", [(512, 768, 1024, 64, True), (300, 260, 96, 0, True), (1024, 512, 8192, 32, False),
                                               (2048, 3584, 2048, 64, True), (4096, 4352, 1024, 32, True)])
def test_tiled_path_with_reference_rounding_in_bf16_arithmetic(M, N, K, r, with_bias):
    """Both operands packed in bf16 arithmetic, reference_rounding: the pipelined kernel multiplies the reference's own
    bf16 dequantized values and rounds where its all-bf16 forward rounds (matmul result, bias add, final sum).  Checked
    against that evaluation carried out in double precision between the roundings: the kernel's binary32 accumulation
    can only move a result that sits on a bf16 rounding boundary.  Shapes cover unsplit tiles, K split over the whole
    grid (1024 x 512 x 8192), and a split last round (4096 x 4352)."""
    from metis_hip import _lib, ops
    g = torch.Generator().manual_seed(5000 + M)
    x = synthetic_activation(70 + M, M, K).cuda()
    w = _weights(71 + N, N, K).cuda()
    t = u = None
    if r:
        t = torch.randn(M, r, generator=g).bfloat16().cuda()
        u = (torch.randn(N, r, generator=g) * 0.05).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda() if with_bias else None
    px, pw = ops.quantize(x, 1), ops.quantize(w, 1)
    xq, wq = ops.dequantize(px, torch.bfloat16).double(), ops.dequantize(pw, torch.bfloat16).double()   # the reference's QDQ values
    want = (xq @ wq.T).bfloat16()
    if bias is not None:
        want = (want.float() + bias.float()).bfloat16()
    want = want.double()
    if r:
        want = want + t.double() @ u.double().T
    want = want.bfloat16()
    if K >= 2048 or M * N >= 4096 * 4096:
        assert _lib.load().metis_linear_tiled_workspace_bytes(M, N, K, 1) > 0
    got = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, reference_rounding=True)
    got32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, reference_rounding=True)
    unsplit = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, reference_rounding=True, split_k=False)
    torch.cuda.synchronize()
    assert torch.equal(got32, got.float())                       # a binary32 buffer receives the same bf16 values
    for y in (got, unsplit):
        differ = (y != want).float().mean().item()
        assert differ < 2e-3, f"{differ:.2e} of the outputs differ from the all-bf16 evaluation"
        assert rel_fro(y.float().cpu(), want.float().cpu()) <= 2e-4
    # and it is a different number from the exact-product result: the two modes are not interchangeable
    exact = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, reference_rounding=False, tiled=True)
    assert 5e-4 < rel_fro(exact.float().cpu(), want.float().cpu()) < 2e-2


@pytest.mark.parametrize("M,N,K,r,with_bias", [(64, 4736, 3584, 64, True), (17, 2052, 2048, 0, True), (1, 4608, 3584, 32, False),
                                               (40, 1536, 8960, 64, True), (64, 3584, 18944, 64, True), (200, 512, 1024, 32, True),
                                               (33, 260, 192, 96, False), (64, 3584, 18944, 0, True)])
def test_decode_shapes_with_reference_rounding_in_bf16_arithmetic(M, N, K, r, with_bias):
    """Below 256 rows the decode-sized kernel serves reference_rounding: it expands both packed operands to the
    reference's twice-rounded bf16 dequantized values in registers and rounds where the all-bf16 forward rounds (residual
    product, bias add, final sum), also when K is cut into slices that meet in a second kernel (the two 18944-long
    contractions).  Same check as for the pipelined kernel: that evaluation in double precision between the roundings."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(6000 + M + N)
    x = synthetic_activation(80 + M, M, K).cuda()
    w = _weights(81 + N, N, K).cuda()
    t = u = None
    if r:
        t = torch.randn(M, r, generator=g).bfloat16().cuda()
        u = (torch.randn(N, r, generator=g) * 0.05).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda() if with_bias else None
    px, pw = ops.quantize(x, 1), ops.quantize(w, 1)
    xq, wq = ops.dequantize(px, torch.bfloat16).double(), ops.dequantize(pw, torch.bfloat16).double()   # the reference's QDQ values
    want = (xq @ wq.T).bfloat16()
    if bias is not None:
        want = (want.float() + bias.float()).bfloat16()
    want = want.double()
    if r:
        want = want + t.double() @ u.double().T
    want = want.bfloat16()
    got = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, reference_rounding=True)
    got32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, reference_rounding=True)
    unsplit = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, reference_rounding=True, split_k=False)
    grouped = ops.linear_fwd_grouped(px, [(pw, t, u, bias), (pw, None, None, None)], reference_rounding=True)
    torch.cuda.synchronize()
    assert torch.equal(got32, got.float())                       # a binary32 buffer receives the same bf16 values
    assert (grouped[1] != (xq @ wq.T).bfloat16()).float().mean().item() < 2e-3     # a member without bias or low-rank term
    for y in (got, unsplit, grouped[0]):                         # (a group has more column tiles: K may be sliced differently)
        differ = (y != want).float().mean().item()
        assert differ < 2e-3, f"{differ:.2e} of the outputs differ from the all-bf16 evaluation"
        assert rel_fro(y.float().cpu(), want.float().cpu()) <= 2e-4
    # the exact-product result is a different number: the two modes are not interchangeable
    exact = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, reference_rounding=False)
    assert 5e-4 < rel_fro(exact.float().cpu(), want.float().cpu()) < 2e-2


@pytest.mark.parametrize("M,N,K,r", [(64, 4736, 3584, 64), (17, 2052, 2048, 0), (1, 4608, 3584, 32), (40, 1536, 8960, 64),
                                     (64, 18944, 3584, 64)])
def test_decode_shapes_with_lowrank_and_bias(M, N, K, r):
    """M <= 64 runs on the skinny kernel (waves split K, partial sums meet in LDS); every layout the shape
    heuristics can pick is covered: one or two row tiles per wave, row tiles in separate workgroups,
    four or eight waves."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(77)
    x = synthetic_activation(40 + M, M, K).cuda()
    w = _weights(41 + N, N, K).cuda()
    t = u = None
    if r:
        t = torch.randn(M, r, generator=g).bfloat16().cuda()
        u = torch.randn(N, r, generator=g).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda()
    px, pw = ops.quantize(x), ops.quantize(w)
    got = ops.linear_fwd(px, pw, t=t, u=u, bias=bias)
    got32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T
    if r:
        want = want + t.double() @ u.double().T
    want = want + bias.double()
    torch.cuda.synchronize()
    assert rel_fro(got32.cpu(), want.cpu()) <= 1e-5
    assert rel_fro(got.cpu(), want.cpu().bfloat16()) <= TOL


@pytest.mark.parametrize("M,N,K,r", [(256, 512, 4096, 64), (300, 260, 4096, 0), (512, 3584, 2048, 32), (1024, 1536, 4160, 64),
                                     (260, 776, 18944, 0)])
def test_split_k_shapes(M, N, K, r):
    """Few output tiles and a long contraction: up to 16 workgroups share a tile, partial tiles meet in a
    caller-supplied workspace.  Covers ragged M and N (N % 8 != 0 takes the plain stores), step counts that
    do not divide by the number of splits, the low-rank term and the bias (which must enter exactly once)."""
    from metis_hip import _lib, ops
    assert _lib.load().metis_linear_workspace_bytes(M, N, K) > 0
    g = torch.Generator().manual_seed(91)
    x = synthetic_activation(50 + M, M, K).cuda()
    w = _weights(51 + N, N, K).cuda()
    t = u = None
    if r:
        t = torch.randn(M, r, generator=g).bfloat16().cuda()
        u = torch.randn(N, r, generator=g).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda()
    px, pw = ops.quantize(x), ops.quantize(w)
    got = ops.linear_fwd(px, pw, t=t, u=u, bias=bias)
    got32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T
    if r:
        want = want + t.double() @ u.double().T
    want = want + bias.double()
    torch.cuda.synchronize()
    assert rel_fro(got32.cpu(), want.cpu()) <= 1e-5
    assert rel_fro(got.cpu(), want.cpu().bfloat16()) <= TOL
    # and against the unsplit kernel on the same operands
    whole32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, split_k=False)
    torch.cuda.synchronize()
    assert rel_fro(got32.cpu(), whole32.cpu()) <= 1e-5


@pytest.mark.parametrize("M,N,K,r", [(4096, 4352, 1024, 32), (4100, 4004, 2112, 0), (4096, 8960, 1536, 64)])
def test_split_k_of_the_last_partial_round(M, N, K, r):
    """A tile count a little over a multiple of the compute units (272 or 560 tiles on 256 units): the full rounds
    run unsplit and write the output directly, only the tiles of the last round are split through the workspace.
    Both kinds of tile are checked against the double-precision product and against the unsplit kernel."""
    from metis_hip import _lib, ops
    tiles = ((M + 255) // 256) * ((N + 255) // 256)
    need = _lib.load().metis_linear_workspace_bytes(M, N, K)
    assert 0 < need < tiles * 256 * 256 * 4                    # fewer partial tiles than two per output tile
    g = torch.Generator().manual_seed(95)
    x = synthetic_activation(52 + M, M, K).cuda()
    w = _weights(53 + N, N, K).cuda()
    t = u = None
    if r:
        t = torch.randn(M, r, generator=g).bfloat16().cuda()
        u = torch.randn(N, r, generator=g).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda()
    px, pw = ops.quantize(x), ops.quantize(w)
    got = ops.linear_fwd(px, pw, t=t, u=u, bias=bias)
    got32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T
    if r:
        want = want + t.double() @ u.double().T
    want = want + bias.double()
    torch.cuda.synchronize()
    assert rel_fro(got32.cpu(), want.cpu()) <= 1e-5
    assert rel_fro(got.cpu(), want.cpu().bfloat16()) <= TOL
    whole32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, split_k=False)
    whole = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, split_k=False)
    torch.cuda.synchronize()
    # the unsplit tiles are bit-identical to the unsplit kernel, the split ones differ in summation order only
    same = (got32 == whole32).float().mean().item()
    assert 0.5 < same < 1.0 or same == 1.0
    assert rel_fro(got32.cpu(), whole32.cpu()) <= 1e-5
    assert (got != whole).float().mean().item() < 0.01


def test_split_k_dgrad_wgrad_and_workspace_errors():
    from metis_hip import _lib, ops
    L, N, K = 512, 2048, 512
    lib = _lib.load()
    assert lib.metis_linear_workspace_bytes(L, K, N) > 0       # dgrad: L x K contracted over N
    g = torch.Generator().manual_seed(92)
    dy = (torch.randn(L, N, generator=g) * 1e-3).bfloat16().cuda()
    w = _weights(93, N, K).cuda()
    p_dy, p_wt = ops.quantize(dy, sr=True, seed=5), ops.quantize(w, col=True)
    gx = ops.linear_dgrad(p_dy, p_wt, out_dtype=torch.float32)
    want = ops.dequantize(p_dy, torch.float32).double() @ ops.dequantize(p_wt, torch.float32).double().T
    assert rel_fro(gx.cpu(), want.cpu()) <= 1e-5
    # wgrad: N x K contracted over L
    L2, N2, K2 = 4096, 256, 512
    assert lib.metis_linear_workspace_bytes(N2, K2, L2) > 0
    dy2 = (torch.randn(L2, N2, generator=g) * 1e-3).bfloat16().cuda()
    x2 = synthetic_activation(94, L2, K2).cuda()
    p_dyt, p_xt = ops.quantize(dy2, col=True, sr=True, seed=6), ops.quantize(x2, col=True, sr=True, seed=7)
    gw = ops.linear_wgrad(p_dyt, p_xt)
    want = ops.dequantize(p_dyt, torch.float32).double() @ ops.dequantize(p_xt, torch.float32).double().T
    assert gw.dtype == torch.float32 and rel_fro(gw.cpu(), want.cpu()) <= 1e-5
    # a workspace that is too small or misaligned is refused; none at all selects the unsplit kernel
    need = lib.metis_linear_workspace_bytes(L, K, N)
    ws = torch.empty(need + 16, dtype=torch.uint8, device="cuda")
    out = torch.empty(L, K, dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (p_dy.codes.data_ptr(), p_dy.scales.data_ptr(), p_dy.unit.data_ptr(), p_wt.codes.data_ptr(),
            p_wt.scales.data_ptr(), p_wt.unit.data_ptr(), L, N, K, out.data_ptr(), _lib.DTYPE_F32)
    assert lib.metis_linear_dgrad_ws(*args, ws.data_ptr(), need - 1, st) == _lib.E_WORKSPACE
    assert lib.metis_linear_dgrad_ws(*args, ws.data_ptr() + 4, need, st) == _lib.E_WORKSPACE
    assert lib.metis_linear_dgrad_ws(*args, None, 0, st) == 0
    torch.cuda.synchronize()
    assert rel_fro(out.cpu(), gx.cpu()) <= 1e-5


def test_output_offsets_beyond_32_bits():
    """2.2 G output elements: element offsets m * N + n pass 2^31.  Activation rows repeat with period 256,
    so output rows must repeat too; one period is checked against the double-precision product."""
    from metis_hip import ops
    M, N, K = 49152, 45056, 64
    base = synthetic_activation(81, 256, K).cuda()
    w = _weights(82, N, K).cuda()
    px, pw = ops.quantize(base.repeat(M // 256, 1)), ops.quantize(w)
    out = ops.linear_fwd(px, pw)
    assert out.numel() > 2 ** 31
    want = ops.dequantize(ops.quantize(base), torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T
    torch.cuda.synchronize()
    assert rel_fro(out[:256].cpu(), want.cpu().bfloat16()) <= TOL
    first = out[:256]
    for rep in (1, 95, 191):
        assert torch.equal(out[rep * 256:(rep + 1) * 256], first), rep


@pytest.mark.parametrize("M,K,Ns,r", [(64, 3584, (3584, 512, 512), 64), (1, 1024, (256, 96), 0), (40, 3584, (18944, 18944), 32),
                                      (64, 320, (100, 36, 64, 2052), 32), (300, 512, (384, 260), 32)])
def test_grouped_projections_equal_member_by_member_calls(M, K, Ns, r):
    """A projection group against one packed activation: bit-identical to calling linear_fwd per member (the
    decode-sized cases run as one launch, the last one falls back to a call per member)."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + K)
    px = ops.quantize(synthetic_activation(60 + M, M, K).cuda())
    members = []
    for i, N in enumerate(Ns):
        pw = ops.quantize(_weights(61 + i, N, K).cuda())
        t = u = None
        if r and i != 1:                                        # one member without a low-rank term
            t = torch.randn(M, r, generator=g).bfloat16().cuda()
            u = torch.randn(N, r, generator=g).bfloat16().cuda()
        bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda() if i % 2 == 0 else None
        members.append((pw, t, u, bias))
    for dt in (torch.bfloat16, torch.float32):
        got = ops.linear_fwd_grouped(px, members, out_dtype=dt)
        for (pw, t, u, bias), y in zip(members, got):
            want = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=dt)
            assert torch.equal(y, want)


@pytest.mark.parametrize("M,K,Ns,r", [(64, 3584, (3584, 512, 512), 64), (1, 1024, (256, 100), 0), (40, 3584, (18944, 18944), 32),
                                      (64, 18944, (3584,), 64), (200, 2048, (132, 64, 36), 32), (17, 256, (4,), 0)])
def test_cached_weights_in_the_decode_layout_give_the_same_bits(M, K, Ns, r):
    """A persistent (cached) weight is also kept in the decode layout -- rows in tiles of 32, K in steps of 256, the 16-byte
    pieces of a wave's lanes side by side -- and decode-sized calls stream that copy.  Same kernel, same order of
    operations: bit-identical outputs with and without it, in exact arithmetic, with the reference's bf16 roundings, with
    a centre inside the launch, with K split into slices, for ragged last tiles (N % 32 != 0); the layout itself is
    checked against its definition."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + K)
    x = synthetic_activation(160 + M, M, K).cuda()
    centre = (torch.randn(K, generator=g) * 0.2).cuda()
    for mode in (0, 1):
        px = ops.quantize(x, mode)
        plain, cached = [], []
        for i, N in enumerate(Ns):
            w = _weights(161 + i, N, K).cuda()
            t = u = None
            if r and i != 1:
                t = torch.randn(M, r, generator=g).bfloat16().cuda()
                u = (torch.randn(N, r, generator=g) * 0.1).bfloat16().cuda()
            bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda() if i % 2 == 0 else None
            pw, pc = ops.quantize(w, mode), ops.quantize(w, mode)
            pw.decode_layout = pc.decode_layout = None          # (a tensor of fewer than 256 rows leaves the quantizer with one)
            pc.persistent = True
            plain.append((pw, t, u, bias))
            cached.append((pc, t, u, bias))
        for kw in ({}, {"reference_rounding": True} if mode == 1 else {"center": centre}, {"split_k": False}):
            want = ops.linear_fwd_grouped(px, plain, **kw)
            got = ops.linear_fwd_grouped(px, cached, **kw)
            assert all(m[0].decode_layout is not None for m in cached) and all(m[0].decode_layout is None for m in plain)
            for a, b in zip(got, want):
                assert torch.equal(a, b), (mode, kw.keys())
    # the layout: block (tile, step) = 4 KiB of codes (piece j of lane l at j * 1024 + l * 16) + 512 scale bytes (lane l at 4096 + l * 8)
    pc = cached[0][0]
    N = Ns[0]
    lay = pc.decode_layout.cpu().reshape((N + 31) // 32, K // 256, 4608)
    codes, scales = pc.codes.cpu(), pc.scales.cpu()
    for tile, step, lane, j in ((0, 0, 0, 0), ((N - 1) // 32, K // 256 - 1, 37, 3), (0, K // 256 - 1, 63, 1)):
        row, h = tile * 32 + (lane & 31), lane >> 5
        got_c = lay[tile, step, j * 1024 + lane * 16: j * 1024 + lane * 16 + 16]
        got_s = lay[tile, step, 4096 + lane * 8: 4096 + lane * 8 + 8]
        if row < N:
            assert torch.equal(got_c, codes[row, step * 128 + h * 64 + 16 * j: step * 128 + h * 64 + 16 * j + 16])
            assert torch.equal(got_s, scales[row, step * 16 + h * 8: step * 16 + h * 8 + 8])
        else:
            assert int(got_c.sum()) == 0 and int(got_s.sum()) == 0


@pytest.mark.parametrize("M,K,Ns,r", [(64, 18944, (3584,), 64), (1, 8192, (256,), 0), (200, 16384, (132, 64), 32),
                                      (33, 8256, (96,), 32)])
def test_decode_sized_products_with_a_long_contraction_split_k(M, K, Ns, r):
    """Few output columns and a long K (a down projection at decode size): K is cut into slices that run as separate
    workgroups and a second kernel adds the binary32 partial sums.  Checked against the double-precision product of the
    dequantized operands, against the unsplit kernel (summation order only), and that the shape really is split."""
    from metis_hip import _lib, ops
    import ctypes
    g = torch.Generator().manual_seed(M + K)
    px = ops.quantize(synthetic_activation(70 + M, M, K).cuda())
    members = []
    for i, N in enumerate(Ns):
        pw = ops.quantize(_weights(71 + i, N, K).cuda())
        t = u = None
        if r:
            t = torch.randn(M, r, generator=g).bfloat16().cuda()
            u = (torch.randn(N, r, generator=g) * 0.1).bfloat16().cuda()
        bias = torch.randn(N, generator=g).cuda() if i == 0 else (torch.randn(N, generator=g) * 0.1).bfloat16().cuda()
        members.append((pw, t, u, bias))
    arr = (_lib.LinearMember * len(Ns))()
    for i, N in enumerate(Ns):
        arr[i].N = N
    assert _lib.load().metis_linear_grouped_workspace_bytes(M, K, ctypes.cast(arr, ctypes.c_void_p), len(Ns)) > 0
    da = ops.dequantize(px, torch.float32).double()
    for dt in (torch.float32, torch.bfloat16):
        got = ops.linear_fwd_grouped(px, members, out_dtype=dt)
        single = [ops.linear_fwd(px, pw, t=t, u=u, bias=b, out_dtype=dt) for pw, t, u, b in members]
        unsplit = ops.linear_fwd_grouped(px, members, out_dtype=dt, split_k=False)
        for (pw, t, u, b), y, y1, y0 in zip(members, got, single, unsplit):
            want = da @ ops.dequantize(pw, torch.float32).double().T + b.double()
            if t is not None:
                want = want + t.double() @ u.double().T
            tol = 5e-5 if dt == torch.float32 else TOL
            want = want.cpu().to(dt)                            # a bf16 result is compared after the same final rounding
            assert rel_fro(y.cpu(), want) <= tol
            assert rel_fro(y1.cpu(), want) <= tol
            assert rel_fro(y.float().cpu(), y0.float().cpu()) <= (1e-5 if dt == torch.float32 else TOL)


def test_config3_full_size_forward_on_row_and_column_slices():
    """8192 x 4096 x 14336 with r = 64 and bias: the full launch is checked on three row slabs and one column slab
    against the double-precision product of the dequantized operands (the slabs straddle tile and XCD boundaries),
    and on linearity in the low-rank term: out(t) - out(0) == t u^T."""
    from metis_hip import ops
    M, K, N, r = 8192, 4096, 14336, 64
    g = torch.Generator().manual_seed(1003)
    x = synthetic_activation(1003, M, K).cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    t = torch.randn(M, r, generator=g).bfloat16().cuda()
    u = (torch.randn(N, r, generator=g) * 0.1).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 0.1).bfloat16().cuda()
    px, pw = ops.quantize(x), ops.quantize(w)
    out = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32)
    xq, wq = ops.dequantize(px, torch.float32).double(), ops.dequantize(pw, torch.float32).double()
    for r0 in (0, 4000, M - 100):
        want = xq[r0:r0 + 100] @ wq.T + t[r0:r0 + 100].double() @ u.double().T + bias.double()
        assert rel_fro(out[r0:r0 + 100].cpu(), want.cpu()) <= 1e-5
    c0 = 7100
    want = xq @ wq[c0:c0 + 100].T + t.double() @ u[c0:c0 + 100].double().T + bias[c0:c0 + 100].double()
    assert rel_fro(out[:, c0:c0 + 100].cpu(), want.cpu()) <= 1e-5
    plain = ops.linear_fwd(px, pw, bias=bias, out_dtype=torch.float32)
    low = (out - plain)[::37].double()
    assert rel_fro(low.cpu(), (t[::37].double() @ u.double().T).cpu()) <= 1e-4
    got16 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias)
    assert rel_fro(got16[::53].float().cpu(), out[::53].bfloat16().float().cpu()) <= 1e-6     # the bf16 store is one rounding


def test_config4_full_size_dgrad_and_wgrad():
    """L = 4096 tokens, 1536 -> 8960 projection: dgrad (split-K: 96 output tiles) and wgrad (210 tiles) on operands
    re-quantized along their contraction, against double precision on row slabs."""
    from metis_hip import ops
    L, K, N = 4096, 1536, 8960
    g = torch.Generator().manual_seed(1004)
    x = synthetic_activation(1004, L, K).cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    dy = (torch.randn(L, N, generator=torch.Generator().manual_seed(2004)) * 1e-3).bfloat16().cuda()
    p_dy, p_wt = ops.quantize(dy, sr=True, seed=2004), ops.quantize(w, col=True)
    gx = ops.linear_dgrad(p_dy, p_wt, out_dtype=torch.float32)
    dq, wq = ops.dequantize(p_dy, torch.float32).double(), ops.dequantize(p_wt, torch.float32).double()      # [L, N], [K, N]
    for r0 in (0, 2000, L - 64):
        assert rel_fro(gx[r0:r0 + 64].cpu(), (dq[r0:r0 + 64] @ wq.T).cpu()) <= 1e-5
    p_dyt, p_xt = ops.quantize(dy, col=True, sr=True, seed=2005), ops.quantize(x, col=True, sr=True, seed=2006)
    gw = ops.linear_wgrad(p_dyt, p_xt)
    dtq, xtq = ops.dequantize(p_dyt, torch.float32).double(), ops.dequantize(p_xt, torch.float32).double()   # [N, L], [K, L]
    for r0 in (0, 5000, N - 64):
        assert rel_fro(gw[r0:r0 + 64].cpu(), (dtq[r0:r0 + 64] @ xtq.T).cpu()) <= 1e-5
    # stochastic rounding keeps the gradients unbiased estimates of the dense ones: FP4 noise level, not a parity bar
    assert rel_fro(gx.cpu(), (dy.double() @ w.double()).cpu()) < 0.2
    assert rel_fro(gw.cpu(), (dy.double().T @ x.double()).cpu()) < 0.3


@pytest.mark.parametrize("M,K,R", [(64, 3584, 64), (64, 18944, 64), (1, 64, 32), (100, 1536, 96), (255, 8960, 192), (33, 3584, 256)])
def test_lowrank_projection_for_decode_sized_batches(M, K, R):
    """x V^T (and its bf16 product with s) on the split-K kernel: one correct bf16 rounding of the double-precision sum;
    t is the bf16 product of the stored bf16 projection and s, as torch.mul on bf16 tensors."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + K + R)
    x = synthetic_activation(70 + M, M, K).cuda()
    v = (torch.randn(R, K, generator=g) / K ** 0.5).bfloat16().cuda()
    s = (torch.rand(R, generator=g) * 4 + 0.1).bfloat16().cuda()
    xv, t = ops.lowrank_project(x, v, s)
    want = x.double() @ v.double().T
    torch.cuda.synchronize()
    assert xv.dtype == torch.bfloat16 and xv.shape == (M, R)
    d = (xv.double() - want).abs()
    assert bool((d <= want.abs() * 2.0 ** -8 + 1e-6 * float(want.abs().max())).all())
    assert torch.equal(t, xv * s)
    assert torch.equal(ops.lowrank_project(x, v), xv)
    wide = torch.zeros(M, K + 64, dtype=torch.bfloat16, device="cuda")
    wide[:, :K] = x
    assert torch.equal(ops.lowrank_project(wide[:, :K], v), xv)
    # ranks that neither kernel takes fall back to the vendor library with the same signature
    big = torch.randn(300, 128, generator=g).bfloat16().cuda()
    vb = torch.randn(16, 128, generator=g).bfloat16().cuda()
    a, b = ops.lowrank_project(big, vb, s[:16])
    assert torch.equal(a, big @ vb.T) and torch.equal(b, a * s[:16])


def test_grouped_members_read_column_slices_of_a_stacked_projection():
    """t operands that are column slices of one [M, sum r] tensor (row stride sum r) are read in place."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(88)
    M, K, Ns, rs = 64, 1024, (512, 96, 256), (64, 32, 32)
    px = ops.quantize(synthetic_activation(89, M, K).cuda())
    stacked = torch.randn(M, sum(rs), generator=g).bfloat16().cuda()
    members, c0 = [], 0
    for i, (N, r) in enumerate(zip(Ns, rs)):
        pw = ops.quantize(_weights(90 + i, N, K).cuda())
        u = torch.randn(N, r, generator=g).bfloat16().cuda()
        members.append((pw, stacked[:, c0:c0 + r], u, None))
        c0 += r
    assert not members[1][1].is_contiguous()
    got = ops.linear_fwd_grouped(px, members, out_dtype=torch.float32)
    for (pw, t, u, _), y in zip(members, got):
        assert torch.equal(y, ops.linear_fwd(px, pw, t=t.contiguous(), u=u, out_dtype=torch.float32))


@pytest.mark.parametrize("M,R,K", [(300, 32, 512), (4096, 64, 4096), (1000, 128, 1536), (8192, 64, 3584), (1024, 64, 18944),
                                   (2048, 32, 4096), (260, 128, 2112)])
def test_rank_r_projection_at_training_sizes(M, R, K):
    """xv = x V^T and t = bf16(xv * s) for 256 rows and more (one pass over x, MFMA): binary32 accumulation rounded once to
    bf16, against double precision rounded the same way (only results on a rounding boundary can differ), and t exactly
    the bf16 product of the kernel's own xv with s.  Few rows against a long contraction run as K slices whose partial
    sums a second launch adds (the last three shapes: 16, 4 and 2 slices on a 256-CU device)."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(6000 + M)
    x = synthetic_activation(80 + M, M, K).cuda()
    v = (torch.randn(R, K, generator=g) / K ** 0.5).bfloat16().cuda()
    s = (torch.rand(R, generator=g) * 4 + 0.1).bfloat16().cuda()
    xv, t = ops.lowrank_project(x, v, s)
    want = (x.double() @ v.double().T)
    torch.cuda.synchronize()
    assert xv.shape == (M, R) and xv.dtype == torch.bfloat16
    assert rel_fro(xv.float().cpu(), want.bfloat16().float().cpu()) <= 5e-4
    assert rel_fro(xv.float().cpu(), want.cpu()) <= 3e-3          # one bf16 rounding of the exact product
    assert torch.equal(t, (xv.float() * s.float()).bfloat16())
    only = ops.lowrank_project(x, v)
    assert torch.equal(only, xv)
    # a strided view (columns of a wider tensor) is read in place
    wide = torch.cat((x, x), dim=1)
    assert torch.equal(ops.lowrank_project(wide[:, :K], v), xv)


@pytest.mark.parametrize("L,C,R", [(1000, 520, 32), (4096, 1536, 64), (4096, 8960, 32), (2048, 14336, 64), (777, 256, 128)])
def test_rank_r_products_that_contract_over_tokens(L, C, R):
    """out[C, R] = sum_l a[l, C] b[l, R] (gradients of U and, transposed, of V): token slices added in a fixed order,
    against double precision; ragged token counts and column counts that are not multiples of the tile."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(7000 + L)
    a = (torch.randn(L, C, generator=g) * 1e-2).bfloat16().cuda()
    b = torch.randn(L, R, generator=g).bfloat16().cuda()
    want = a.double().T @ b.double()
    got = ops.lowrank_contract_tokens(a, b, out_dtype=torch.float32)
    got_t = ops.lowrank_contract_tokens(a, b, out_dtype=torch.bfloat16, transpose=True)
    again = ops.lowrank_contract_tokens(a, b, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert got.shape == (C, R) and got_t.shape == (R, C)
    assert rel_fro(got.cpu(), want.cpu()) <= 1e-5
    assert torch.equal(got, again)                              # fixed summation order
    assert torch.equal(got_t, got.bfloat16().T)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("M,R,K", [(256, 32, 64), (300, 64, 192), (1024, 64, 4096), (4100, 32, 1536), (8192, 64, 4096)])
def test_quantizer_and_rank_r_projection_in_one_pass(M, R, K, mode):
    """metis_nvfp4_quant_project_deferred: the packed activation has the bytes of the quantizer (codes, parked block maxima,
    and the scale bytes and unit formed from them), the projection is that of the projection call; ragged rows, a short
    last step of K, K slices (1024 rows), both ranks the kernel takes, both arithmetics."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(9000 + M + mode)
    x = synthetic_activation(90 + M, M, K).cuda()
    v = (torch.randn(R, K, generator=g) / K ** 0.5).bfloat16().cuda()
    s = (torch.rand(R, generator=g) * 4 + 0.1).bfloat16().cuda()
    assert ops.quantize_project_applies(x, v, mode)
    p, xv, t = ops.quantize_project(x, v, s, mode)
    want = ops.quantize(x, mode)
    lazy = ops.quantize(x, mode, deferred=True)
    xv0, t0 = ops.lowrank_project(x, v, s)
    torch.cuda.synchronize()
    nb = M * K // 16
    assert torch.equal(p.codes, want.codes)
    assert torch.equal(p.deferred[8192:8192 + 2 * nb], lazy.deferred[8192:8192 + 2 * nb])       # parked bf16 block maxima
    assert torch.equal(p.scales, want.scales) and torch.equal(p.unit, want.unit)
    assert torch.equal(xv, xv0) and torch.equal(t, t0)
    assert rel_fro(xv.float().cpu(), (x.double() @ v.double().T).cpu()) <= 3e-3
    # the consumer of the parked data: the tiled expansion forms the same operand from either packing
    if K % 32 == 0:
        fresh = ops.quantize_project(x, v, s, mode)[0]
        assert torch.equal(ops.expand_tiled(fresh, cache=False, mode=mode), ops.expand_tiled(want, cache=False, mode=mode))


def test_quantizer_and_projection_argument_checks():
    from metis_hip import _lib, ops
    L = _lib.load()
    x = torch.zeros(256, 64, dtype=torch.bfloat16, device="cuda")
    v = torch.zeros(32, 64, dtype=torch.bfloat16, device="cuda")
    s = torch.zeros(32, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(256, 32, dtype=torch.bfloat16, device="cuda")
    codes = torch.zeros(256, 32, dtype=torch.uint8, device="cuda")
    parked = torch.zeros(L.metis_nvfp4_deferred_bytes(256, 64), dtype=torch.uint8, device="cuda")

    def call(rows=256, cols=64, mode=0, R=32, parked_bytes=None, xp=None):
        return L.metis_nvfp4_quant_project_deferred(x.data_ptr() if xp is None else xp, rows, cols, mode, v.data_ptr(), R, s.data_ptr(),
                                                    out.data_ptr(), out.data_ptr(), codes.data_ptr(), parked.data_ptr(),
                                                    parked.numel() if parked_bytes is None else parked_bytes, None, 0, None)

    assert call() == 0
    assert call(rows=0) == 0
    assert call(mode=2) == _lib.E_ARG                               # binary32 input has no fused form
    assert call(R=48) == _lib.E_SHAPE and call(cols=48) == _lib.E_SHAPE and call(R=128) == _lib.E_SHAPE
    assert call(rows=70000) == _lib.E_TOO_LARGE                     # more row tiles than partial maxima: call the two functions
    assert call(parked_bytes=1024) == _lib.E_WORKSPACE
    assert call(xp=x.data_ptr() + 2) == _lib.E_ARG
    assert not ops.quantize_project_applies(x[:, :32], v[:, :32], 0)       # a strided view
    assert not ops.quantize_project_applies(x[:128], v, 0)                 # decode-sized batches have their own kernels
    torch.cuda.synchronize()


@pytest.mark.parametrize("L,R", [(4096, 32), (1000, 64), (16384, 128), (1, 8), (255, 40)])
def test_gradient_of_the_rank_r_scale_vector(L, R):
    """g_s = sum over tokens of the bf16 products g * xv (what autograd computes for torch.mul(s, y) on bf16 tensors) in one
    launch: the products rounded to bf16 exactly as torch rounds them, summed in binary32 in a fixed order."""
    from metis_hip import ops
    g_ = torch.Generator().manual_seed(8000 + L)
    g = torch.randn(L, R, generator=g_).bfloat16().cuda()
    xv = (torch.randn(L, R, generator=g_) * 3).bfloat16().cuda()
    got = ops.lowrank_scale_grad(g, xv)
    again = ops.lowrank_scale_grad(g, xv)
    want = (g * xv).double().sum(dim=0)                          # torch's bf16 products, summed exactly
    torch.cuda.synchronize()
    assert got.shape == (R,) and got.dtype == torch.float32
    assert torch.equal(got, again)
    scale = (g * xv).double().abs().sum(dim=0).clamp_min(1e-30)
    assert float(((got.double() - want).abs() / scale).max()) <= 1e-6
    # a view that the kernel does not take (strided) falls back to torch's own ops
    wide = torch.cat((g, g), dim=1)
    torch.testing.assert_close(ops.lowrank_scale_grad(wide[:, :R], xv), got, rtol=1e-4, atol=1e-4)
    assert torch.equal(ops.lowrank_scale_grad(g[:0], xv[:0]), torch.zeros(R, device="cuda"))
    assert torch.equal(ops.lowrank_scale_grad(g, xv, out_dtype=torch.bfloat16), got.bfloat16())

def test_memory_bound_deployments_can_drop_the_derived_weight_copies(monkeypatch):
    """A cached weight holds 0.5625 B per parameter packed; the tiled binary16 expansion (2 B, one per arithmetic) and
    the decode layout (0.5625 B) are built on first use.  With both switches off nothing but the packed form stays,
    and the outputs keep their bits: prefill on the packed operands (binary32 arithmetic) or on an expansion made per
    call (bf16 arithmetic), decode on the row-major packing."""
    from metis_hip import ops
    N, K = 512, 1024
    w = _weights(171, N, K).cuda()
    for mode in (0, 1):
        kw = {"reference_rounding": True, "split_k": False} if mode == 1 else {"split_k": False}   # one order of additions
        outs = {}
        for keep in (True, False):
            monkeypatch.setattr(ops, "tiled_weight_copies", keep)
            monkeypatch.setattr(ops, "decode_layout_weights", keep)
            pw = ops.quantize(w, mode)
            pw.persistent = True
            ys = []
            for M in (512, 48):
                px = ops.quantize(synthetic_activation(172 + M, M, K).cuda(), mode)
                ys.append(ops.linear_fwd_grouped(px, [(pw, None, None, None)], **kw)[0])
                ys.append(ops.linear_fwd(px, pw, **kw))
            held = pw.held_bytes()
            packed = N * K // 2 + N * K // 16
            assert held["packed"] == packed
            if keep:
                assert held["tiled_pb16" if mode == 1 else "tiled"] >= 2 * N * K and held["decode_layout"] >= packed
                assert sum(held.values()) >= 3.1 * N * K
            else:
                assert set(held) == {"packed"}
            outs[keep] = ys
        for a, b in zip(outs[True], outs[False]):
            assert torch.equal(a, b), mode


@pytest.mark.parametrize("M,K,Ns,r", [(64, 3584, (3584, 512, 512), 64), (1, 1024, (256, 100), 0), (40, 3584, (18944,), 32),
                                      (64, 18944, (3584,), 64), (200, 2048, (132, 64), 32), (17, 256, (4,), 0)])
def test_decode_sized_activations_leave_the_quantizer_in_the_decode_layout(M, K, Ns, r, monkeypatch):
    """The quantizer's second launch writes a decode-sized activation (fewer than 256 rows, K % 256 == 0) once more in
    the layout the decode-sized kernel streams as whole lines, and the grouped GEMM reads that instead of the row-major
    packing: the same kernel in the same order, so the same bits -- exact products, the reference's bf16 roundings, a
    centre inside the launch, K in slices, ragged M and N -- and the same codes, scale bytes and unit as the plain
    quantizer.  The fused RMSNorm -> NVFP4 call does the same."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M * 3 + K)
    x = synthetic_activation(260 + M, M, K).cuda()
    gamma = (1 + 0.1 * torch.randn(K, generator=g)).bfloat16().cuda()
    centre = (torch.randn(K, generator=g) * 0.2).cuda()
    for mode in (0, 1):
        members = []
        for i, N in enumerate(Ns):
            pw = ops.quantize(_weights(261 + i, N, K).cuda(), mode)
            pw.persistent = i % 2 == 0                          # with and without the weight's own decode layout
            t = u = None
            if r:
                t = torch.randn(M, r, generator=g).bfloat16().cuda()
                u = (torch.randn(N, r, generator=g) * 0.1).bfloat16().cuda()
            members.append((pw, t, u, (torch.randn(N, generator=g) * 0.1).bfloat16().cuda() if i == 0 else None))
        packs = {}
        for on in (False, True):
            monkeypatch.setattr(ops, "decode_layout_activations", on)
            packs[on] = (ops.quantize(x, mode), ops.rmsnorm_quantize(x, gamma, 1e-6, mode) if K <= 16384 else None)   # the norm holds a row in registers
        plain, dec = packs[False][0], packs[True][0]
        assert plain.decode_layout is None and dec.decode_layout is not None
        pairs = [(plain, dec)]
        if K <= 16384:
            (normed_plain, fused_plain), (normed_dec, fused_dec) = packs[False][1], packs[True][1]
            assert torch.equal(normed_plain, normed_dec) and fused_plain.decode_layout is None
            pairs.append((fused_plain, fused_dec))
        for a, b in pairs:
            assert torch.equal(a.codes, b.codes) and torch.equal(a.scales, b.scales) and torch.equal(a.unit, b.unit)
            # the layout against its definition (the weight's re-tiling kernel applied to the packed activation)
            assert torch.equal(b.decode_layout, ops.decode_weight(a, cache=False))
        for kw in ({}, {"reference_rounding": True} if mode == 1 else {"center": centre}, {"split_k": False}):
            want = ops.linear_fwd_grouped(plain, members, **kw)
            got = ops.linear_fwd_grouped(dec, members, **kw)
            for a, b in zip(got, want):
                assert torch.equal(a, b), (mode, kw.keys())


@pytest.mark.parametrize("mode", [0, 1])
def test_large_backward_products_take_the_pipelined_kernel_with_the_same_bits(mode):
    """From about 2e11 flop on, linear_dgrad and linear_wgrad expand their operands for the one call and run on the
    pipelined kernel (ops._tiled_backward_pays); the products are the packed kernels', bit for bit."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(4242 + mode)
    N, K, L = 4096, 4352, 8192
    assert ops._tiled_backward_pays(L, K, N, 0) and ops._tiled_backward_pays(N, K, L, 0)
    assert not ops._tiled_backward_pays(4096, 1536, 8960, 0)               # the config-4 projection stays packed
    dy = (torch.randn(L, N, generator=g) * 1e-3).bfloat16().cuda()
    x = torch.randn(L, K, generator=g).bfloat16().cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    p_dy, p_dyt, p_xt = ops.quantize(dy, mode), ops.quantize(dy, mode, col=True), ops.quantize(x, mode, col=True)
    p_wt = ops.quantize(w, mode, col=True)
    p_wt.persistent = True
    gx, gw = ops.linear_dgrad(p_dy, p_wt), ops.linear_wgrad(p_dyt, p_xt)
    ops.tiled_weight_copies = False
    try:
        gx_p, gw_p = ops.linear_dgrad(p_dy, p_wt), ops.linear_wgrad(p_dyt, p_xt)
    finally:
        ops.tiled_weight_copies = True
    torch.cuda.synchronize()
    assert torch.equal(gx, gx_p) and torch.equal(gw, gw_p)
    ref = dy.double() @ w.double()
    assert rel_fro(gx.double().cpu(), ref.cpu()) <= 0.2                     # FP4 operands: a coarse sanity bound on the product itself


def test_large_products_with_rank_r_operands_and_binary32_bias_on_either_kernel():
    """The size criterion also sends gradient products that carry a low-rank term (t, u) and the mean mode's binary32
    bias to the pipelined kernel.  Same products as the packed kernel; the low-rank term joins the binary32 sum at
    another point, so the results agree to binary32 rounding of the sums rather than bit for bit."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(77)
    M, N, K, r = 4096, 4352, 8192, 32
    a = ops.quantize(torch.randn(M, K, generator=g).bfloat16().cuda())
    b = ops.quantize((torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda())
    t = torch.randn(M, r, generator=g).bfloat16().cuda()
    u = torch.randn(N, r, generator=g).bfloat16().cuda()
    bias = torch.randn(N, generator=g).cuda()
    assert ops._tiled_backward_pays(M, N, K, 0)
    for out_dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 2e-4)):
        auto = ops.linear_fwd(a, b, t=t, u=u, bias=bias, out_dtype=out_dtype)
        packed = ops.linear_fwd(a, b, t=t, u=u, bias=bias, out_dtype=out_dtype, tiled=False)
        forced = ops.linear_fwd(a, b, t=t, u=u, bias=bias, out_dtype=out_dtype, tiled=True)
        torch.cuda.synchronize()
        assert torch.equal(auto, forced), out_dtype                   # the criterion picked the pipelined kernel
        err = (auto.float() - packed.float()).norm() / packed.float().norm()
        assert err <= tol, (out_dtype, float(err))


@pytest.mark.parametrize("M,K,R", [(64, 3584, 192), (1, 256, 32), (200, 2048, 64), (255, 18944, 64), (33, 512, 256)])
@pytest.mark.parametrize("mode,centred", [(1, False), (1, True), (0, False)])
def test_projection_finish_and_operand_build_in_one_launch(M, K, R, mode, centred):
    """metis_decode_prepare_deferred against metis_lowrank_project + metis_nvfp4_decode_operand_deferred on the same
    activation: the same xv, t, operand bytes and tensor unit, bit for bit; and its argument checks."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + K + R)
    x = (torch.randn(M, K, generator=g) * 3).bfloat16().cuda()
    v = (torch.randn(R, K, generator=g) * 0.05).bfloat16().cuda()
    s = torch.rand(R, generator=g).bfloat16().cuda()
    centre = (torch.randn(K, generator=g) * 0.1).bfloat16().cuda() if centred else None
    want_xv, want_t = ops.lowrank_project(x, v, s)
    p1 = ops.quantize(x, mode, deferred=True)
    want_op = ops.decode_operand(p1, mode, centre)
    p2 = ops.quantize(x, mode, deferred=True)
    assert ops.project_and_operand_applies(x, v, s, p2)
    xv, t, op = ops.project_and_operand(x, v, s, p2, mode, centre)
    torch.cuda.synchronize()
    assert torch.equal(xv, want_xv) and torch.equal(t, want_t)
    assert torch.equal(op, want_op)
    assert torch.equal(p2.unit, p1.unit)
    # once its scale bytes exist the tensor no longer qualifies (the operand call for written bytes is another one)
    p1.scales
    assert not ops.project_and_operand_applies(x, v, s, p1)
    with pytest.raises(ValueError):
        ops.project_and_operand(x, v, s, p1, mode, centre)


def test_decode_prepare_rejects_what_its_two_halves_reject():
    from metis_hip import _lib, ops
    L = _lib.load()
    M, K, R = 64, 512, 64
    x = torch.randn(M, K).bfloat16().cuda()
    v = torch.randn(R, K).bfloat16().cuda()
    s = torch.rand(R).bfloat16().cuda()
    p = ops.quantize(x, 1, deferred=True)
    xv = torch.empty(M, R, dtype=torch.bfloat16, device="cuda")
    t = torch.empty_like(xv)
    out = torch.empty(L.metis_nvfp4_decode_operand_bytes(M, K), dtype=torch.uint8, device="cuda")
    need = L.metis_lowrank_project_workspace_bytes(M, R, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    unit = torch.zeros(1, device="cuda")

    def call(rows=M, cols=K, r=R, wsb=need, mode=1, centre=None, xp=x.data_ptr(), up=unit.data_ptr(), rotate=0):
        return L.metis_decode_prepare_deferred(xp, cols, v.data_ptr(), r, s.data_ptr(), xv.data_ptr(), t.data_ptr(), ws.data_ptr(), wsb,
                                               p.codes.data_ptr(), p.deferred.data_ptr(), rows, cols, 1, mode, centre, up, out.data_ptr(),
                                               rotate, 0x5a3c, None)
    assert call() == 0
    assert call(rows=256) != 0 and call(rows=0) != 0          # decode-sized only
    assert call(cols=320) != 0                                # wide runs: K % 256 == 0
    assert call(r=48) != 0                                    # rank a multiple of 32
    assert call(wsb=need - 1) != 0                            # workspace too small
    assert call(mode=7) != 0
    assert call(mode=0, centre=x.data_ptr()) != 0             # a centre belongs to bf16 arithmetic
    assert call(up=None) != 0
    assert call(xp=None) == 0                                 # x = NULL: the partial sums are taken from the workspace
    assert call(xp=None, r=160) != 0                          # ... which the quantizer's launch fills for R <= 128 only
    assert call(rotate=1) == 0                                # the operand rotated for a weight packed in the rotated domain
    centre16 = torch.zeros(K, dtype=torch.bfloat16, device="cuda")
    assert call(rotate=1, centre=centre16.data_ptr()) != 0    # ... which takes no centre
    torch.cuda.synchronize()


@pytest.mark.parametrize("M,K,R", [(64, 3584, 64), (1, 256, 32), (200, 2048, 128), (255, 18944, 64), (33, 512, 96)])
@pytest.mark.parametrize("mode", [1, 0])
def test_quantizer_launch_carries_the_projections_first_step(M, K, R, mode):
    """metis_decode_quant_project_deferred + metis_decode_prepare_deferred(x = NULL) against the separate quantizer,
    projection and operand calls: codes, parked maxima, unit, xv, t and operand bytes, bit for bit."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(3 * M + K + R)
    x = (torch.randn(M, K, generator=g) * 2).bfloat16().cuda()
    v = (torch.randn(R, K, generator=g) * 0.05).bfloat16().cuda()
    s = torch.rand(R, generator=g).bfloat16().cuda()
    want_xv, want_t = ops.lowrank_project(x, v, s)
    p1 = ops.quantize(x, mode, deferred=True)
    assert ops.quantize_project_decode_applies(x, v, mode)
    p2, pending = ops.quantize_project_decode(x, v, mode)
    nb = M * K // 16
    assert torch.equal(p2.codes, p1.codes)
    assert torch.equal(p2.deferred[:8192 + 2 * nb], p1.deferred[:8192 + 2 * nb])     # partial maxima, parked block maxima
    xv, t, op = ops.project_and_operand(x, v, s, p2, mode, None, pending=pending)
    want_op = ops.decode_operand(p1, mode)
    torch.cuda.synchronize()
    assert torch.equal(xv, want_xv) and torch.equal(t, want_t)
    assert torch.equal(op, want_op) and torch.equal(p2.unit, p1.unit)


def test_decode_quant_project_rejects_shapes_outside_its_domain():
    from metis_hip import _lib
    L = _lib.load()
    M, K, R = 64, 512, 64
    x = torch.randn(M, K).bfloat16().cuda()
    v = torch.randn(R, K).bfloat16().cuda()
    codes = torch.empty(M, K // 2, dtype=torch.uint8, device="cuda")
    parked = torch.empty(L.metis_nvfp4_deferred_bytes(M, K), dtype=torch.uint8, device="cuda")
    need = L.metis_lowrank_project_workspace_bytes(M, R, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")

    def call(rows=M, cols=K, r=R, mode=1, wsb=need, pb=parked.numel(), xp=x.data_ptr()):
        return L.metis_decode_quant_project_deferred(xp, rows, cols, mode, codes.data_ptr(), parked.data_ptr(), pb, v.data_ptr(), r,
                                                     ws.data_ptr(), wsb, None)
    assert call() == 0
    assert call(rows=256) != 0 and call(rows=0) != 0
    assert call(cols=48) != 0
    assert call(r=160) != 0 and call(r=40) != 0
    assert call(mode=2) != 0
    assert call(wsb=need - 1) != 0 and call(pb=16) != 0
    assert call(xp=None) != 0
    torch.cuda.synchronize()
