"""The allocation-free row quantizer (metis_nvfp4_quant_row_static: the workspace is a static device array inside the
library) against metis_nvfp4_quant_row with a caller workspace, through the C ABI: same codes, scale bytes and unit,
bit for bit, on two calls in a row of which the second is smaller (the shared array keeps the first call's contents)."""
import pytest
import torch

from helpers import synthetic_activation

pytestmark = pytest.mark.gpu


def _both(L, x, mode):
    rows, cols = x.shape
    dev = x.device
    st = torch.cuda.current_stream().cuda_stream
    out = []
    for static in (False, True):
        codes = torch.full((rows, cols // 2), 0xA5, dtype=torch.uint8, device=dev)
        scales = torch.full((rows, cols // 16), 0xA5, dtype=torch.uint8, device=dev)
        unit = torch.full((1,), -1.0, dtype=torch.float32, device=dev)
        if static:
            rc = L.metis_nvfp4_quant_row_static(x.data_ptr(), rows, cols, x.stride(0), mode, codes.data_ptr(), scales.data_ptr(),
                                                unit.data_ptr(), st)
        else:
            ws = torch.zeros(L.metis_nvfp4_workspace_bytes(rows, cols), dtype=torch.uint8, device=dev)
            rc = L.metis_nvfp4_quant_row(x.data_ptr(), rows, cols, x.stride(0), mode, codes.data_ptr(), scales.data_ptr(),
                                         unit.data_ptr(), ws.data_ptr(), ws.numel(), st)
        assert rc == 0
        torch.cuda.synchronize()
        out.append((codes.cpu(), scales.cpu(), unit.cpu()))
    return out


@pytest.mark.parametrize("mode", [0, 1])
def test_static_scratch_quantizer_matches_workspace_quantizer(mode):
    from metis_hip import _lib
    L = _lib.load()
    # a large call first, then a smaller one whose maxima are smaller too: stale words of the first call must not leak
    big = synthetic_activation(901, 4096, 4096).cuda()
    small = (synthetic_activation(902, 272, 1008) * 0.01).bfloat16().cuda()
    for x in (big, small):
        (c0, s0, u0), (c1, s1, u1) = _both(L, x, mode)
        assert torch.equal(c0, c1), f"codes differ: {(c0 != c1).sum().item()} bytes"
        assert torch.equal(s0, s1), f"scale bytes differ: {(s0 != s1).sum().item()}"
        assert u0.view(torch.int32).item() == u1.view(torch.int32).item()
    # binary32 input goes through the same array (parked maxima are binary32 then)
    xf = (torch.randn(512, 768, generator=torch.Generator().manual_seed(903)) * 3).cuda()
    (c0, s0, u0), (c1, s1, u1) = _both(L, xf, 2)
    assert torch.equal(c0, c1) and torch.equal(s0, s1) and u0.view(torch.int32).item() == u1.view(torch.int32).item()


def test_static_scratch_quantizer_rejects_what_does_not_fit():
    from metis_hip import _lib
    L = _lib.load()
    x = torch.zeros(16, 16, dtype=torch.bfloat16, device="cuda")
    buf = torch.zeros(64, dtype=torch.uint8, device="cuda")
    unit = torch.full((1,), -1.0, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    # 2^26 + 16 elements: refused before anything is read or launched
    rc = L.metis_nvfp4_quant_row_static(x.data_ptr(), (1 << 22) + 1, 16, 16, 0, buf.data_ptr(), buf.data_ptr(), unit.data_ptr(), st)
    assert rc == _lib.E_TOO_LARGE
    assert b"static scratch" in L.metis_error_string(rc)
    assert L.metis_nvfp4_quant_row_static(x.data_ptr(), 16, 24, 24, 0, buf.data_ptr(), buf.data_ptr(), unit.data_ptr(), st) == _lib.E_SHAPE
    torch.cuda.synchronize()
    assert float(unit.cpu()) == -1.0


def test_static_scratch_quantizer_allocates_nothing_and_replays_from_a_graph():
    """What the entry point exists for.  After its first call on the device (which looks the array's address up once)
    further calls of several sizes leave the device's free memory where it was; and, warmed up like that, the call can
    be captured into a HIP graph (two kernel nodes, no memset node) and replayed on changed input with the bytes of
    metis_nvfp4_quant_row each time, eager work and synchronisations between the replays."""
    from metis_hip import _lib
    L = _lib.load()
    dev = torch.device("cuda")
    rows, cols = 1024, 2048
    x = synthetic_activation(911, rows, cols).cuda()
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(rows, cols // 16, dtype=torch.uint8, device=dev)
    unit = torch.empty(1, dtype=torch.float32, device=dev)
    ws = torch.zeros(L.metis_nvfp4_workspace_bytes(rows, cols), dtype=torch.uint8, device=dev)
    ref = [torch.empty_like(codes), torch.empty_like(scales), torch.empty_like(unit)]

    def static_call(t, r, c, stream):
        return L.metis_nvfp4_quant_row_static(t.data_ptr(), r, c, c, 0, codes.data_ptr(), scales.data_ptr(), unit.data_ptr(), stream)

    st = torch.cuda.current_stream().cuda_stream
    assert static_call(x, rows, cols, st) == 0                   # warm-up: the first call on a device looks the address up
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for r, c in ((rows, cols), (64, 256), (512, 1024), (rows, cols)):
        assert static_call(x, r, c, st) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    # capture
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert static_call(x, rows, cols, torch.cuda.current_stream().cuda_stream) == 0
    for k in range(3):
        x.copy_(synthetic_activation(920 + k, rows, cols))        # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rc = L.metis_nvfp4_quant_row(x.data_ptr(), rows, cols, cols, 0, ref[0].data_ptr(), ref[1].data_ptr(), ref[2].data_ptr(),
                                     ws.data_ptr(), ws.numel(), st)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(codes, ref[0]) and torch.equal(scales, ref[1]) and torch.equal(unit, ref[2]), k
