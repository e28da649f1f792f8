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
