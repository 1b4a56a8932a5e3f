"""trakhip_project_static (the entry point that allocates nothing) against trakhip_project, through
the C ABI: same bits on two calls in a row, the second with a smaller input, so that whatever the
first call left in the shared static array would show if the second call relied on it."""
import ctypes

import pytest
import torch

from trak_amd import _lib

pytestmark = pytest.mark.gpu

_DT = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


def _project(lib, x, k, seed, tiles, pt, static):
    B, P = x.shape
    out = torch.full((B, k), float("nan"), dtype=torch.float32, device=x.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    if static:
        code = lib.trakhip_project_static(ctypes.c_void_p(x.data_ptr()), _DT[x.dtype], B, P, x.stride(0),
                                          ctypes.c_void_p(out.data_ptr()), k, seed, tiles, pt, stream)
    else:
        nbytes = lib.trakhip_project_workspace(B, P, k, tiles)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        code = lib.trakhip_project(ctypes.c_void_p(x.data_ptr()), _DT[x.dtype], B, P, x.stride(0),
                                   ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(ws.data_ptr()), nbytes, k, seed,
                                   tiles, pt, stream)
    assert code == 0, _lib.strerror(code)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("pt", [_lib.RADEMACHER, _lib.NORMAL])
def test_static_entry_point_equals_workspace_entry_point_twice(gpu, pt):
    lib = _lib.load()
    gen = torch.Generator(device="cpu").manual_seed(5)
    # first call: 40 rows (two passes of 32 + 8 through the array - a 40-row pass would need 40 MiB -, against
    # one 40-row pass with the workspace), ragged P; second: smaller in every way; third: 70 rows whose 64-row
    # pass fits into the array (64 + 6, the same passes as with the workspace)
    shapes = [(40, 300_001, 1024, torch.float16), (7, 20_011, 512, torch.float32), (70, 50_001, 512, torch.bfloat16)]
    for B, P, k, dt in shapes:
        x = (torch.randn(B, P, generator=gen) * 1e-2).to(dt).to(gpu)
        want = _project(lib, x, k, 11, 256, pt, static=False)
        got = _project(lib, x, k, 11, 256, pt, static=True)
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), (B, P, k, dt)


def test_static_entry_point_limit_and_validation(gpu):
    lib = _lib.load()
    assert lib.trakhip_project_static_limit() == 36 << 20
    x = torch.zeros(32, 1024, dtype=torch.float16, device=gpu)
    out = torch.zeros(32, 307_200, dtype=torch.float32, device=gpu)
    args = lambda k, tiles: (ctypes.c_void_p(x.data_ptr()), _lib.F16, 32, 1024, 1024, ctypes.c_void_p(out.data_ptr()),
                             k, 0, tiles, 0, None)
    assert lib.trakhip_project_workspace(32, 1024, 307_200, 2) > 36 << 20
    assert lib.trakhip_project_static(*args(307_200, 2)) == -12
    assert lib.trakhip_project_static(*args(100, 2)) == -1
