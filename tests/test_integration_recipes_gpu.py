"""The two ways a TRAK installation binds the library without using this package's projector classes.

1. The package's `fast_jl` namespace registered under the name the reference imports: the call sequence of
   the reference's own `CudaProjector` (trak/projectors.py:372-378 the probe at construction, :389-410 the
   function looked up by name from the batch size, seed + 10^4 * model_id, the device's multiprocessor count
   as the number of feature tiles) must go through and give the oracle's numbers.
2. A binding written from the C header alone (ctypes, no import of this package's loader): what a maintainer
   would put in place of the pybind11 module of fast_jl/fast_jl.cu:102-110.
"""
import ctypes
import os
import sys

import numpy as np
import pytest
import torch

from oracle import jl_oracle as npo

pytestmark = pytest.mark.gpu

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "trak_amd", "libtrakhip.so")


def _rel_rows(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float((np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)).max())


@pytest.fixture
def fast_jl_stand_in(gpu):
    import trak_amd.fast_jl

    assert "fast_jl" not in sys.modules
    sys.modules["fast_jl"] = trak_amd.fast_jl
    yield
    del sys.modules["fast_jl"]


def test_reference_projector_call_sequence_through_the_stand_in_module(gpu, c_oracle, fast_jl_stand_in):
    from trak_amd import CudaProjector, ProjectionType

    num_sms = torch.cuda.get_device_properties(gpu.index).multi_processor_count
    import fast_jl

    # the probe the reference runs when a projector is constructed
    probe = fast_jl.project_rademacher_8(torch.zeros(8, 1_000, device="cuda"), 512, 0, num_sms)
    assert probe.shape == (8, 512) and probe.dtype == torch.float32 and not probe.any()

    P, k, seed = 30_011, 1024, 42
    gen = torch.Generator(device="cpu").manual_seed(5)
    for proj_type, kind in (("rademacher", npo.RADEMACHER), ("normal", npo.NORMAL)):
        for batch_size, max_batch_size, model_id in ((5, 32, 0), (13, 32, 3), (32, 32, 1), (13, 8, 2)):
            grads = torch.randn(batch_size, P, generator=gen).half().to(gpu)
            effective = 8 if batch_size <= 8 else 16 if batch_size <= 16 else 32
            effective = min(max_batch_size, effective)
            fn = getattr(fast_jl, f"project_{proj_type}_{effective}")
            call_seed = seed + int(1e4) * model_id
            out = fn(grads, k, call_seed, num_sms)
            assert out.shape == (batch_size, k) and out.dtype == torch.float32 and out.device == grads.device
            want = c_oracle.project(grads.float().cpu().numpy(), call_seed, num_sms, 0, 64, kind)
            assert _rel_rows(out[:, :64].cpu().numpy(), want) < 1e-3, (proj_type, batch_size)
            # this package's projector class makes the same call
            mine = CudaProjector(P, k, seed, ProjectionType(proj_type), gpu, max_batch_size).project(grads, model_id)
            assert torch.equal(mine, out), (proj_type, batch_size)
    # what the reference's callers catch: a projection dimension that is not a multiple of 512
    with pytest.raises((ValueError, RuntimeError)):
        fast_jl.project_rademacher_8(torch.zeros(8, 1_000, device="cuda"), 500, 0, num_sms)


def _bind():
    lib = ctypes.CDLL(LIB)
    u32, u64, vp = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p
    lib.trakhip_project_workspace.restype = ctypes.c_size_t
    lib.trakhip_project_workspace.argtypes = [u64, u64, u32, u32]
    lib.trakhip_project.restype = ctypes.c_int
    lib.trakhip_project.argtypes = [vp, ctypes.c_int, u64, u64, u64, vp, vp, ctypes.c_size_t, u32, u32, u32,
                                    ctypes.c_int, vp]
    lib.trakhip_strerror.restype = ctypes.c_char_p
    dtypes = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}

    def project(x, N, seed, num_feature_tiles, proj_type):
        B, P = x.shape
        out = torch.empty(B, N, dtype=torch.float32, device=x.device)
        ws = torch.empty(lib.trakhip_project_workspace(B, P, N, num_feature_tiles), dtype=torch.uint8, device=x.device)
        rc = lib.trakhip_project(x.data_ptr(), dtypes[x.dtype], B, P, x.stride(0), out.data_ptr(), ws.data_ptr(),
                                 ws.numel(), N, seed & 0xFFFFFFFF, num_feature_tiles, proj_type,
                                 torch.cuda.current_stream().cuda_stream)
        if rc == -1:
            raise ValueError(lib.trakhip_strerror(rc).decode())
        if rc:
            raise RuntimeError(lib.trakhip_strerror(rc).decode())
        return out

    return project


def test_binding_written_from_the_header_alone(gpu, c_oracle):
    from trak_amd import fast_jl

    project = _bind()
    gen = torch.Generator(device="cpu").manual_seed(11)
    for B, P, k, tiles, dt, kind in ((8, 9_001, 512, 7, torch.float32, npo.RADEMACHER),
                                     (70, 40_003, 1536, 256, torch.float16, npo.RADEMACHER),
                                     (33, 12_345, 2048, 108, torch.bfloat16, npo.NORMAL)):
        x = torch.randn(B, P, generator=gen).to(dt).to(gpu)
        out = project(x, k, 2**32 + 77, tiles, kind)        # the seed is reduced to 32 bits by the caller
        want = c_oracle.project(x.float().cpu().numpy(), 77, tiles, k - 32, 32, kind)
        assert _rel_rows(out[:, k - 32:].cpu().numpy(), want) < (1e-5 if dt == torch.float32 else 1e-3), (B, P, k)
        name = "rademacher" if kind == npo.RADEMACHER else "normal"
        assert torch.equal(out, getattr(fast_jl, f"project_{name}_32")(x, k, 77, tiles))
        # a row pitch larger than the row: a view of a wider matrix
        wide = torch.zeros(B, P + 24, dtype=dt, device=gpu)
        wide[:, :P] = x
        assert torch.equal(project(wide[:, :P], k, 77, tiles, kind), out)
    with pytest.raises(ValueError):
        project(torch.zeros(8, 1000, device=gpu), 500, 0, 4, 0)
