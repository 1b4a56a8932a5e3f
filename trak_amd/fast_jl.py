"""Function namespace of the reference's `fast_jl` extension, backed by libtrakhip.

`project_{rademacher,normal}_{8,16,32}(input, N, seed, num_feature_tiles) -> Tensor`
(fast_jl/fast_jl.cu:81-110).  The numeric suffix is the number of rows the reference
processes per kernel launch; here every variant walks the batch in groups of 32 rows and
the suffix does not change the result.
"""
import ctypes

import torch

from . import _lib

_DTYPES = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}
_workspaces = {}


def _workspace(device, nbytes):
    """One growing scratch buffer per device (stands in for the per-call torch::zeros of
    fast_jl/fast_jl.cu:48-49).  Calls on one device must not overlap on different streams."""
    buf = _workspaces.get(device)
    if buf is None or buf.numel() < nbytes:
        buf = None
        _workspaces.pop(device, None)
        buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _workspaces[device] = buf
    return buf


def free_workspaces():
    _workspaces.clear()


def _project(input, N, seed, num_feature_tiles, proj_type, ld=None):
    # fast_jl/fast_jl.cu:20-27: CHECK_INPUT -> RuntimeError
    if not isinstance(input, torch.Tensor):
        raise TypeError("input must be a torch.Tensor")
    if not input.is_cuda:
        raise RuntimeError("input must be a CUDA tensor")
    if input.dim() != 2:
        raise RuntimeError("input must be 2D")
    if input.dtype not in _DTYPES:
        raise RuntimeError("input must be fp16, bf16 or fp32")
    if input.stride(1) != 1 and input.shape[1] > 1:
        raise RuntimeError("input must be contiguous")
    B, P = input.shape
    if ld is None:
        ld = input.stride(0) if B > 1 else max(P, 1)
        if ld < P:
            raise RuntimeError("input must be contiguous")
    N, seed, tiles = int(N), int(seed) & 0xFFFFFFFF, int(num_feature_tiles)
    lib = _lib.load()
    if N <= 0 or N % 512 != 0:
        _lib.check(_lib.ERR_PROJ_DIM)
    with torch.cuda.device(input.device):
        out = torch.empty((B, N), dtype=torch.float32, device=input.device)
        nbytes = lib.trakhip_project_workspace(B, P, N, tiles)
        ws = _workspace(input.device, nbytes)
        stream = torch.cuda.current_stream(input.device).cuda_stream
        code = lib.trakhip_project(
            ctypes.c_void_p(input.data_ptr()),
            _DTYPES[input.dtype],
            B,
            P,
            ld,
            ctypes.c_void_p(out.data_ptr()),
            ctypes.c_void_p(ws.data_ptr()),
            ws.numel(),
            N,
            seed,
            tiles,
            proj_type,
            ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return out


def project_rademacher_8(input, N, seed, num_feature_tiles):
    return _project(input, N, seed, num_feature_tiles, _lib.RADEMACHER)


def project_rademacher_16(input, N, seed, num_feature_tiles):
    return _project(input, N, seed, num_feature_tiles, _lib.RADEMACHER)


def project_rademacher_32(input, N, seed, num_feature_tiles):
    return _project(input, N, seed, num_feature_tiles, _lib.RADEMACHER)


def project_normal_8(input, N, seed, num_feature_tiles):
    return _project(input, N, seed, num_feature_tiles, _lib.NORMAL)


def project_normal_16(input, N, seed, num_feature_tiles):
    return _project(input, N, seed, num_feature_tiles, _lib.NORMAL)


def project_normal_32(input, N, seed, num_feature_tiles):
    return _project(input, N, seed, num_feature_tiles, _lib.NORMAL)


def materialize(seed, num_feature_tiles, P, f0, nf, c0, nc, proj_type, device=None):
    """Block S[f0:f0+nf, c0:c0+nc] of the matrix `project_*` uses, as fp32.  device=None runs
    the library's host code and returns a CPU tensor; a CUDA device runs the device kernel."""
    lib = _lib.load()
    pt = _lib.NORMAL if str(getattr(proj_type, "value", proj_type)) in ("normal", "1") else _lib.RADEMACHER
    if device is None or torch.device(device).type == "cpu":
        out = torch.empty((nf, nc), dtype=torch.float32)
        code = lib.trakhip_materialize(
            int(seed) & 0xFFFFFFFF, num_feature_tiles, P, f0, nf, c0, nc, pt, ctypes.c_void_p(out.data_ptr()), 0, None
        )
        _lib.check(code)
        return out
    device = torch.device(device)
    with torch.cuda.device(device):
        out = torch.empty((nf, nc), dtype=torch.float32, device=device)
        stream = torch.cuda.current_stream(device).cuda_stream
        code = lib.trakhip_materialize(
            int(seed) & 0xFFFFFFFF,
            num_feature_tiles,
            P,
            f0,
            nf,
            c0,
            nc,
            pt,
            ctypes.c_void_p(out.data_ptr()),
            1,
            ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return out
