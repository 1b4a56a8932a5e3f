"""Function namespace of the reference's `fast_jl` extension, backed by libtrakhip.

`project_{rademacher,normal}_{8,16,32}(input, N, seed, num_feature_tiles) -> Tensor`
(fast_jl/fast_jl.cu:81-110).  The numeric suffix is the number of rows the reference
processes per kernel launch; here every variant walks the batch in passes of 64 rows (16-bit
gradients) or 32 rows (fp32) and the suffix does not change the result.
"""
import contextlib
import ctypes
from collections import OrderedDict

import torch

from . import _lib

_DTYPES = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}
_workspaces = OrderedDict()  # (device, stream) -> scratch buffer, least recently used first
_WORKSPACE_CACHE = 8         # streams that keep a scratch buffer (tens of MiB each at proj_dim 4096)
_segment_tables = {}  # (device, stream, rows) -> device table; the key holds every pointer, so a hit is exact
_SEGMENT_TABLE_CACHE = 16
_workspace_bytes = {}  # (B, P, N, tiles, device index) -> trakhip_project_workspace(...)
_NO_CONTEXT = contextlib.nullcontext()


def _on(device):
    """Context that makes `device` current; nothing to do (and nothing to pay) when it already is."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return _NO_CONTEXT if index == torch.cuda.current_device() else torch.cuda.device(device)


def _workspace_size(lib, B, P, N, tiles, device):
    key = (B, P, N, tiles, device.index)
    n = _workspace_bytes.get(key)
    if n is None:
        if len(_workspace_bytes) > 256:
            _workspace_bytes.clear()
        n = _workspace_bytes[key] = lib.trakhip_project_workspace(B, P, N, tiles)
    return n


def _workspace(device, nbytes, stream=None):
    """One growing scratch buffer per device and stream (stands in for the per-call torch::zeros of
    fast_jl/fast_jl.cu:48-49): calls on different streams never share scratch, calls on one stream
    are ordered by the stream.  The buffers of the `_WORKSPACE_CACHE` most recently used streams are
    kept (a program that keeps making streams does not keep a buffer per stream handle ever seen);
    `free_workspaces()` releases them all."""
    if stream is None:
        stream = torch.cuda.current_stream(device).cuda_stream
    key = (device, stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = None
        _workspaces.pop(key, None)
        while len(_workspaces) >= _WORKSPACE_CACHE:
            _workspaces.popitem(last=False)
        buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    else:
        _workspaces.move_to_end(key)
    return buf


def free_workspaces():
    """Releases the cached scratch buffers, segment tables and size look-ups."""
    _workspaces.clear()
    _segment_tables.clear()
    _workspace_bytes.clear()


def _segment_table(device, rows):
    """Device array of trakhip_segment {ptr, first, numel, ld} for these rows.  Gradient buffers
    come back at the same addresses batch after batch (caching allocator), so the upload is
    usually skipped.  The cache is per stream: the upload is enqueued on the stream that later
    reads the table, so a hit never races with it."""
    key = (device, torch.cuda.current_stream(device).cuda_stream, rows)
    table = _segment_tables.get(key)
    if table is None:
        if len(_segment_tables) >= _SEGMENT_TABLE_CACHE:
            _segment_tables.pop(next(iter(_segment_tables)))
        host = torch.tensor(rows, dtype=torch.int64).pin_memory()
        table = host.to(device, non_blocking=True)
        _segment_tables[key] = table
        table._host = host  # keeps the pinned source alive until the copy has certainly run
    return table


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
    device = input.device
    with _on(device):
        out = torch.empty((B, N), dtype=torch.float32, device=device)
        stream = torch.cuda.current_stream(device).cuda_stream
        ws = _workspace(device, _workspace_size(lib, B, P, N, tiles, device), stream)
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


def _flat_rows(p):
    """[B, numel] view of one gradient tensor [B, ...] with unit inner stride (a copy only when the
    tensor cannot be viewed that way); tensors with fewer than two dims count as one column
    (trak/utils.py:99-104)."""
    B = p.shape[0]
    flat = p.reshape(B, 1) if p.dim() < 2 else p.flatten(start_dim=1)
    if flat.shape[1] > 1 and flat.stride(1) != 1:
        flat = flat.contiguous()
    if B > 1 and flat.stride(0) < flat.shape[1]:
        flat = flat.contiguous()
    return flat


def gather_supported(tensors):
    """True when a list of gradient tensors can be projected in place (no flatten-and-copy): same
    supported dtype, same CUDA device, same batch size."""
    tensors = list(tensors)
    if not tensors:
        return False
    t0 = tensors[0]
    if not isinstance(t0, torch.Tensor) or not t0.is_cuda or t0.dtype not in _DTYPES or t0.dim() < 1:
        return False
    return all(
        isinstance(t, torch.Tensor) and t.device == t0.device and t.dtype == t0.dtype and t.dim() >= 1
        and t.shape[0] == t0.shape[0] and t.numel() > 0
        for t in tensors
    )


def _proj_type_code(proj_type):
    return _lib.NORMAL if str(getattr(proj_type, "value", proj_type)) in ("normal", "1") else _lib.RADEMACHER


def _check_destination(out, B, N, device):
    """`out` receives [B, N] results: a CUDA tensor on `device`, or a page-locked CPU tensor that the
    kernel writes over PCIe (pageable memory would fault the GPU, so it is refused here)."""
    if not isinstance(out, torch.Tensor) or out.dim() != 2 or tuple(out.shape) != (B, N):
        raise RuntimeError(f"out must be a [{B}, {N}] tensor")
    if out.dtype not in _DTYPES:
        raise RuntimeError("out must be fp16, bf16 or fp32")
    if out.is_cuda:
        if out.device != device:
            raise RuntimeError("out must live on the input's device")
    elif not out.is_pinned():
        raise RuntimeError("a CPU destination must be page-locked (pin_memory)")
    if out.stride(1) != 1 or (B > 1 and (out.stride(0) < N or out.stride(0) % 4)):
        raise RuntimeError("out rows must be contiguous with a pitch that is a multiple of 4 elements")


def project_into(source, N, seed, num_feature_tiles, proj_type, out, scale=1.0):
    """out[B, N] = cast(project(source) * scale): the projection with the epilogue of
    TRAKer.featurize (`grads /= normalize_factor; grads.to(dtype).cpu()`, trak/traker.py:426-428)
    folded into the cross-tile sum.  `source` is a 2-D CUDA tensor [B, P] or a list of per-parameter
    gradient tensors [B, ...] (projected in place, as `project_gather`); `out` is a CUDA tensor or a
    page-locked CPU tensor (fp16 / bf16 / fp32), written on the current stream: synchronize (or
    wait on an event recorded after this call) before reading a CPU destination."""
    lib = _lib.load()
    N, seed, tiles = int(N), int(seed) & 0xFFFFFFFF, int(num_feature_tiles)
    if N <= 0 or N % 512 != 0:
        _lib.check(_lib.ERR_PROJ_DIM)
    pt = _proj_type_code(proj_type)
    if isinstance(source, torch.Tensor):
        if not source.is_cuda or source.dim() != 2 or source.dtype not in _DTYPES:
            raise RuntimeError("input must be a 2D CUDA tensor of fp16, bf16 or fp32")
        if source.shape[1] > 1 and source.stride(1) != 1:
            raise RuntimeError("input must be contiguous")
        B, P = source.shape
        ld = source.stride(0) if B > 1 else max(P, 1)
        if ld < P:
            raise RuntimeError("input must be contiguous")
        device, dtype, esz = source.device, source.dtype, source.element_size()
        rows = None
    else:
        tensors = list(source)
        if not gather_supported(tensors):
            raise RuntimeError("project_into needs CUDA tensors of one supported dtype, device and batch size")
        flats = [_flat_rows(t) for t in tensors]
        device, dtype, esz = flats[0].device, flats[0].dtype, flats[0].element_size()
        B = flats[0].shape[0]
        rows, first = [], 0
        for f in flats:
            numel = f.shape[1]
            rows.append([f.data_ptr(), first, numel, f.stride(0) if B > 1 else numel])
            first += numel
        P = first
    _check_destination(out, B, N, device)
    out_ld = out.stride(0) if B > 1 else N
    with _on(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        ws = _workspace(device, _workspace_size(lib, B, P, N, tiles, device), stream)
        step = int(lib.trakhip_project_rows_per_pass(_DTYPES[dtype], pt))
        for b0 in range(0, B, step):
            nb = min(step, B - b0)
            if rows is None:
                code = lib.trakhip_project_partials(
                    ctypes.c_void_p(source.data_ptr() + b0 * ld * esz), _DTYPES[dtype], nb, P, ld,
                    ctypes.c_void_p(ws.data_ptr()), ws.numel(), N, seed, tiles, pt, ctypes.c_void_p(stream),
                )
            else:
                table_dev = _segment_table(device, tuple((p + b0 * l * esz, fi, n, l) for p, fi, n, l in rows))
                code = lib.trakhip_project_gather_partials(
                    ctypes.c_void_p(table_dev.data_ptr()), len(rows), _DTYPES[dtype], nb, P,
                    ctypes.c_void_p(ws.data_ptr()), ws.numel(), N, seed, tiles, pt, ctypes.c_void_p(stream),
                )
            _lib.check(code)
            code = lib.trakhip_project_reduce_store(
                ctypes.c_void_p(ws.data_ptr()), nb, P, N, tiles, float(scale), _DTYPES[out.dtype],
                ctypes.c_void_p(out.data_ptr() + b0 * out_ld * out.element_size()), out_ld,
                ctypes.c_void_p(stream),
            )
            _lib.check(code)
    return out


def project_gather(tensors, N, seed, num_feature_tiles, proj_type, scale=1.0):
    """Projects the gradient given as a list of per-parameter tensors [B, ...] (in order) without
    materializing the [B, P] matrix: same result, bit for bit, as `project_*` on
    `trak.utils.vectorize` of the same tensors.  Returns fp32 [B, N] times `scale`."""
    tensors = list(tensors)
    if not gather_supported(tensors):
        raise RuntimeError("project_gather needs CUDA tensors of one supported dtype, device and batch size")
    t0 = tensors[0]
    with _on(t0.device):
        out = torch.empty((t0.shape[0], int(N)), dtype=torch.float32, device=t0.device)
    return project_into(tensors, N, seed, num_feature_tiles, proj_type, out, scale)


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
    pt = _proj_type_code(proj_type)
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
