"""Helpers on either side of the projection and scoring kernels.

Mirrors the hot-path part of the reference's trak/utils.py: `vectorize` (:80-110),
`get_parameter_chunk_sizes` (:297-331) and `get_matrix_mult` (:248-294).
"""
import ctypes
import logging

import numpy as np
import torch

from . import _lib


def vectorize(g, arr=None, device="cuda"):
    """Flattens a dict {name: grad[batch, ...]} to one [batch, num_params] tensor, in dict
    order (trak/utils.py:80-110).  Gradients with fewer than two dims count as one column."""
    if arr is None:
        first = next(iter(g.values()))
        batch_size = first.shape[0]
        num_params = 0
        for param in g.values():
            assert param.shape[0] == batch_size
            num_params += int(param.numel() / batch_size)
        arr = torch.empty(size=(batch_size, num_params), dtype=first.dtype, device=device)

    pointer = 0
    for param in g.values():
        if param.dim() < 2:
            width = 1
            flat = param.data.reshape(-1, 1)
        else:
            width = param[0].numel()
            flat = param.flatten(start_dim=1).data
        arr[:, pointer : pointer + width] = flat.to(device)
        pointer += width
    return arr


def chunk_sizes_from_numels(numels, batch_size):
    """Greedy grouping of parameter sizes into chunks whose element count times the batch
    size stays below 2^32 (trak/utils.py:312-331).  Returns (max_chunk_size, params_per_chunk)."""
    numels = np.array([int(n) for n in numels], dtype=np.int64)
    max_chunk_size = int(np.iinfo(np.uint32).max // batch_size)
    params_per_chunk = []
    chunk_sum = 0
    for ps in numels:
        if chunk_sum + ps >= max_chunk_size:
            params_per_chunk.append(int(chunk_sum))
            chunk_sum = 0
        chunk_sum += int(ps)
    rest = int(numels.sum()) - int(np.sum(params_per_chunk))
    if rest > 0:
        params_per_chunk.append(rest)
    return max_chunk_size, params_per_chunk


def get_parameter_chunk_sizes(model, batch_size):
    """(max_chunk_size, params_per_chunk) for a torch module (trak/utils.py:297-331)."""
    return chunk_sizes_from_numels([p.numel() for p in model.parameters()], batch_size)


def _as_f32_rows(t, name):
    if t.dim() != 2:
        raise RuntimeError(f"{name} must be 2D")
    if t.dtype != torch.float32:
        t = t.float()
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    return t


def _ld(t):
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def gemm_nt(a, b, out=None, alpha=1.0, beta=0.0, row_scale=None):
    """out[M, N] = alpha * a[M, K] @ b[N, K].T + beta * out (fp32 on the GPU), rows optionally
    scaled by row_scale[M]."""
    a = _as_f32_rows(a, "a")
    b = _as_f32_rows(b, "b")
    if not a.is_cuda or b.device != a.device:
        raise RuntimeError("gemm_nt needs both operands on the same GPU")
    M, K = a.shape
    N, K2 = b.shape
    if K != K2:
        raise RuntimeError(f"inner dimensions differ: {K} vs {K2}")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
        beta = 0.0
    if out.dtype != torch.float32 or out.shape != (M, N) or out.stride(1) != 1:
        raise RuntimeError("out must be an fp32 [M, N] tensor with unit column stride")
    rs = None
    if row_scale is not None:
        rs = row_scale.to(device=a.device, dtype=torch.float32).contiguous().reshape(-1)
        if rs.numel() != M:
            raise RuntimeError("row_scale must have M elements")
    lib = _lib.load()
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        code = lib.trakhip_gemm_nt(
            ctypes.c_void_p(a.data_ptr()),
            _ld(a),
            ctypes.c_void_p(b.data_ptr()),
            _ld(b),
            ctypes.c_void_p(out.data_ptr()),
            _ld(out),
            M,
            N,
            K,
            float(alpha),
            float(beta),
            ctypes.c_void_p(rs.data_ptr()) if rs is not None else None,
            ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return out


def gemm_tn(a, b, out=None, alpha=1.0, beta=0.0):
    """out[M, N] = alpha * a[K, M].T @ b[K, N] + beta * out (fp32 on the GPU)."""
    a = _as_f32_rows(a, "a")
    b = _as_f32_rows(b, "b")
    if not a.is_cuda or b.device != a.device:
        raise RuntimeError("gemm_tn needs both operands on the same GPU")
    K, M = a.shape
    K2, N = b.shape
    if K != K2:
        raise RuntimeError(f"inner dimensions differ: {K} vs {K2}")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
        beta = 0.0
    if out.dtype != torch.float32 or out.shape != (M, N) or out.stride(1) != 1:
        raise RuntimeError("out must be an fp32 [M, N] tensor with unit column stride")
    lib = _lib.load()
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        code = lib.trakhip_gemm_tn(
            ctypes.c_void_p(a.data_ptr()),
            _ld(a),
            ctypes.c_void_p(b.data_ptr()),
            _ld(b),
            ctypes.c_void_p(out.data_ptr()),
            _ld(out),
            M,
            N,
            K,
            float(alpha),
            float(beta),
            ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return out


class SplitOperand:
    """A matrix [rows, K] in the operand format of `gemm_nt_split`: three bf16 planes whose sum is
    the matrix exactly (fp32 source), the matrix itself as one plane (fp16 / bf16 source), or - from
    `split2_rows` - two fp16 planes of the row-scaled matrix with the inverse row factors in `scales`."""

    def __init__(self, planes, rows, K, dtype, scales=None):
        self.planes, self.rows, self.K, self.dtype, self.scales = planes, int(rows), int(K), dtype, scales

    @property
    def device(self):
        return self.planes.device


def split_rows(t, transposed=False):
    """Brings the CUDA matrix `t` (fp32, fp16 or bf16; anything else is converted to fp32) into the
    operand format of `gemm_nt_split`.  transposed=False: the operand is `t` itself ([rows, K]);
    transposed=True: the operand is `t.T` (t is [K, rows]), read in place."""
    if t.dim() != 2:
        raise RuntimeError("t must be 2D")
    if t.dtype not in _STORE_DTYPES:
        t = t.float()
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    if not t.is_cuda:
        raise RuntimeError("split_rows needs a CUDA tensor")
    rows, K = (t.shape[1], t.shape[0]) if transposed else (t.shape[0], t.shape[1])
    lib = _lib.load()
    code_dtype = _STORE_DTYPES[t.dtype]
    nbytes = lib.trakhip_split_bytes(rows, K, code_dtype)
    with torch.cuda.device(t.device):
        planes = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=t.device)
        stream = torch.cuda.current_stream(t.device).cuda_stream
        code = lib.trakhip_split_rows(
            ctypes.c_void_p(t.data_ptr()), code_dtype, _ld(t), rows, K, int(bool(transposed)),
            ctypes.c_void_p(planes.data_ptr()), planes.numel(), ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return SplitOperand(planes, rows, K, t.dtype)


def split2_rows(t, transposed=False):
    """The cheaper, slightly less accurate operand format for an fp32 CUDA matrix: every row times a power
    of two, then two fp16 planes (22 significand bits for entries within 2^-18 of the row's largest
    magnitude).  `gemm_nt_split` / `gram_split` of two such operands run three fp16 MFMAs per k step
    instead of six bf16 ones.  Arguments as for `split_rows`."""
    if t.dim() != 2:
        raise RuntimeError("t must be 2D")
    t = t.float()
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    if not t.is_cuda:
        raise RuntimeError("split2_rows needs a CUDA tensor")
    rows, K = (t.shape[1], t.shape[0]) if transposed else (t.shape[0], t.shape[1])
    lib = _lib.load()
    nbytes = lib.trakhip_split2_bytes(rows, K)
    with torch.cuda.device(t.device):
        planes = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=t.device)
        scales = torch.empty(2 * max(rows, 1), dtype=torch.float32, device=t.device)
        stream = torch.cuda.current_stream(t.device).cuda_stream
        code = lib.trakhip_split2_rows(
            ctypes.c_void_p(t.data_ptr()), _ld(t), rows, K, int(bool(transposed)), ctypes.c_void_p(planes.data_ptr()),
            planes.numel(), ctypes.c_void_p(scales.data_ptr()), ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return SplitOperand(planes, rows, K, torch.float32, scales=scales)


def split_pair(a, b, a_transposed=False):
    """Both operands of one product in a common format: 16-bit operands of one type stay as they
    are (one plane each), any other combination is multiplied from fp32 splits."""
    if a.dtype != b.dtype or a.dtype not in (torch.float16, torch.bfloat16):
        a, b = a.float(), b.float()
    return split_rows(a, transposed=a_transposed), split_rows(b)


def gemm_nt_split(a, b, out=None, alpha=1.0, beta=0.0, row_scale=None):
    """out[M, N] = alpha * A @ B.T + beta * out (rows optionally scaled) for SplitOperands A [M, K]
    and B [N, K] made from matrices of one dtype: exact products on the 16-bit matrix cores, fp32
    accumulation, fp32-level accuracy."""
    if not isinstance(a, SplitOperand) or not isinstance(b, SplitOperand):
        raise TypeError("gemm_nt_split takes SplitOperand arguments (see split_rows)")
    if a.K != b.K or a.device != b.device or a.dtype != b.dtype or (a.scales is None) != (b.scales is None):
        raise RuntimeError("operands must share the inner dimension, the device, the source dtype and the format")
    M, N, K = a.rows, b.rows, a.K
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
        beta = 0.0
    if out.dtype != torch.float32 or tuple(out.shape) != (M, N) or (N > 1 and out.stride(1) != 1) or out.device != a.device:
        raise RuntimeError("out must be an fp32 [M, N] tensor with unit column stride on the operands' device")
    rs = None
    if row_scale is not None:
        rs = row_scale.to(device=a.device, dtype=torch.float32).contiguous().reshape(-1)
        if rs.numel() != M:
            raise RuntimeError("row_scale must have M elements")
    lib = _lib.load()
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        rs_ptr = ctypes.c_void_p(rs.data_ptr()) if rs is not None else None
        if a.scales is not None:
            code = lib.trakhip_gemm_nt_split2(
                ctypes.c_void_p(a.planes.data_ptr()), ctypes.c_void_p(a.scales.data_ptr()), M,
                ctypes.c_void_p(b.planes.data_ptr()), ctypes.c_void_p(b.scales.data_ptr()), N, K,
                ctypes.c_void_p(out.data_ptr()), _ld(out), float(alpha), float(beta), rs_ptr, ctypes.c_void_p(stream),
            )
        else:
            code = lib.trakhip_gemm_nt_split(
                ctypes.c_void_p(a.planes.data_ptr()), M, ctypes.c_void_p(b.planes.data_ptr()), N, K,
                _STORE_DTYPES[a.dtype], ctypes.c_void_p(out.data_ptr()), _ld(out), float(alpha), float(beta),
                rs_ptr, ctypes.c_void_p(stream),
            )
    _lib.check(code)
    return out


def nt16_ok(a, b):
    """Whether `gemm_nt16` can read these operands where they are."""
    if a.dtype != b.dtype or a.dtype not in (torch.float16, torch.bfloat16):
        return False
    if a.dim() != 2 or b.dim() != 2 or not a.is_cuda or a.device != b.device:
        return False
    if a.shape[1] != b.shape[1] or a.shape[1] == 0 or a.shape[1] % 64:
        return False
    for t in (a, b):
        if t.stride(1) != 1 or t.data_ptr() % 16 or (t.shape[0] > 1 and (t.stride(0) % 8 or t.stride(0) < t.shape[1])):
            return False
        if max(t.stride(0), t.shape[1]) >= 1 << 23:  # the kernel keeps a lane's offset inside a tile in 32 bits
            return False
    return True


def gemm_nt16(a, b, out=None, alpha=1.0, beta=0.0, row_scale=None):
    """out[M, N] (fp32) = alpha * a @ b.T + beta * out (rows optionally scaled) for fp16 or bf16 CUDA
    matrices a [M, K], b [N, K] read in place: K a multiple of 64, rows 16-byte aligned (see
    `matmul_nt` for the general case).  Exact products, fp32 accumulation."""
    if not nt16_ok(a, b):
        raise RuntimeError("gemm_nt16 needs two fp16 or two bf16 CUDA matrices with K % 64 == 0 and 16-byte aligned rows")
    M, N, K = a.shape[0], b.shape[0], a.shape[1]
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
        beta = 0.0
    if out.dtype != torch.float32 or tuple(out.shape) != (M, N) or (N > 1 and out.stride(1) != 1) or out.device != a.device:
        raise RuntimeError("out must be an fp32 [M, N] tensor with unit column stride on the operands' device")
    rs = None
    if row_scale is not None:
        rs = row_scale.to(device=a.device, dtype=torch.float32).contiguous().reshape(-1)
        if rs.numel() != M:
            raise RuntimeError("row_scale must have M elements")
    lib = _lib.load()
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        code = lib.trakhip_gemm_nt16(
            ctypes.c_void_p(a.data_ptr()), _ld(a), ctypes.c_void_p(b.data_ptr()), _ld(b), _STORE_DTYPES[a.dtype],
            ctypes.c_void_p(out.data_ptr()), _ld(out), M, N, K, float(alpha), float(beta),
            ctypes.c_void_p(rs.data_ptr()) if rs is not None else None, ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return out


def matmul_nt(a, b, out=None, alpha=1.0, beta=0.0, row_scale=None, two_planes=False):
    """alpha * a @ b.T + beta * out with fp32 accuracy on the 16-bit matrix cores, whatever the operand
    types: two fp16 or two bf16 matrices that qualify are multiplied where they are (`gemm_nt16`),
    other 16-bit pairs as single planes, anything else from fp32 splits (`gemm_nt_split`; the exact
    three-plane split, or the two-plane one of `split2_rows` when `two_planes` is set)."""
    if nt16_ok(a, b):
        return gemm_nt16(a, b, out=out, alpha=alpha, beta=beta, row_scale=row_scale)
    if two_planes and not (a.dtype == b.dtype and a.dtype in (torch.float16, torch.bfloat16)):
        return gemm_nt_split(split2_rows(a), split2_rows(b), out=out, alpha=alpha, beta=beta, row_scale=row_scale)
    return gemm_nt_split(*split_pair(a, b), out=out, alpha=alpha, beta=beta, row_scale=row_scale)


def gram_split(a, out=None, alpha=1.0, beta=0.0):
    """out[N, N] = alpha * A @ A.T + beta * out for a SplitOperand A [N, K]: the lower-triangle tiles
    are computed and mirrored, so the result is exactly symmetric at about half the cost of
    `gemm_nt_split(a, a)`.  An `out` that is accumulated into must come from this function."""
    if not isinstance(a, SplitOperand):
        raise TypeError("gram_split takes a SplitOperand (see split_rows)")
    N = a.rows
    if out is None:
        out = torch.empty((N, N), dtype=torch.float32, device=a.device)
        beta = 0.0
    if out.dtype != torch.float32 or tuple(out.shape) != (N, N) or (N > 1 and out.stride(1) != 1) or out.device != a.device:
        raise RuntimeError("out must be an fp32 [N, N] tensor with unit column stride on the operand's device")
    lib = _lib.load()
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        # scratch that lets a product with few tiles share its k range out over the idle CUs
        two = a.scales is not None
        ws_bytes = lib.trakhip_gram_split_workspace(N, a.K, _STORE_DTYPES[a.dtype], int(two))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
        ws_ptr = ctypes.c_void_p(ws.data_ptr()) if ws is not None else None
        if two:
            code = lib.trakhip_gram_split2(
                ctypes.c_void_p(a.planes.data_ptr()), ctypes.c_void_p(a.scales.data_ptr()), N, a.K,
                ctypes.c_void_p(out.data_ptr()), _ld(out), float(alpha), float(beta), ws_ptr, ws_bytes,
                ctypes.c_void_p(stream),
            )
        else:
            code = lib.trakhip_gram_split(
                ctypes.c_void_p(a.planes.data_ptr()), N, a.K, _STORE_DTYPES[a.dtype], ctypes.c_void_p(out.data_ptr()),
                _ld(out), float(alpha), float(beta), ws_ptr, ws_bytes, ctypes.c_void_p(stream),
            )
    _lib.check(code)
    return out


def _inverse_call(a, lambda_reg, normalize, general):
    """One call of trakhip_spd_inverse (Cholesky) or trakhip_general_inverse (pivoted elimination):
    (inverse, mean_abs, status word)."""
    n = a.shape[0]
    lib = _lib.load()
    size, run = ((lib.trakhip_general_inverse_workspace, lib.trakhip_general_inverse) if general
                 else (lib.trakhip_spd_inverse_workspace, lib.trakhip_spd_inverse))
    with torch.cuda.device(a.device):
        nbytes = size(n)
        if general and nbytes == 0:
            raise torch.linalg.LinAlgError(
                f"the matrix is not positive definite and too large (n = {n}) for the general inverse of this library")
        inv = torch.empty((n, n), dtype=torch.float32, device=a.device)
        mean_abs = torch.zeros(1, dtype=torch.float32, device=a.device)
        status = torch.zeros(1, dtype=torch.int32, device=a.device)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=a.device)
        stream = torch.cuda.current_stream(a.device).cuda_stream
        code = run(
            ctypes.c_void_p(a.data_ptr()),
            _ld(a),
            float(lambda_reg),
            ctypes.c_void_p(inv.data_ptr()),
            n,
            n,
            int(bool(normalize)),
            ctypes.c_void_p(mean_abs.data_ptr()),
            ctypes.c_void_p(status.data_ptr()),
            ctypes.c_void_p(ws.data_ptr()),
            ws.numel(),
            ctypes.c_void_p(stream),
        )
        _lib.check(code)
        bad = int(status.item())  # also orders the workspace's lifetime after the kernels
    return inv, mean_abs, bad


def general_inverse(a, lambda_reg=0.0, normalize=False):
    """(a + lambda*I)^-1 for any nonsingular fp32 matrix on the GPU, by elimination with
    partial pivoting - the pivoting of the LU behind torch.linalg.inv, the reference's call
    (trak/score_computers.py:163); with normalize=True divided by mean(|inverse|).  Returns (inverse,
    mean_abs).  An exactly singular matrix (a zero pivot) raises torch.linalg.LinAlgError, as the
    reference's call does; an inverse with huge or non-finite entries is returned as it is."""
    if a.dim() != 2 or a.shape[0] != a.shape[1]:
        raise RuntimeError("general_inverse needs a square matrix")
    a = _as_f32_rows(a, "a")
    if not a.is_cuda:
        raise RuntimeError("general_inverse needs a GPU tensor")
    inv, mean_abs, bad = _inverse_call(a, lambda_reg, normalize, general=True)
    if bad != 0:
        raise torch.linalg.LinAlgError(f"general_inverse: the matrix is singular (pivot {bad - 1} is zero)")
    return inv, mean_abs


def spd_inverse(a, lambda_reg=0.0, normalize=False, general_fallback=False):
    """(a + lambda*I)^-1 for a symmetric positive definite fp32 matrix on the GPU; with
    normalize=True the result is divided by mean(|inverse|) (trak/score_computers.py:160-166).
    Returns (inverse, mean_abs tensor of 1 element).

    A matrix that is not positive definite raises torch.linalg.LinAlgError, unless
    general_fallback=True: then it is inverted by `general_inverse` (elimination with partial
    pivoting on the device, the pivoting of the reference's torch.linalg.inv at
    trak/score_computers.py:163), which returns something for every matrix that is not exactly
    singular (a Gram matrix rounded to fp16, or one of deficient rank, is symmetric but need not
    be positive definite)."""
    if a.dim() != 2 or a.shape[0] != a.shape[1]:
        raise RuntimeError("spd_inverse needs a square matrix")
    a = _as_f32_rows(a, "a")
    if not a.is_cuda:
        raise RuntimeError("spd_inverse needs a GPU tensor")
    inv, mean_abs, bad = _inverse_call(a, lambda_reg, normalize, general=False)
    if bad != 0:
        if not general_fallback:
            raise torch.linalg.LinAlgError(
                f"spd_inverse: the matrix is not positive definite (pivot {bad - 1} is not positive)"
            )
        logging.getLogger("ScoreComputer").warning(
            "X^T X + lambda I is not positive definite (pivot %d): inverting it with partial pivoting, as the "
            "reference's LU does", bad - 1
        )
        return general_inverse(a, lambda_reg, normalize)
    return inv, mean_abs


_STORE_DTYPES = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


def scores_finalize(acc, divisor, row_factor, out):
    """out[i, j] = cast((acc[i, j] / divisor) * row_factor[i]): the closing expression of
    TRAKer.finalize_scores (trak/traker.py:670-678) for fp32 score sums `acc` [N, M] on the GPU.
    `out` [N, M] (fp16 / bf16 / fp32) is a CUDA tensor on the same device or a page-locked CPU
    tensor; row_factor (N values, or None) is moved to the device as fp32.  Enqueued on the
    current stream; synchronize before reading a CPU destination."""
    if not acc.is_cuda or acc.dtype != torch.float32 or acc.dim() != 2 or (acc.shape[1] > 1 and acc.stride(1) != 1):
        raise RuntimeError("acc must be an fp32 [N, M] CUDA tensor with unit column stride")
    N, M = acc.shape
    if out.dim() != 2 or tuple(out.shape) != (N, M) or out.dtype not in _STORE_DTYPES:
        raise RuntimeError(f"out must be a [{N}, {M}] tensor of fp16, bf16 or fp32")
    if M > 1 and out.stride(1) != 1:
        raise RuntimeError("out must have unit column stride")
    if out.is_cuda:
        if out.device != acc.device:
            raise RuntimeError("out must live on acc's device")
    elif not out.is_pinned():
        raise RuntimeError("a CPU destination must be page-locked (pin_memory)")
    rf = None
    if row_factor is not None:
        rf = torch.as_tensor(row_factor).reshape(-1).to(device=acc.device, dtype=torch.float32).contiguous()
        if rf.numel() != N:
            raise RuntimeError("row_factor must have N elements")
    lib = _lib.load()
    with torch.cuda.device(acc.device):
        stream = torch.cuda.current_stream(acc.device).cuda_stream
        code = lib.trakhip_scores_finalize(
            ctypes.c_void_p(acc.data_ptr()),
            _ld(acc),
            N,
            M,
            float(divisor),
            ctypes.c_void_p(rf.data_ptr()) if rf is not None else None,
            _STORE_DTYPES[out.dtype],
            ctypes.c_void_p(out.data_ptr()),
            _ld(out),
            ctypes.c_void_p(stream),
        )
    _lib.check(code)
    return out


def output_fits_on_device(n_rows, n_cols, device, reserve=0.25):
    """Whether an fp32 [n_rows, n_cols] result can be held on `device` next to what is there, keeping
    `reserve` of the free memory for operands in their product format."""
    free, _ = torch.cuda.mem_get_info(device)
    return n_rows * n_cols * 4 <= free * (1.0 - reserve)


def _block_extents(total, size):
    return [(lo, min(lo + size, total)) for lo in range(0, total, size)]


def get_matrix_mult_blockwise(features, target_grads, target_dtype=None, bs=8096, out=None, accumulate=False,
                              product=None, block_bytes=1 << 30):
    """features @ target_grads.T computed block by block on the GPU and collected on the host, for
    results that do not fit in device memory (trak/utils.py:135-245).  Operands may live on the host
    or on the device; the result is a CPU tensor (`out`, when given: written, or added to with
    `accumulate`).  Two device blocks and two page-locked host blocks: while block i is copied out and
    stored by the host, block i + 1 is being multiplied.  `bs` is the least block edge (the reference's
    meaning); blocks are grown to about `block_bytes` of fp32 results, since there is no small device
    memory to fit here.  `product(a, b, out)` overrides the product used for a block."""
    if target_dtype is None:
        target_dtype = features.dtype
    if product is None:
        product = lambda a, b, o: matmul_nt(a, b, out=o)  # noqa: E731
    N, M = features.shape[0], target_grads.shape[0]
    if features.is_cuda:
        dev = features.device
    elif target_grads.is_cuda:
        dev = target_grads.device
    else:
        dev = torch.device("cuda", torch.cuda.current_device())
    final = out if out is not None else torch.empty((N, M), dtype=target_dtype, device="cpu")
    if final.device.type != "cpu" or tuple(final.shape) != (N, M):
        raise RuntimeError("out must be a CPU tensor of shape [features rows, target rows]")
    if N == 0 or M == 0:
        return final
    bs, elements = max(int(bs), 1), max(int(block_bytes) // 4, 1)
    cb = min(M, max(bs, elements // bs))
    rb = min(N, max(bs, elements // cb))
    row_blocks, col_blocks = _block_extents(N, rb), _block_extents(M, cb)
    with torch.cuda.device(dev):
        main = torch.cuda.current_stream(dev)
        copy_stream = torch.cuda.Stream(device=dev)
        dbuf = [torch.empty((rb, cb), dtype=torch.float32, device=dev) for _ in range(2)]
        pbuf = [torch.empty((rb, cb), dtype=final.dtype, pin_memory=True) for _ in range(2)]
        computed = [torch.cuda.Event() for _ in range(2)]
        copied = [None, None]
        targets_on_device = {}
        pending = None  # (event, pinned view, destination view) of the block before

        def consume(p):
            event, src, dst = p
            event.synchronize()
            if accumulate:
                dst += src
            else:
                dst.copy_(src)

        idx = 0
        for r0, r1 in row_blocks:
            f = features[r0:r1].to(dev, non_blocking=True)
            for c0, c1 in col_blocks:
                if len(col_blocks) == 1:
                    t = targets_on_device.setdefault(0, target_grads.to(dev, non_blocking=True))
                else:
                    t = target_grads[c0:c1].to(dev, non_blocking=True)
                slot = idx % 2
                if copied[slot] is not None:
                    main.wait_event(copied[slot])  # the copy that read this device block two blocks ago
                d = dbuf[slot][: r1 - r0, : c1 - c0]
                product(f, t, d)
                converted = d if final.dtype == torch.float32 else d.to(final.dtype)
                computed[slot].record(main)
                # (the host finished with pinned block `slot` when it stored block idx - 2, one iteration ago)
                with torch.cuda.stream(copy_stream):
                    copy_stream.wait_event(computed[slot])
                    p = pbuf[slot][: r1 - r0, : c1 - c0]
                    p.copy_(converted, non_blocking=True)
                    converted.record_stream(copy_stream)
                    ev = torch.cuda.Event()
                    ev.record(copy_stream)
                    copied[slot] = ev
                if pending is not None:
                    consume(pending)  # overlaps with the product and the copy just queued
                pending = (ev, p, final[r0:r1, c0:c1])
                idx += 1
        consume(pending)
    return final


def get_matrix_mult(features, target_grads, target_dtype=None, batch_size=8096, use_blockwise=False):
    """features @ target_grads.T (trak/utils.py:248-294).  On the GPU this is one GEMM of fp32 accuracy
    on the matrix cores (see `matmul_nt`); CPU inputs take torch's matmul as in the reference
    (trak/utils.py:128-132).  A result that does not fit in device memory, or `use_blockwise`, goes
    block by block to the host (`get_matrix_mult_blockwise`; a CPU tensor comes back, as in the
    reference)."""
    if target_dtype is None:
        target_dtype = features.dtype
    if use_blockwise:
        return get_matrix_mult_blockwise(features, target_grads, target_dtype, batch_size)
    if features.device.type == "cpu":
        return (features @ target_grads.t()).clone().to(target_dtype)
    if not output_fits_on_device(features.shape[0], target_grads.shape[0], features.device):
        return get_matrix_mult_blockwise(features, target_grads, target_dtype, batch_size)
    out = matmul_nt(features, target_grads.to(features.device))
    return out.to(target_dtype)
