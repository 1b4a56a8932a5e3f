"""No-GPU checks of libtrakhip.so: it loads, exports every symbol the public header declares,
validates arguments before touching the device, and its host-side matrix materializer agrees
with the oracle bit for bit."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import jl_oracle as npo
from trak_amd import _lib, fast_jl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "trakhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(trakhip_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 9
    for name in names:
        assert getattr(lib, name) is not None, name


def test_abi_version_and_strerror():
    lib = _lib.load()
    assert lib.trakhip_abi_version() == 1
    assert _lib.strerror(0) == "success"
    # the text the reference throws at fast_jl/fast_jl_kernel.cuh:113-115
    assert _lib.strerror(-1) == "Invalid Number of JL dimensions it has to be a multiple of 512"
    for code in range(-13, 0):
        assert "unknown trakhip error" not in _lib.strerror(code)
    assert "unknown trakhip error" in _lib.strerror(-999)


def test_project_argument_validation_needs_no_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)  # never dereferenced: every call below fails validation first
    call = lambda **kw: lib.trakhip_project(
        kw.get("inp", p), kw.get("dtype", 0), kw.get("B", 8), kw.get("P", 1000), kw.get("ld", 1000),
        kw.get("out", p), kw.get("ws", p), kw.get("wsb", 1 << 40), kw.get("k", 512), 0, kw.get("tiles", 256),
        kw.get("pt", 0), None)
    assert call(k=100) == -1 and call(k=0) == -1 and call(k=768) == -1
    assert call(B=0) == -2 and call(P=0) == -2 and call(P=2**32) == -2 and call(ld=999) == -2 and call(tiles=0) == -2
    assert call(dtype=3) == -3 and call(dtype=-1) == -3
    assert call(pt=2) == -4
    assert call(inp=None) == -5 and call(out=None) == -5 and call(ws=None) == -5
    assert call(wsb=16) == -6
    assert call(inp=ctypes.c_void_p(4097)) == -7 and call(out=ctypes.c_void_p(4100)) == -7
    with pytest.raises(ValueError, match="multiple of 512"):
        _lib.check(-1)
    with pytest.raises(RuntimeError):
        _lib.check(-2)


def test_static_entry_point_validates_before_touching_the_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    call = lambda **kw: lib.trakhip_project_static(
        kw.get("inp", p), kw.get("dtype", 0), kw.get("B", 32), kw.get("P", 1024), kw.get("ld", 1024),
        kw.get("out", p), kw.get("k", 512), 0, kw.get("tiles", 2), kw.get("pt", 0), None)
    assert lib.trakhip_project_static_limit() == 36 << 20
    assert call(k=100) == -1 and call(B=0) == -2 and call(dtype=5) == -3 and call(pt=9) == -4
    assert call(inp=None) == -5 and call(out=None) == -5 and call(out=ctypes.c_void_p(4100)) == -7
    # 300 column blocks are more than the 256 CUs: one run, 37.5 MiB of partial sums, more than the 36 MiB array
    assert lib.trakhip_project_workspace(32, 1024, 307_200, 2) == 32 * 307_200 * 4
    assert call(k=307_200) == -12
    assert lib.trakhip_project_workspace_min(64, 1024, 262_144, 2) == 32 << 20  # the largest below that
    assert "static" in _lib.strerror(-12)


def test_workspace_size():
    lib = _lib.load()
    # G * min(B, 64) * k floats, G = runs of consecutive feature chunks = floor(256 CUs / column blocks),
    # at most one per chunk (no device in this process: the library assumes the 256 CUs of an MI355X)
    assert lib.trakhip_project_workspace(32, 11_689_512, 4096, 256) == 64 * 32 * 4096 * 4
    assert lib.trakhip_project_workspace(48, 1000, 512, 256) == 256 * 48 * 512 * 4      # 256 tiles x 1 chunk
    assert lib.trakhip_project_workspace_min(48, 1000, 512, 256) == 256 * 32 * 512 * 4
    assert lib.trakhip_project_workspace(200, 1000, 512, 256) == 256 * 64 * 512 * 4
    assert lib.trakhip_project_workspace_min(8, 25, 1024, 256) == 25 * 8 * 1024 * 4
    F16, BF16, F32 = _lib.F16, _lib.BF16, _lib.F32
    rpp = lib.trakhip_project_rows_per_pass
    assert rpp(F16, _lib.RADEMACHER) == 64 and rpp(BF16, _lib.RADEMACHER) == 64 and rpp(F32, _lib.RADEMACHER) == 32
    assert rpp(F16, _lib.NORMAL) == 64 and rpp(BF16, _lib.NORMAL) == 64 and rpp(F32, _lib.NORMAL) == 32
    assert lib.trakhip_project_workspace(8, 25, 1024, 256) == 25 * 8 * 1024 * 4
    assert lib.trakhip_project_workspace(16, 1_048_576, 512, 256) == 256 * 16 * 512 * 4  # one 512-column block
    assert lib.trakhip_project_workspace(0, 25, 1024, 256) == 0
    # column-block counts that do not divide 256: never more workgroups than CUs
    for k, blocks in ((1536, 2), (2560, 5), (3072, 3), (4608, 6), (5120, 5), (15_360, 15), (40_960, 40)):  # 768-, 512-, 1024-column blocks
        groups = 256 // blocks
        assert lib.trakhip_project_workspace(32, 11_689_512, k, 256) == groups * 32 * k * 4, k
    assert lib.trakhip_spd_inverse_workspace(4096) >= 3 * 4096 * 4096 * 4
    assert lib.trakhip_spd_inverse_workspace(100) >= 3 * 128 * 128 * 4


@pytest.mark.parametrize("proj_type,name", [(npo.RADEMACHER, "rademacher"), (npo.NORMAL, "normal")])
@pytest.mark.parametrize(
    "seed,tiles,P,f0,nf,c0,nc",
    [(0, 256, 1000, 0, 1000, 0, 8), (42, 256, 1_048_576, 4090, 300, 500, 12), (7, 108, 10_241, 9_900, 341, 2040, 8),
     (2**32 - 1, 256, 25, 0, 25, 0, 16), (7 + 10_000 * 3, 256, 11_689_512, 11_689_000, 512, 4064, 32)],
)
def test_host_materialize_equals_oracle(c_oracle, proj_type, name, seed, tiles, P, f0, nf, c0, nc):
    got = fast_jl.materialize(seed, tiles, P, f0, nf, c0, nc, name).numpy()
    want = c_oracle.materialize(seed, tiles, P, f0, nf, c0, nc, proj_type)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_materialize_argument_validation():
    lib = _lib.load()
    buf = (ctypes.c_float * 16)()
    assert lib.trakhip_materialize(0, 256, 100, 90, 20, 0, 1, 0, buf, 0, None) == -2   # f0 + nf > P
    assert lib.trakhip_materialize(0, 256, 100, 0, 4, 0, 4, 5, buf, 0, None) == -4
    assert lib.trakhip_materialize(0, 256, 100, 0, 4, 0, 4, 0, None, 0, None) == -5
    assert lib.trakhip_materialize(0, 256, 100, 0, 0, 0, 4, 0, None, 0, None) == 0      # empty block


def test_gemm_argument_validation_needs_no_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    assert lib.trakhip_gemm_nt(p, 8, p, 8, p, 4, 4, 4, 16, 1.0, 0.0, None, None) == -2   # lda < K
    assert lib.trakhip_gemm_nt(None, 16, p, 16, p, 4, 4, 4, 16, 1.0, 0.0, None, None) == -5
    assert lib.trakhip_gemm_nt(p, 16, p, 16, p, 4, 0, 4, 16, 1.0, 0.0, None, None) == 0  # empty
    assert lib.trakhip_gemm_tn(p, 2, p, 8, p, 8, 4, 4, 16, 1.0, 0.0, None) == -2          # lda < M
    assert lib.trakhip_spd_inverse(p, 2, 0.0, p, 4, 4, 0, None, None, p, 1 << 30, None) == -2
    assert lib.trakhip_spd_inverse(p, 4, 0.0, p, 4, 4, 0, None, None, p, 16, None) == -6
    # the general (pivoted) inverse: same argument checks; an augmented matrix [A | I] as workspace; n <= 12288
    assert lib.trakhip_general_inverse_workspace(4096) >= 2 * 4096 * 4096 * 4
    assert lib.trakhip_general_inverse_workspace(100) >= 2 * 128 * 128 * 4
    assert lib.trakhip_general_inverse_workspace(0) == 0 and lib.trakhip_general_inverse_workspace(12_289) == 0
    assert lib.trakhip_general_inverse(p, 2, 0.0, p, 4, 4, 0, None, None, p, 1 << 30, None) == -2
    assert lib.trakhip_general_inverse(p, 4, 0.0, p, 4, 4, 0, None, None, p, 16, None) == -6
    assert lib.trakhip_general_inverse(None, 4, 0.0, p, 4, 4, 0, None, None, p, 1 << 30, None) == -5
    assert lib.trakhip_general_inverse(p, 20_000, 0.0, p, 20_000, 20_000, 0, None, None, p, 1 << 40, None) == -2
    assert lib.trakhip_general_inverse(p, 4, 0.0, p, 4, 0, 0, None, None, p, 0, None) == 0      # empty matrix


def test_store_entry_points_validate_before_touching_the_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    red = lambda **kw: lib.trakhip_project_reduce_store(
        kw.get("ws", p), kw.get("B", 8), kw.get("P", 1000), kw.get("k", 512), kw.get("tiles", 256), 1.0,
        kw.get("dt", 0), kw.get("out", p), kw.get("ld", 512), None)
    assert red(k=100) == -1
    assert red(B=0) == -2 and red(B=65) == -2 and red(ld=508) == -2 and red(P=0) == -2
    assert red(dt=3) == -3
    assert red(ws=None) == -5 and red(out=None) == -5
    assert red(out=ctypes.c_void_p(4100)) == -7 and red(ld=514) == -7
    assert red(dt=2, out=ctypes.c_void_p(4104)) == -7
    # a pointer HIP knows nothing about (pageable host memory, here an arbitrary address) is
    # refused on the host instead of faulting the GPU
    assert red() == -11
    fin = lambda **kw: lib.trakhip_scores_finalize(
        kw.get("acc", p), kw.get("lda", 8), kw.get("N", 4), kw.get("M", 8), kw.get("div", 2.0), None,
        kw.get("dt", 2), kw.get("out", p), kw.get("ldo", 8), None)
    assert fin(dt=5) == -3
    assert fin(lda=7) == -2 and fin(ldo=7) == -2 and fin(div=0.0) == -2
    assert fin(N=0) == 0 and fin(M=0, lda=0, ldo=0) == 0
    assert fin(acc=None) == -5 and fin(out=None) == -5
    assert fin(acc=ctypes.c_void_p(4098)) == -7 and fin(dt=0, out=ctypes.c_void_p(4097)) == -7
    assert fin() == -11
    assert "page-locked" in _lib.strerror(-11)


def test_split2_entry_points_validate_before_touching_the_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    # two fp16 planes x octets padded to 8 x rows padded to 256 x 16 bytes
    assert lib.trakhip_split2_bytes(1, 1) == 2 * 8 * 256 * 16
    assert lib.trakhip_split2_bytes(50_000, 4096) == 2 * 512 * 50_176 * 16
    assert lib.trakhip_split2_bytes(0, 5) == 0 and lib.trakhip_split2_bytes(5, 0) == 0
    sp = lambda **kw: lib.trakhip_split2_rows(
        kw.get("src", p), kw.get("ld", 64), kw.get("rows", 10), kw.get("K", 64), kw.get("tr", 0), kw.get("out", p),
        kw.get("bytes", 1 << 30), kw.get("scales", p), None)
    assert sp(rows=0) == -2 and sp(K=0) == -2 and sp(ld=63) == -2 and sp(tr=1, ld=9) == -2
    assert sp(src=None) == -5 and sp(out=None) == -5 and sp(scales=None) == -5
    assert sp(bytes=100) == -6
    assert sp(src=ctypes.c_void_p(4098)) == -7 and sp(out=ctypes.c_void_p(4104)) == -7
    assert sp(scales=ctypes.c_void_p(4097)) == -7
    mm = lambda **kw: lib.trakhip_gemm_nt_split2(
        kw.get("a", p), kw.get("sa", p), kw.get("M", 8), kw.get("b", p), kw.get("sb", p), kw.get("N", 8),
        kw.get("K", 16), kw.get("c", p), kw.get("ldc", 8), 1.0, 0.0, None, None)
    assert mm(sa=None) == -5 and mm(sb=None) == -5
    assert mm(M=0) == 0 and mm(N=0) == 0
    assert mm(K=0) == -2 and mm(ldc=7) == -2
    assert mm(a=None) == -5 and mm(b=None) == -5 and mm(c=None) == -5
    assert mm(a=ctypes.c_void_p(4104)) == -7 and mm(c=ctypes.c_void_p(4098)) == -7
    gr = lambda **kw: lib.trakhip_gram_split2(kw.get("a", p), kw.get("sa", p), kw.get("N", 8), kw.get("K", 16),
                                              kw.get("c", p), kw.get("ldc", 8), 1.0, 0.0, kw.get("ws", None),
                                              kw.get("wsb", 0), None)
    assert gr(N=0) == 0 and gr(sa=None) == -5 and gr(a=None) == -5 and gr(ldc=7) == -2
    # with a workspace the k range is shared out when there is enough of it: same validation
    assert gr(K=4096, N=300, ws=p, wsb=1 << 30, ldc=299) == -2 and gr(K=4096, N=300, ws=p, wsb=1 << 30, c=None) == -5


def test_gemm_nt16_validates_before_touching_the_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    F16, BF16, F32 = _lib.F16, _lib.BF16, _lib.F32
    mm = lambda **kw: lib.trakhip_gemm_nt16(
        kw.get("a", p), kw.get("lda", 64), kw.get("b", p), kw.get("ldb", 64), kw.get("dt", F16), kw.get("c", p),
        kw.get("ldc", 8), kw.get("M", 8), kw.get("N", 8), kw.get("K", 64), 1.0, 0.0, None, None)
    assert mm(dt=F32) == -3 and mm(dt=5) == -3
    assert mm(M=0) == 0 and mm(N=0, dt=BF16) == 0
    assert mm(K=0) == -2 and mm(K=32) == -2 and mm(K=100, lda=104, ldb=104) == -2     # K % 64
    assert mm(lda=56) == -2 and mm(ldb=63) == -2 and mm(ldc=7) == -2
    assert mm(lda=1 << 23) == -2 and mm(ldb=1 << 23) == -2     # a lane's offset inside a tile stays in 32 bits
    assert mm(a=None) == -5 and mm(b=None) == -5 and mm(c=None) == -5
    assert mm(a=ctypes.c_void_p(4104)) == -7 and mm(b=ctypes.c_void_p(4098)) == -7     # 16-byte rows
    assert mm(lda=68) == -7 and mm(ldb=100) == -7 and mm(c=ctypes.c_void_p(4098)) == -7


def test_split_gemm_entry_points_validate_before_touching_the_device():
    lib = _lib.load()
    p = ctypes.c_void_p(4096)
    F16, BF16, F32 = _lib.F16, _lib.BF16, _lib.F32
    # planes (3 for fp32, 1 for 16-bit types) x octets padded to 8 x rows padded to 256 x 16 bytes
    assert lib.trakhip_split_bytes(1, 1, F32) == 3 * 8 * 256 * 16
    assert lib.trakhip_split_bytes(50_000, 4096, F32) == 3 * 512 * 50_176 * 16
    assert lib.trakhip_split_bytes(50_000, 4096, F16) == 512 * 50_176 * 16
    assert lib.trakhip_split_bytes(257, 65, BF16) == 16 * 512 * 16
    assert lib.trakhip_split_bytes(0, 5, F32) == 0 and lib.trakhip_split_bytes(5, 5, 7) == 0
    sp = lambda **kw: lib.trakhip_split_rows(
        kw.get("src", p), kw.get("dt", F32), kw.get("ld", 64), kw.get("rows", 10), kw.get("K", 64), kw.get("tr", 0),
        kw.get("out", p), kw.get("bytes", 1 << 30), None)
    assert sp(dt=9) == -3
    assert sp(rows=0) == -2 and sp(K=0) == -2 and sp(ld=63) == -2 and sp(tr=1, ld=9) == -2
    assert sp(src=None) == -5 and sp(out=None) == -5
    assert sp(bytes=100) == -6
    assert sp(src=ctypes.c_void_p(4098)) == -7 and sp(out=ctypes.c_void_p(4104)) == -7
    assert sp(dt=F16, src=ctypes.c_void_p(4097)) == -7
    mm = lambda **kw: lib.trakhip_gemm_nt_split(
        kw.get("a", p), kw.get("M", 8), kw.get("b", p), kw.get("N", 8), kw.get("K", 16), kw.get("dt", F32),
        kw.get("c", p), kw.get("ldc", 8), 1.0, 0.0, None, None)
    assert mm(dt=-1) == -3
    assert mm(M=0) == 0 and mm(N=0) == 0
    assert mm(K=0) == -2 and mm(ldc=7) == -2
    assert mm(a=None) == -5 and mm(b=None) == -5 and mm(c=None) == -5
    assert mm(a=ctypes.c_void_p(4104)) == -7 and mm(c=ctypes.c_void_p(4098)) == -7
    gr = lambda **kw: lib.trakhip_gram_split(kw.get("a", p), kw.get("N", 8), kw.get("K", 16), kw.get("dt", F32),
                                             kw.get("c", p), kw.get("ldc", 8), 1.0, 0.0, kw.get("ws", None),
                                             kw.get("wsb", 0), None)
    assert gr(N=0) == 0 and gr(dt=5) == -3 and gr(ldc=7) == -2 and gr(a=None) == -5
    # scratch for sharing the k range of a product with few tiles: three N x N fp32 matrices, or none
    ws = lib.trakhip_gram_split_workspace
    assert ws(4096, 50_000, F32, 0) == 3 * 4096 * 4096 * 4 and ws(4096, 50_000, F16, 0) == 3 * 4096 * 4096 * 4
    assert ws(4096, 50_000, F32, 1) == 3 * 4096 * 4096 * 4
    assert ws(8192, 50_000, F32, 0) == 0            # 528 lower tiles keep every CU busy as they are
    assert ws(4096, 256, F32, 0) == 0 and ws(4096, 1024, F16, 0) == 0      # too few k steps to share out
    assert ws(0, 5, F32, 0) == 0 and ws(5, 0, F32, 0) == 0 and ws(5, 5, 9, 0) == 0
    assert gr(K=4096, N=300, ws=p, wsb=1 << 30, ldc=299) == -2 and gr(K=4096, N=300, ws=p, wsb=1 << 30, c=None) == -5
