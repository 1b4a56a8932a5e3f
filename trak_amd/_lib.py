"""ctypes binding of libtrakhip.so (the C ABI declared in include/trakhip.h)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtrakhip.so")

F16, BF16, F32 = 0, 1, 2
RADEMACHER, NORMAL = 0, 1

ERR_PROJ_DIM = -1

_lib = None


class TrakHipError(RuntimeError):
    """Error reported by libtrakhip (a RuntimeError, like the reference's AT_ASSERTM failures)."""

    def __init__(self, code, text):
        super().__init__(f"trakhip error {code}: {text}")
        self.code = code


def load():
    """Loads the library once.  There is no fallback: a missing build is an ImportError."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m trak_amd.build` "
            "(hipcc --offload-arch=gfx950); there is no CPU fallback"
        )
    lib = ctypes.CDLL(LIB_PATH)
    u32, u64, i32, sz = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int, ctypes.c_size_t
    vp, f32 = ctypes.c_void_p, ctypes.c_float
    lib.trakhip_strerror.argtypes = [i32]
    lib.trakhip_strerror.restype = ctypes.c_char_p
    lib.trakhip_abi_version.argtypes = []
    lib.trakhip_abi_version.restype = i32
    lib.trakhip_project_workspace.argtypes = [u64, u64, u32, u32]
    lib.trakhip_project_workspace.restype = sz
    lib.trakhip_project_workspace_min.argtypes = [u64, u64, u32, u32]
    lib.trakhip_project_workspace_min.restype = sz
    lib.trakhip_project_rows_per_pass.argtypes = [i32, i32]
    lib.trakhip_project_rows_per_pass.restype = u32
    lib.trakhip_project.argtypes = [vp, i32, u64, u64, u64, vp, vp, sz, u32, u32, u32, i32, vp]
    lib.trakhip_project.restype = i32
    lib.trakhip_project_static_limit.argtypes = []
    lib.trakhip_project_static_limit.restype = sz
    lib.trakhip_project_static.argtypes = [vp, i32, u64, u64, u64, vp, u32, u32, u32, i32, vp]
    lib.trakhip_project_static.restype = i32
    lib.trakhip_project_partials.argtypes = [vp, i32, u64, u64, u64, vp, sz, u32, u32, u32, i32, vp]
    lib.trakhip_project_partials.restype = i32
    lib.trakhip_project_gather_partials.argtypes = [vp, u32, i32, u64, u64, vp, sz, u32, u32, u32, i32, vp]
    lib.trakhip_project_gather_partials.restype = i32
    lib.trakhip_project_reduce.argtypes = [vp, u64, u64, u32, u32, f32, vp, vp]
    lib.trakhip_project_reduce.restype = i32
    lib.trakhip_project_reduce_store.argtypes = [vp, u64, u64, u32, u32, f32, i32, vp, u64, vp]
    lib.trakhip_project_reduce_store.restype = i32
    lib.trakhip_scores_finalize.argtypes = [vp, u64, u64, u64, f32, vp, i32, vp, u64, vp]
    lib.trakhip_scores_finalize.restype = i32
    lib.trakhip_materialize.argtypes = [u32, u32, u64, u64, u64, u32, u32, i32, vp, i32, vp]
    lib.trakhip_materialize.restype = i32
    lib.trakhip_gemm_nt.argtypes = [vp, u64, vp, u64, vp, u64, u64, u64, u64, f32, f32, vp, vp]
    lib.trakhip_gemm_nt.restype = i32
    lib.trakhip_gemm_tn.argtypes = [vp, u64, vp, u64, vp, u64, u64, u64, u64, f32, f32, vp]
    lib.trakhip_gemm_tn.restype = i32
    lib.trakhip_split_bytes.argtypes = [u64, u64, i32]
    lib.trakhip_split_bytes.restype = sz
    lib.trakhip_split_rows.argtypes = [vp, i32, u64, u64, u64, i32, vp, sz, vp]
    lib.trakhip_split_rows.restype = i32
    lib.trakhip_gemm_nt_split.argtypes = [vp, u64, vp, u64, u64, i32, vp, u64, f32, f32, vp, vp]
    lib.trakhip_gemm_nt_split.restype = i32
    lib.trakhip_gram_split_workspace.argtypes = [u64, u64, i32, i32]
    lib.trakhip_gram_split_workspace.restype = sz
    lib.trakhip_gram_split.argtypes = [vp, u64, u64, i32, vp, u64, f32, f32, vp, sz, vp]
    lib.trakhip_gram_split.restype = i32
    lib.trakhip_split2_bytes.argtypes = [u64, u64]
    lib.trakhip_split2_bytes.restype = sz
    lib.trakhip_split2_rows.argtypes = [vp, u64, u64, u64, i32, vp, sz, vp, vp]
    lib.trakhip_split2_rows.restype = i32
    lib.trakhip_gemm_nt_split2.argtypes = [vp, vp, u64, vp, vp, u64, u64, vp, u64, f32, f32, vp, vp]
    lib.trakhip_gemm_nt_split2.restype = i32
    lib.trakhip_gram_split2.argtypes = [vp, vp, u64, u64, vp, u64, f32, f32, vp, sz, vp]
    lib.trakhip_gram_split2.restype = i32
    lib.trakhip_gemm_nt16.argtypes = [vp, u64, vp, u64, i32, vp, u64, u64, u64, u64, f32, f32, vp, vp]
    lib.trakhip_gemm_nt16.restype = i32
    lib.trakhip_spd_inverse_workspace.argtypes = [u64]
    lib.trakhip_spd_inverse_workspace.restype = sz
    lib.trakhip_spd_inverse.argtypes = [vp, u64, f32, vp, u64, u64, i32, vp, vp, vp, sz, vp]
    lib.trakhip_spd_inverse.restype = i32
    lib.trakhip_general_inverse_workspace.argtypes = [u64]
    lib.trakhip_general_inverse_workspace.restype = sz
    lib.trakhip_general_inverse.argtypes = [vp, u64, f32, vp, u64, u64, i32, vp, vp, vp, sz, vp]
    lib.trakhip_general_inverse.restype = i32
    _lib = lib
    return lib


def strerror(code):
    return load().trakhip_strerror(code).decode()


def check(code):
    """0 passes; the proj-dim error becomes ValueError (std::invalid_argument in the reference,
    fast_jl/fast_jl_kernel.cuh:113-115); everything else a RuntimeError."""
    if code == 0:
        return
    text = strerror(code)
    if code == ERR_PROJ_DIM:
        raise ValueError(text)
    raise TrakHipError(code, text)
