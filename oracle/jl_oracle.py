"""TEST INFRASTRUCTURE ONLY -- numpy oracle for the JL projection matrix, plus the loader of
the C oracle (oracle/jl_oracle.c).

This is a second, independent statement of the random stream (vectorized numpy, written
from the specification, not from the C oracle or the library's header).  Only tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py may import it.

Restated reference behaviour (MadryLab/trak):
  * stream_name   -- fast_jl/random.cuh:15-17: the 32-bit value that names the random stream of
    a (JL column, feature tile) pair (the reference seeds the pair's generator with it); block n
    of the stream named s is Philox(counter = (n, s, 0, 0), key = (seed, 0))
  * tiling        -- fast_jl/fast_jl.cu:42, fast_jl/fast_jl_kernel.cuh:124
  * Rademacher: one random bit per entry, bit set -> +1 -- fast_jl/random.cuh:33-37
  * Normal: Box-Muller normal in fp16 (fp16 radius times fp16 cos/sin, rounded once)
    -- fast_jl/random.cuh:50-60
The generator is Philox4x32-10 (Random123), pinned by Random123's known-answer vectors in
tests/test_oracle_philox.py; the position -> (block, bit) map is this build's definition and
is pinned by agreement of this file with oracle/jl_oracle.c and by the property tests.
"""
import ctypes
import os
import subprocess

import numpy as np

RADEMACHER = 0
NORMAL = 1

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = 0x9E3779B9
_W1 = 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(ctr, key):
    """ctr: (..., 4) uint32, key: (..., 2) uint32 -> (..., 4) uint32."""
    ctr = np.asarray(ctr, dtype=np.uint32)
    key = np.asarray(key, dtype=np.uint32)
    c = [ctr[..., i].astype(np.uint64) for i in range(4)]
    k0 = key[..., 0].astype(np.uint64)
    k1 = key[..., 1].astype(np.uint64)
    for r in range(10):
        kk0 = (k0 + np.uint64((_W0 * r) & 0xFFFFFFFF)) & _MASK
        kk1 = (k1 + np.uint64((_W1 * r) & 0xFFFFFFFF)) & _MASK
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        c = [
            (p1 >> np.uint64(32)) ^ c[1] ^ kk0,
            p1 & _MASK,
            (p0 >> np.uint64(32)) ^ c[3] ^ kk1,
            p0 & _MASK,
        ]
    return np.stack(c, axis=-1).astype(np.uint32)


def stream_name(seed, column, tile):
    v = (
        np.uint64(seed)
        + np.uint64(658105236) * np.asarray(column, dtype=np.uint64)
        + np.uint64(359124577) * np.asarray(tile, dtype=np.uint64)
    )
    return (v & _MASK).astype(np.uint32)


def stream_blocks(seed, name, block):
    """Blocks of the streams named `name`, broadcast over the arguments -> (..., 4) uint32."""
    name, block = np.broadcast_arrays(np.asarray(name, dtype=np.uint32), np.asarray(block, dtype=np.uint32))
    ctr = np.stack([block, name, np.zeros_like(block), np.zeros_like(block)], axis=-1)
    key = np.zeros(block.shape + (2,), dtype=np.uint32)
    key[..., 0] = np.uint32(seed & 0xFFFFFFFF)
    return philox4x32_10(ctr, key)


def tiling(P, num_feature_tiles):
    tiles = min(int(P), int(num_feature_tiles))
    tile_size = -(-int(P) // tiles)
    return tiles, tile_size


# ---- exact binary32 fma on numpy arrays -----------------------------------------------------


def _fma32(a, b, c):
    """Correctly rounded float32 fma(a, b, c) for float32 arrays.

    a*b is exact in float64 (24+24 bits).  p + c is computed in float64 with its rounding
    error (TwoSum); if the float64 sum lands exactly half way between two float32 values the
    error term decides the direction, which removes the double-rounding hazard."""
    shape = np.broadcast(np.asarray(a), np.asarray(b), np.asarray(c)).shape
    a = np.atleast_1d(np.asarray(a, dtype=np.float32)).astype(np.float64)
    b = np.atleast_1d(np.asarray(b, dtype=np.float32)).astype(np.float64)
    c = np.atleast_1d(np.asarray(c, dtype=np.float32)).astype(np.float64)
    a, b, c = np.broadcast_arrays(a, b, c)
    p = a * b
    s = p + c
    bb = s - p
    err = (p - (s - bb)) + (c - bb)
    r = s.astype(np.float32)
    low = np.ascontiguousarray(s).view(np.uint64) & np.uint64((1 << 29) - 1)
    tie = (low == np.uint64(1 << 28)) & (err != 0.0) & np.isfinite(s) & (s != 0.0)
    if tie.any():
        # the true value is s + err: it lies strictly on one side of the midpoint
        lo = np.nextafter(s[tie], -np.inf)
        hi = np.nextafter(s[tie], np.inf)
        r[tie] = np.where(err[tie] > 0, hi, lo).astype(np.float32)
    return r.reshape(shape)


def _f32(x):
    return np.asarray(x, dtype=np.float32)


def radius_f32(x):
    """sqrt(-2 ln u), u = (x + 1/2) / 2^14, for 14-bit indices x: the specified binary32
    operation sequence (log by exponent/mantissa split and a degree-9 polynomial, square root by
    three Newton steps on the reciprocal root)."""
    x = np.asarray(x, dtype=np.uint32)
    one = np.float32(1.0)
    odd = (x << np.uint32(1)) | np.uint32(1)
    xf = odd.astype(np.float32)  # exact, < 2^15
    xb = xf.view(np.uint32)
    expo = (xb >> np.uint32(23)).astype(np.int32) - 127
    mant = ((xb & np.uint32(0x7FFFFF)) | np.uint32(0x3F800000)).view(np.float32)
    big = mant > np.float32(1.41421354)
    mant = np.where(big, mant * np.float32(0.5), mant).astype(np.float32)
    expo = np.where(big, expo + 1, expo)
    t = (mant - one).astype(np.float32)
    z = (t * t).astype(np.float32)
    coef = [
        7.0376836292e-2,
        -1.1514610310e-1,
        1.1676998740e-1,
        -1.2420140846e-1,
        1.4249322787e-1,
        -1.6668057665e-1,
        2.0000714765e-1,
        -2.4999993993e-1,
        3.3333331174e-1,
    ]
    poly = np.full(t.shape, np.float32(coef[0]), dtype=np.float32)
    for cf in coef[1:]:
        poly = _fma32(poly, t, np.float32(cf))
    y = (t * (z * poly).astype(np.float32)).astype(np.float32)
    y = _fma32(np.float32(-0.5), z, y)
    ln_m = (t + y).astype(np.float32)
    ln_u = _fma32((expo - 15).astype(np.float32), np.float32(0.693147182), ln_m)
    s = (np.float32(-2.0) * ln_u).astype(np.float32)
    guess = (np.uint32(0x5F3759DF) - (s.view(np.uint32) >> np.uint32(1))).view(np.float32)
    half_s = (np.float32(0.5) * s).astype(np.float32)
    for _ in range(3):
        gg = (guess * guess).astype(np.float32)
        corr = _fma32(-half_s, gg, np.float32(1.5))
        guess = (guess * corr).astype(np.float32)
    return (s * guess).astype(np.float32)


def cos_sin_f32(a):
    """cos and sin of (a + 1/2) * 2 pi / 2^14 for 14-bit indices a, as binary32.  a // 4096 is the quadrant,
    a % 4096 the angle (a % 4096 + 1/2) * (pi/2) / 2^12 inside it: polynomials on (0, pi/4), the upper half of
    the quadrant as the mirror image (index 4095 - a % 4096, cos <-> sin), and the quadrant as an exact
    rotation by a multiple of pi/2."""
    a = np.asarray(a, dtype=np.uint32)
    one = np.float32(1.0)
    quadrant = (a >> np.uint32(12)) & np.uint32(3)
    aq = a & np.uint32(4095)
    mirror = aq >= np.uint32(2048)
    am = np.where(mirror, np.uint32(4095) - aq, aq).astype(np.uint32)
    yv = ((am.astype(np.float32) + np.float32(0.5)).astype(np.float32) * np.float32(3.83495208e-4)).astype(np.float32)
    y2 = (yv * yv).astype(np.float32)
    ps = _fma32(np.float32(-1.9515295891e-4), y2, np.float32(8.3321608736e-3))
    ps = _fma32(ps, y2, np.float32(-1.6666654611e-1))
    sn = _fma32((ps * y2).astype(np.float32), yv, yv)
    pc = _fma32(np.float32(2.443315711809948e-5), y2, np.float32(-1.388731625493765e-3))
    pc = _fma32(pc, y2, np.float32(4.166664568298827e-2))
    cs = _fma32((pc * y2).astype(np.float32), y2, _fma32(np.float32(-0.5), y2, one))
    c1 = np.where(mirror, sn, cs).astype(np.float32)
    s1 = np.where(mirror, cs, sn).astype(np.float32)
    # rotation by quadrant * pi/2: (c, s) -> (c, s), (-s, c), (-c, -s), (s, -c)
    c = np.choose(quadrant, [c1, -s1, -c1, s1]).astype(np.float32)
    sn_out = np.choose(quadrant, [s1, c1, -s1, -c1]).astype(np.float32)
    return c, sn_out


_TABLES = None


def normal_tables():
    """(R, C, S): the fp16 factor tables of the normal entries (round to nearest even of the
    binary32 sequences above), as float16 arrays of 2^14 entries each (C and S signed, around the circle)."""
    global _TABLES
    if _TABLES is None:
        r = radius_f32(np.arange(1 << 14, dtype=np.uint32)).astype(np.float16)
        c, s = cos_sin_f32(np.arange(1 << 14, dtype=np.uint32))
        _TABLES = (r, c.astype(np.float16), s.astype(np.float16))
    return _TABLES


def normal_from_word(w, sine):
    """fp16 normal entries (returned as float16) from random words w: radius index bits 17..30,
    angle index bits 2..15 (the tables C and S are signed; bits 0, 1, 16, 31 are not used).  The
    product of the two fp16 factors is exact in float64 and rounded once."""
    w = np.asarray(w, dtype=np.uint32)
    sine = np.asarray(sine, dtype=bool)
    R, C, S = normal_tables()
    x = ((w >> np.uint32(17)) & np.uint32(0x3FFF)).astype(np.int64)
    a = ((w >> np.uint32(2)) & np.uint32(0x3FFF)).astype(np.int64)
    trig = np.where(sine, S[a], C[a]).astype(np.float64)
    return (R[x].astype(np.float64) * trig).astype(np.float16)  # numpy rounds float64 -> float16 once, to nearest even


def materialize(seed, num_feature_tiles, P, f0, nf, c0, nc, proj_type):
    """S[f0:f0+nf, c0:c0+nc] as float32 (every value is exactly an fp16 value)."""
    tiles, tile_size = tiling(P, num_feature_tiles)
    f = np.arange(f0, f0 + nf, dtype=np.uint64)[:, None]
    c = np.arange(c0, c0 + nc, dtype=np.uint64)[None, :]
    tile = f // np.uint64(tile_size)
    off = (f - tile * np.uint64(tile_size)).astype(np.uint32)
    off = np.broadcast_to(off, (nf, nc))
    name = stream_name(seed, np.broadcast_to(c, (nf, nc)), np.broadcast_to(tile, (nf, nc)))
    if proj_type == RADEMACHER:
        # entry i of a 128-entry block is bit i of the block: word i // 32, bit i % 32
        w = stream_blocks(seed, name, off // np.uint32(128))
        i = off % np.uint32(128)
        word = np.take_along_axis(w, (i // np.uint32(32))[..., None].astype(np.int64), axis=-1)[..., 0]
        bit = (word >> (i % np.uint32(32))) & np.uint32(1)
        return np.where(bit == 1, np.float32(1.0), np.float32(-1.0)).astype(np.float32)
    w = stream_blocks(seed, name, off // np.uint32(8))
    e = off % np.uint32(8)
    word = np.take_along_axis(w, (e // np.uint32(2))[..., None].astype(np.int64), axis=-1)[..., 0]
    return normal_from_word(word, e % np.uint32(2) == 1).astype(np.float32)


def project_fp64(G, seed, num_feature_tiles, proj_dim_cols, proj_type, chunk=4096):
    """float64 contraction G[B, P] x S[:, cols] with S from this file (small shapes only)."""
    G = np.asarray(G)
    B, P = G.shape
    cols = np.asarray(proj_dim_cols)
    out = np.zeros((B, len(cols)), dtype=np.float64)
    c0, nc = int(cols[0]), len(cols)
    assert np.array_equal(cols, np.arange(c0, c0 + nc))
    for f0 in range(0, P, chunk):
        nf = min(chunk, P - f0)
        S = materialize(seed, num_feature_tiles, P, f0, nf, c0, nc, proj_type).astype(np.float64)
        out += G[:, f0 : f0 + nf].astype(np.float64) @ S
    return out


# ---- C oracle loader ---------------------------------------------------------------------------

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libjl_oracle.so")


def build_c_oracle(force=False):
    src = os.path.join(_HERE, "jl_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-s", "libjl_oracle.so"])
    return _SO


class COracle:
    """ctypes view of oracle/libjl_oracle.so."""

    def __init__(self):
        if not os.path.exists(_SO):
            build_c_oracle()
        lib = ctypes.CDLL(_SO)
        u32, u64, i32 = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int
        fp = ctypes.POINTER(ctypes.c_float)
        dp = ctypes.POINTER(ctypes.c_double)
        up = ctypes.POINTER(u32)
        lib.jlo_philox4x32_10.argtypes = [up, up, up]
        lib.jlo_philox4x32_10.restype = None
        lib.jlo_stream_name.argtypes = [u32, u32, u32]
        lib.jlo_stream_name.restype = u32
        lib.jlo_stream_block.argtypes = [u32, u32, u32, up]
        lib.jlo_stream_block.restype = None
        lib.jlo_tiling.argtypes = [u64, u32, up, ctypes.POINTER(u64)]
        lib.jlo_tiling.restype = None
        lib.jlo_entry.argtypes = [u32, u32, u64, u64, u32, i32]
        lib.jlo_entry.restype = ctypes.c_float
        lib.jlo_normal_from_word.argtypes = [u32, i32]
        lib.jlo_normal_from_word.restype = ctypes.c_float
        for name in ("jlo_radius_half", "jlo_cos_half", "jlo_sin_half"):
            getattr(lib, name).argtypes = [u32]
            getattr(lib, name).restype = ctypes.c_uint16
        lib.jlo_half_bits.argtypes = [ctypes.c_float]
        lib.jlo_half_bits.restype = ctypes.c_uint16
        lib.jlo_materialize.argtypes = [u32, u32, u64, u64, u64, u32, u32, i32, fp]
        lib.jlo_materialize.restype = None
        lib.jlo_project.argtypes = [fp, u64, u64, u64, u32, u32, u32, u32, i32, dp]
        lib.jlo_project.restype = None
        self.lib = lib

    def philox(self, ctr, key):
        c = (ctypes.c_uint32 * 4)(*[int(x) for x in ctr])
        k = (ctypes.c_uint32 * 2)(*[int(x) for x in key])
        o = (ctypes.c_uint32 * 4)()
        self.lib.jlo_philox4x32_10(c, k, o)
        return [int(x) for x in o]

    def stream_name(self, seed, column, tile):
        return int(self.lib.jlo_stream_name(seed, column, tile))

    def stream_block(self, seed, name, block):
        o = (ctypes.c_uint32 * 4)()
        self.lib.jlo_stream_block(seed, name, block, o)
        return [int(x) for x in o]

    def tiling(self, P, num_feature_tiles):
        t = ctypes.c_uint32()
        s = ctypes.c_uint64()
        self.lib.jlo_tiling(P, num_feature_tiles, ctypes.byref(t), ctypes.byref(s))
        return int(t.value), int(s.value)

    def entry(self, seed, tiles, P, f, c, proj_type):
        return float(self.lib.jlo_entry(seed, tiles, P, f, c, proj_type))

    def normal_from_word(self, w, sine):
        return float(self.lib.jlo_normal_from_word(int(w), int(sine)))

    def radius_half(self, x):
        return int(self.lib.jlo_radius_half(int(x)))

    def cos_half(self, a):
        return int(self.lib.jlo_cos_half(int(a)))

    def sin_half(self, a):
        return int(self.lib.jlo_sin_half(int(a)))

    def half_bits(self, v):
        return int(self.lib.jlo_half_bits(ctypes.c_float(v)))

    def materialize(self, seed, tiles, P, f0, nf, c0, nc, proj_type):
        out = np.empty((nf, nc), dtype=np.float32)
        self.lib.jlo_materialize(
            seed, tiles, P, f0, nf, c0, nc, proj_type, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
        )
        return out

    def project(self, G32, seed, tiles, c0, nc, proj_type):
        """G32: float32 [B, P] C-contiguous (exact image of the fp16/bf16/fp32 input)."""
        G32 = np.ascontiguousarray(G32, dtype=np.float32)
        B, P = G32.shape
        out = np.empty((B, nc), dtype=np.float64)
        self.lib.jlo_project(
            G32.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
            B,
            P,
            P,
            seed,
            tiles,
            c0,
            nc,
            proj_type,
            out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
        )
        return out
