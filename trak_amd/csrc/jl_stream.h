// Definition of the JL projection matrix S[f, c] as a counter-based random stream.
//
// Shared by the device kernels and the host-side materializer of this library.
// (The CPU oracle used by the tests is written separately and does not include
// this file.)
//
// What is kept from the reference kernel (fast_jl):
//   * the feature axis is cut into T = min(P, num_feature_tiles) tiles of
//     fts = ceil(P / T) features (fast_jl/fast_jl.cu:42, fast_jl/fast_jl_kernel.cuh:124);
//   * every (JL column c, feature tile t) pair owns one random stream, named by the 32-bit
//     value  seed + 658105236*c + 359124577*t  with uint32 wrap-around
//     (fast_jl/random.cuh:15-17, where it seeds the pair's generator);
//   * entries are consumed in feature order inside a tile; a Rademacher entry
//     costs one random bit, bit set -> +1 (fast_jl/random.cuh:33-37); a normal
//     entry is a Box-Muller normal in fp16 (fast_jl/random.cuh:50-60).
//
// What is new: the generator is Philox4x32-10 (the reference uses cuRAND XORWOW,
// whose draws cannot be reproduced off an NVIDIA toolchain).  The stream named s of a
// projector with seed `seed` is the block sequence
//       block(n) = Philox4x32-10(counter = (n, s, 0, 0), key = (seed, 0)).
// The stream's name sits in the counter and not in the key so that the ten round keys are the
// same for every lane of a kernel (scalar operands, no per-lane key schedule).
//
// Rademacher: feature offset o inside the tile uses block n = o / 128, and the entry is bit
//   o % 128 of the block read as a 128-bit little-endian number (bit j % 32 of word j / 32).
//   The 8 entries a lane feeds to one 32x32x16 MFMA (offsets 8q .. 8q + 7) are byte q of the
//   block: the kernel looks the eight signs up in a 256-entry table.
//
// Normal: feature offset o uses block n = o / 8; word (o % 8) / 2 of the block makes the
//   Box-Muller pair of entries o % 8 = 2i (cosine) and 2i + 1 (sine):
//       entry = fp16( R[x] * C[a] )   resp.   fp16( R[x] * S[a] )
//   with a 14-bit radius index x (bits 17..30 of the word) and a 14-bit angle index a (bits 2..15),
//       R[x] = fp16( sqrt(-2 ln((x + 1/2) / 2^14)) ),
//       C[a], S[a] = fp16( cos, sin of (a + 1/2) * 2 pi / 2^14 ),
//   i.e. a uniform angle on a grid of 2^14 directions around the whole circle (C and S carry their
//   signs) and a uniform u on a grid of 2^14 values.  The fields sit so that each table's byte address
//   is one instruction: (w >> 16) & 0x7FFE for the 2-byte entries of R (a 16-bit sub-word select and a
//   mask), w & 0xFFFC for the 4-byte pairs (C, S); with the quadrant in the table no sign is applied
//   afterwards.  R, C and S are spelled out below in IEEE binary32 operations (add, mul, fma,
//   int<->float conversions of exactly representable values) and rounded to fp16 (nearest even),
//   so any IEEE machine reproduces them bit for bit; the product of the two fp16 factors is
//   exact in binary32 and is rounded once.  The kernel keeps R and (C, S) as tables in LDS.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define JL_HD __host__ __device__ __forceinline__
#else
#define JL_HD inline
#endif

namespace jl {

constexpr uint32_t kPhiloxM0 = 0xD2511F53u;
constexpr uint32_t kPhiloxM1 = 0xCD9E8D57u;
constexpr uint32_t kPhiloxW0 = 0x9E3779B9u;
constexpr uint32_t kPhiloxW1 = 0xBB67AE85u;

constexpr uint32_t kColumnStride = 658105236u;  // fast_jl/random.cuh:16
constexpr uint32_t kTileStride = 359124577u;    // fast_jl/random.cuh:17

struct u32x4 {
    uint32_t x, y, z, w;
};

// Name of the stream of (column, tile).
JL_HD uint32_t stream_name(uint32_t seed, uint32_t column, uint32_t tile) {
    return seed + kColumnStride * column + kTileStride * tile;
}

// a ^ b ^ c: one v_bitop3_b32 (truth table 0x96) on the device.
JL_HD uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
#else
    return a ^ b ^ c;
#endif
}

// Philox4x32-10, general counter and key.
JL_HD u32x4 philox4x32_10(u32x4 c, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)kPhiloxM0 * c.x;
        const uint64_t p1 = (uint64_t)kPhiloxM1 * c.z;
        u32x4 n;
        n.x = xor3((uint32_t)(p1 >> 32), c.y, k0);
        n.y = (uint32_t)p1;
        n.z = xor3((uint32_t)(p0 >> 32), c.w, k1);
        n.w = (uint32_t)p0;
        c = n;
        k0 += kPhiloxW0;
        k1 += kPhiloxW1;
    }
    return c;
}

// Block n of the stream named s: counter (n, s, 0, 0), key (seed, 0).
JL_HD u32x4 stream_block(uint32_t seed, uint32_t s, uint32_t n) {
    u32x4 c = {n, s, 0u, 0u};
    return philox4x32_10(c, seed, 0u);
}

JL_HD uint32_t word_of(const u32x4& b, uint32_t i) {
    return i == 0 ? b.x : (i == 1 ? b.y : (i == 2 ? b.z : b.w));
}

// Rademacher entry for offset j (0..127) inside a 128-entry block: 1 -> +1, 0 -> -1.
JL_HD uint32_t rademacher_bit(const u32x4& b, uint32_t j) {
    return (word_of(b, j >> 5) >> (j & 31u)) & 1u;
}

// ---- Box-Muller in explicit binary32 arithmetic -------------------------------------------

JL_HD float u2f(uint32_t u) {
    union {
        uint32_t u;
        float f;
    } v;
    v.u = u;
    return v.f;
}
JL_HD uint32_t f2u(float f) {
    union {
        uint32_t u;
        float f;
    } v;
    v.f = f;
    return v.u;
}

#if defined(__HIP_DEVICE_COMPILE__)
#define JL_FMA(a, b, c) __builtin_fmaf((a), (b), (c))
#define JL_MUL(a, b) __fmul_rn((a), (b))
#define JL_ADD(a, b) __fadd_rn((a), (b))
#else
#define JL_FMA(a, b, c) __builtin_fmaf((a), (b), (c))
JL_HD float jl_mul_(float a, float b) {
    volatile float r = a * b;
    return r;
}
JL_HD float jl_add_(float a, float b) {
    volatile float r = a + b;
    return r;
}
#define JL_MUL(a, b) jl::jl_mul_((a), (b))
#define JL_ADD(a, b) jl::jl_add_((a), (b))
#endif

constexpr uint32_t kRadiusBits = 14, kAngleBits = 14;  // 2^14 entries each: 32 KB of fp16 radii, 64 KB of fp16 pairs

// Radius table entry: r = sqrt(-2 ln u), u = (2x + 1) / 2^15 in (0, 1), for a 14-bit index x.
JL_HD float bm_radius(uint32_t x) {
    const uint32_t odd = (x << 1) | 1u;  // < 2^15: exact as float
    const uint32_t xb = f2u((float)odd);
    int e = (int)(xb >> 23) - 127;
    float m = u2f((xb & 0x007FFFFFu) | 0x3F800000u);  // [1, 2)
    if (m > 1.41421354f) {
        m = JL_MUL(m, 0.5f);
        e += 1;
    }
    const float t = JL_ADD(m, -1.0f);
    const float z = JL_MUL(t, t);
    float p = 7.0376836292e-2f;
    p = JL_FMA(p, t, -1.1514610310e-1f);
    p = JL_FMA(p, t, 1.1676998740e-1f);
    p = JL_FMA(p, t, -1.2420140846e-1f);
    p = JL_FMA(p, t, 1.4249322787e-1f);
    p = JL_FMA(p, t, -1.6668057665e-1f);
    p = JL_FMA(p, t, 2.0000714765e-1f);
    p = JL_FMA(p, t, -2.4999993993e-1f);
    p = JL_FMA(p, t, 3.3333331174e-1f);
    float y = JL_MUL(t, JL_MUL(z, p));
    y = JL_FMA(-0.5f, z, y);
    const float lnm = JL_ADD(t, y);
    const float lnu = JL_FMA((float)(e - 15), 0.693147182f, lnm);
    const float s = JL_MUL(-2.0f, lnu);
    // sqrt(s) by three Newton steps on 1/sqrt(s) from an integer seed
    float g = u2f(0x5f3759dfu - (f2u(s) >> 1));
    const float h = JL_MUL(0.5f, s);
#pragma unroll
    for (int it = 0; it < 3; ++it) {
        const float gg = JL_MUL(g, g);
        const float c = JL_FMA(-h, gg, 1.5f);
        g = JL_MUL(g, c);
    }
    return JL_MUL(s, g);
}

// Angle table entry: cos and sin of theta = (a + 1/2) * 2 pi / 2^14 for a 14-bit index a.  The two top
// bits of a are the quadrant, the other twelve the angle (a' + 1/2) * (pi/2) / 2^12 in (0, pi/2) inside it;
// the upper half of that range is the mirror image of the lower one (cos <-> sin), so the polynomials only
// see (0, pi/4), and the quadrant turns the pair by a multiple of pi/2 (exact: swaps and sign changes).
JL_HD void bm_cossin(uint32_t a, float* c_out, float* s_out) {
    const uint32_t quadrant = (a >> 12) & 3u, aq = a & 4095u;
    const bool mirror = aq >= 2048u;
    const uint32_t am = mirror ? 4095u - aq : aq;
    const float yv = JL_MUL(JL_ADD((float)am, 0.5f), 3.83495208e-4f);  // pi / 2^13
    const float y2 = JL_MUL(yv, yv);
    float ps = JL_FMA(-1.9515295891e-4f, y2, 8.3321608736e-3f);
    ps = JL_FMA(ps, y2, -1.6666654611e-1f);
    const float sn = JL_FMA(JL_MUL(ps, y2), yv, yv);
    float pc = JL_FMA(2.443315711809948e-5f, y2, -1.388731625493765e-3f);
    pc = JL_FMA(pc, y2, 4.166664568298827e-2f);
    const float cs = JL_FMA(JL_MUL(pc, y2), y2, JL_FMA(-0.5f, y2, 1.0f));
    const float c1 = mirror ? sn : cs, s1 = mirror ? cs : sn;  // first quadrant
    *c_out = quadrant == 0 ? c1 : quadrant == 1 ? -s1 : quadrant == 2 ? -c1 : s1;
    *s_out = quadrant == 0 ? s1 : quadrant == 1 ? c1 : quadrant == 2 ? -s1 : -c1;
}

// binary32 -> binary16 bit pattern, round to nearest even (|v| < 65504 here, no NaN).  On the
// device this is the hardware conversion (v_cvt_f16_f32, IEEE round-to-nearest-even with
// subnormals); the host spells the same rounding out in integer arithmetic.
JL_HD uint16_t f32_to_f16_rne(float v) {
#if defined(__HIP_DEVICE_COMPILE__)
    // the empty asm keeps the binary32 value a separate, already rounded operand: without it the
    // compiler folds a preceding multiply into a mixed-precision FMA that rounds only once
    asm("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, (_Float16)v);
#else
    const uint32_t b = f2u(v);
    const uint32_t sign = (b >> 16) & 0x8000u;
    const uint32_t a = b & 0x7FFFFFFFu;
    if (a < 0x38800000u) {              // below the smallest normal half: subnormal or zero
        if (a < 0x33000000u) return (uint16_t)sign;   // < 2^-25 rounds to zero
        const uint32_t e = a >> 23;                    // 102..112
        const uint32_t man = (a & 0x007FFFFFu) | 0x00800000u;
        const uint32_t shift = 126u - e;               // 14..24
        uint32_t hm = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (hm & 1u))) hm += 1u;
        return (uint16_t)(sign | hm);
    }
    uint32_t r = a - 0x38000000u;        // rebias exponent
    const uint32_t rem = r & 0x1FFFu;
    r >>= 13;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r += 1u;
    return (uint16_t)(sign | r);
#endif
}

JL_HD float f16_bits_to_f32(uint16_t hbits) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (float)__builtin_bit_cast(_Float16, hbits);  // exact
#else
    const uint32_t sign = ((uint32_t)hbits & 0x8000u) << 16;
    const uint32_t e = (hbits >> 10) & 0x1Fu;
    const uint32_t m = hbits & 0x3FFu;
    if (e == 0) {
        // subnormal: m * 2^-24, exact in binary32
        const float v = (float)m * 5.9604644775390625e-8f;
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
#endif
}

// ---- entry of the matrix --------------------------------------------------------------------

// o = feature offset inside the tile.  Returns the value as binary32 (always exactly
// representable in fp16).
JL_HD float entry_rademacher(uint32_t seed, uint32_t column, uint32_t tile, uint32_t o) {
    const u32x4 b = stream_block(seed, stream_name(seed, column, tile), o >> 7);
    return rademacher_bit(b, o & 127u) ? 1.0f : -1.0f;
}

// The fields of one random word: it makes one Box-Muller pair.
//   bits 17..30  radius index x          bits 2..15  angle index a          (bits 0, 1, 16, 31 unused)
JL_HD uint32_t normal_radius_index(uint32_t w) { return (w >> 17) & 0x3FFFu; }
JL_HD uint32_t normal_angle_index(uint32_t w) { return (w >> 2) & 0x3FFFu; }

// fp16 product of two fp16 values, round to nearest even (the product is exact in binary32).
JL_HD uint16_t f16_mul_rne(uint16_t a, uint16_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    const _Float16 p = __builtin_bit_cast(_Float16, a) * __builtin_bit_cast(_Float16, b);
    return __builtin_bit_cast(uint16_t, p);
#else
    return f32_to_f16_rne(JL_MUL(f16_bits_to_f32(a), f16_bits_to_f32(b)));
#endif
}

JL_HD uint16_t entry_normal_f16bits(uint32_t seed, uint32_t column, uint32_t tile, uint32_t o) {
    const u32x4 b = stream_block(seed, stream_name(seed, column, tile), o >> 3);
    const uint32_t e = o & 7u;
    const uint32_t w = word_of(b, e >> 1);
    const uint16_t r = f32_to_f16_rne(bm_radius(normal_radius_index(w)));
    float c, s;
    bm_cossin(normal_angle_index(w), &c, &s);
    const uint16_t t = f32_to_f16_rne((e & 1u) ? s : c);
    return f16_mul_rne(r, t);
}

JL_HD float entry_normal(uint32_t seed, uint32_t column, uint32_t tile, uint32_t o) {
    return f16_bits_to_f32(entry_normal_f16bits(seed, column, tile, o));
}

// Tiling of the feature axis (fast_jl/fast_jl.cu:42, fast_jl/fast_jl_kernel.cuh:124).
struct Tiling {
    uint32_t tiles;      // T = min(P, num_feature_tiles)
    uint64_t tile_size;  // fts = ceil(P / T)
};
JL_HD Tiling make_tiling(uint64_t P, uint32_t num_feature_tiles) {
    Tiling t;
    t.tiles = (uint64_t)num_feature_tiles < P ? num_feature_tiles : (uint32_t)P;
    t.tile_size = (P - 1) / t.tiles + 1;
    return t;
}

}  // namespace jl
