/* TEST INFRASTRUCTURE ONLY -- CPU oracle for the JL projection path.
 *
 * Plain C restatement of what the projection computes, written without looking at (and
 * without including) the library's own stream header, so that agreement between the two is
 * evidence and not a tautology.  Only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py may load this file's shared object; the product path never does.
 *
 * What each function restates
 *   jlo_philox4x32_10     Philox4x32-10 of Salmon et al. (Random123 v1.09, philox.h); the
 *                         reference's own generator is cuRAND XORWOW (fast_jl/random.cuh:19),
 *                         which is replaced by Philox in this build.
 *                         PINNED by Random123's kat_vectors (tests/test_oracle_philox.py).
 *   jlo_stream_name       fast_jl/random.cuh:15-17  (closed form, uint32 wrap): the 32-bit value
 *                         that names the stream of (column, tile); the reference seeds the
 *                         pair's generator with it.  PINNED by hand-computed values.
 *   jlo_stream_block      block number n of the stream named s: Philox with counter
 *                         (n, s, 0, 0) and key (seed, 0) - a definition of this build.
 *                         PINNED by Random123's kat_vectors through jlo_philox4x32_10.
 *   jlo_tiling            fast_jl/fast_jl.cu:42 (T = min(F, tiles)) and
 *                         fast_jl/fast_jl_kernel.cuh:124 (fts = ceil(F / T)).  PINNED by the
 *                         iteration counts of the reference's shapes.
 *   jlo_entry             position -> (stream, block, bit) map.  This map is a definition of
 *                         this build (the reference's XORWOW draw order cannot be reproduced);
 *                         what it keeps from fast_jl/random.cuh:27-60 -- one stream per
 *                         (column, tile), entries in feature order, one bit per Rademacher
 *                         entry with bit set -> +1, Box-Muller normals in fp16 -- is
 *                         PINNED by a second independent implementation (oracle/jl_oracle.py),
 *                         by exhaustive "every bit of a block used exactly once" checks, by the
 *                         parity property of tests/test_rademacher.py:65-108 and by
 *                         float64 math-library Box-Muller (tests/test_oracle_entries.py).
 *   jlo_project           out[b, c] = sum_f G[b, f] * S[f, c] in float64, i.e. what
 *                         fast_jl/fast_jl_kernel.cuh:60-104 + fast_jl/fast_jl.cu:78 compute in
 *                         fp16 x fp16 -> fp32.  PINNED against numpy matmul with the
 *                         materialized matrix.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define JLO_RADEMACHER 0
#define JLO_NORMAL 1

void jlo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int round = 0; round < 10; ++round) {
        if (round > 0) {
            k0 += 0x9E3779B9u; /* golden ratio */
            k1 += 0xBB67AE85u; /* sqrt(3) - 1 */
        }
        uint64_t prod0 = (uint64_t)0xD2511F53u * (uint64_t)c0;
        uint64_t prod1 = (uint64_t)0xCD9E8D57u * (uint64_t)c2;
        uint32_t hi0 = (uint32_t)(prod0 >> 32), lo0 = (uint32_t)prod0;
        uint32_t hi1 = (uint32_t)(prod1 >> 32), lo1 = (uint32_t)prod1;
        uint32_t n0 = hi1 ^ c1 ^ k0;
        uint32_t n2 = hi0 ^ c3 ^ k1;
        c0 = n0;
        c1 = lo1;
        c2 = n2;
        c3 = lo0;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

uint32_t jlo_stream_name(uint32_t seed, uint32_t column, uint32_t tile) {
    uint64_t v = (uint64_t)seed + (uint64_t)658105236u * column + (uint64_t)359124577u * tile;
    return (uint32_t)(v & 0xFFFFFFFFu);
}

void jlo_stream_block(uint32_t seed, uint32_t name, uint32_t block, uint32_t out[4]) {
    uint32_t ctr[4] = {block, name, 0u, 0u};
    uint32_t key[2] = {seed, 0u};
    jlo_philox4x32_10(ctr, key, out);
}

void jlo_tiling(uint64_t P, uint32_t num_feature_tiles, uint32_t* tiles, uint64_t* tile_size) {
    uint64_t t = num_feature_tiles;
    if (P < t) t = P;
    *tiles = (uint32_t)t;
    *tile_size = (P + t - 1) / t;
}

static float bits_to_float(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static uint32_t float_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* Radius of a Box-Muller pair for the 14-bit index x: sqrt(-2 ln u) with u = (x + 1/2) / 2^14
 * = (2x + 1) / 2^15, evaluated in binary32 by a fixed sequence of IEEE operations. */
static float radius_from_index(uint32_t x) {
    uint32_t odd = 2u * x + 1u;
    float xf = (float)odd;
    uint32_t xb = float_to_bits(xf);
    int expo = (int)((xb >> 23) & 0xFFu) - 127;
    float mant = bits_to_float((xb & 0x7FFFFFu) | 0x3F800000u);
    if (mant > 1.41421354f) {
        mant = mant * 0.5f;
        expo = expo + 1;
    }
    float t = mant - 1.0f;
    float z = t * t;
    static const float coef[9] = {7.0376836292e-2f, -1.1514610310e-1f, 1.1676998740e-1f,
                                  -1.2420140846e-1f, 1.4249322787e-1f, -1.6668057665e-1f,
                                  2.0000714765e-1f, -2.4999993993e-1f, 3.3333331174e-1f};
    float poly = coef[0];
    for (int i = 1; i < 9; ++i) poly = fmaf(poly, t, coef[i]);
    float zp = z * poly;
    float y = t * zp;
    y = fmaf(-0.5f, z, y);
    float ln_m = t + y;
    float ln_u = fmaf((float)(expo - 15), 0.693147182f, ln_m);
    float s = -2.0f * ln_u;
    float guess = bits_to_float(0x5f3759dfu - (float_to_bits(s) >> 1));
    float half_s = 0.5f * s;
    for (int it = 0; it < 3; ++it) {
        float gg = guess * guess;
        float corr = fmaf(-half_s, gg, 1.5f);
        guess = guess * corr;
    }
    return s * guess;
}

/* cos and sin of the angle (a + 1/2) * 2 pi / 2^14 for the 14-bit index a: a / 4096 is the quadrant,
 * a % 4096 the angle (a % 4096 + 1/2) * (pi/2) / 2^12 inside it.  Inside a quadrant, angles above pi/4
 * are evaluated at their mirror image pi/2 - angle (index 4095 - a % 4096) with cos and sin exchanged;
 * the quadrant then turns the pair by k * pi/2: (c, s) -> (-s, c) per quarter turn. */
static void cos_sin_from_index(uint32_t a, float* c, float* s) {
    uint32_t turns = (a / 4096u) % 4u, in_q = a % 4096u;
    int upper = in_q > 2047u;
    uint32_t idx = upper ? 4095u - in_q : in_q;
    float steps = (float)idx + 0.5f;
    float y = steps * 3.83495208e-4f; /* pi / 2^13 */
    float y2 = y * y;
    float ps = fmaf(-1.9515295891e-4f, y2, 8.3321608736e-3f);
    ps = fmaf(ps, y2, -1.6666654611e-1f);
    float psy2 = ps * y2;
    float sn = fmaf(psy2, y, y);
    float pc = fmaf(2.443315711809948e-5f, y2, -1.388731625493765e-3f);
    pc = fmaf(pc, y2, 4.166664568298827e-2f);
    float pcy2 = pc * y2;
    float base = fmaf(-0.5f, y2, 1.0f);
    float cs = fmaf(pcy2, y2, base);
    float cq = upper ? sn : cs, sq = upper ? cs : sn;
    for (uint32_t t = 0; t < turns; ++t) { /* a quarter turn */
        float nc = -sq, ns = cq;
        cq = nc;
        sq = ns;
    }
    *c = cq;
    *s = sq;
}

/* IEEE binary32 -> binary16 bits, round to nearest even, finite inputs well inside range. */
static uint16_t half_bits_rne(float v) {
    /* exact scaled-integer formulation: find h with |h| closest to |v| */
    uint32_t b = float_to_bits(v);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    double a = fabs((double)v);
    if (a == 0.0) return sign;
    int e;
    (void)frexp(a, &e);          /* a = m * 2^e, m in [0.5, 1) */
    int ue = e - 1;              /* a in [2^ue, 2^(ue+1)) */
    if (ue < -14) ue = -14;      /* subnormal range shares the exponent of 2^-14 */
    double ulp = ldexp(1.0, ue - 10);
    double q = a / ulp;          /* exact: power-of-two scaling */
    double fl = floor(q);
    double rem = q - fl;
    uint64_t n = (uint64_t)fl;
    if (rem > 0.5 || (rem == 0.5 && (n & 1u))) n += 1;
    /* n in [0, 2048]; value = n * 2^(ue-10) */
    uint32_t bits;
    if (n >= 2048u) {            /* rounded up to next binade */
        n = 1024u;
        ue += 1;
    }
    if (n < 1024u) {
        bits = (uint32_t)n;      /* subnormal (ue == -14) */
    } else {
        bits = ((uint32_t)(ue + 15) << 10) | ((uint32_t)n - 1024u);
    }
    return (uint16_t)(sign | bits);
}

static float half_bits_to_float(uint16_t h) {
    int sign = (h >> 15) & 1;
    int e = (h >> 10) & 0x1F;
    int m = h & 0x3FF;
    double v;
    if (e == 0)
        v = ldexp((double)m, -24);
    else
        v = ldexp((double)(m + 1024), e - 25);
    return (float)(sign ? -v : v);
}

/* The three factor tables as fp16 bit patterns (tests compare them with a float64 math library). */
uint16_t jlo_radius_half(uint32_t x) { return half_bits_rne(radius_from_index(x & 0x3FFFu)); }
uint16_t jlo_cos_half(uint32_t a) {
    float c, s;
    cos_sin_from_index(a & 0x3FFFu, &c, &s);
    return half_bits_rne(c);
}
uint16_t jlo_sin_half(uint32_t a) {
    float c, s;
    cos_sin_from_index(a & 0x3FFFu, &c, &s);
    return half_bits_rne(s);
}

/* One normal entry from one random word: radius index = bits 17..30, angle index = bits 2..15 (the
 * cosine and sine tables carry their signs; bits 0, 1, 16 and 31 of the word are not used).
 * The two fp16 factors are multiplied exactly (22-bit product, exact in double) and rounded once. */
float jlo_normal_from_word(uint32_t w, int sine) {
    static uint16_t rtab[1 << 14], ctab[1 << 14], stab[1 << 14];
    static int ready = 0;
    if (!ready) {
        for (uint32_t i = 0; i < (1u << 14); ++i) {
            rtab[i] = jlo_radius_half(i);
            ctab[i] = jlo_cos_half(i);
            stab[i] = jlo_sin_half(i);
        }
        ready = 1;
    }
    uint32_t x = (w >> 17) % 16384u;
    uint32_t a = (w >> 2) % 16384u;
    double radius = (double)half_bits_to_float(rtab[x]);
    double trig = (double)half_bits_to_float(sine ? stab[a] : ctab[a]);
    double prod = radius * trig;
    float pf = (float)prod; /* exact: 22 significant bits, well inside the binary32 range */
    return half_bits_to_float(half_bits_rne(pf));
}

/* Value of S[f, c] (as float; always exactly an fp16 value). */
float jlo_entry(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f, uint32_t c,
                int proj_type) {
    uint32_t tiles;
    uint64_t tile_size;
    jlo_tiling(P, num_feature_tiles, &tiles, &tile_size);
    uint32_t tile = (uint32_t)(f / tile_size);
    uint32_t offset = (uint32_t)(f - (uint64_t)tile * tile_size);
    uint32_t out[4];
    if (proj_type == JLO_RADEMACHER) {
        /* 128 entries per block: entry number i is bit i of the block, words in order, least
         * significant bit first */
        jlo_stream_block(seed, jlo_stream_name(seed, c, tile), offset / 128u, out);
        uint32_t bit = offset % 128u;
        return ((out[bit / 32u] >> (bit % 32u)) & 1u) ? 1.0f : -1.0f;
    } else {
        /* eight entries per block; word i of the block makes entries 2i (cosine) and 2i+1 (sine) */
        jlo_stream_block(seed, jlo_stream_name(seed, c, tile), offset / 8u, out);
        uint32_t e = offset % 8u;
        return jlo_normal_from_word(out[e / 2u], (int)(e % 2u));
    }
}

uint16_t jlo_half_bits(float v) { return half_bits_rne(v); }

/* out[nf, nc] = S[f0:f0+nf, c0:c0+nc] */
void jlo_materialize(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                     uint32_t c0, uint32_t nc, int proj_type, float* out) {
    for (uint64_t i = 0; i < nf; ++i)
        for (uint32_t j = 0; j < nc; ++j)
            out[i * nc + j] = jlo_entry(seed, num_feature_tiles, P, f0 + i, c0 + j, proj_type);
}

/* Float64 contraction for a window of columns: out[B, nc] = G[B, P] * S[:, c0:c0+nc].
 * G is given as binary32 (the test converts fp16/bf16 inputs exactly).  Rademacher blocks are
 * expanded 128 features at a time to keep this usable at full P on a column sample. */
void jlo_project(const float* G, uint64_t B, uint64_t P, uint64_t ld, uint32_t seed,
                 uint32_t num_feature_tiles, uint32_t c0, uint32_t nc, int proj_type, double* out) {
    uint32_t tiles;
    uint64_t tile_size;
    jlo_tiling(P, num_feature_tiles, &tiles, &tile_size);
    for (uint64_t b = 0; b < B; ++b)
        for (uint32_t j = 0; j < nc; ++j) out[b * nc + j] = 0.0;
    float* col = (float*)malloc(sizeof(float) * 128);
    for (uint32_t j = 0; j < nc; ++j) {
        uint32_t c = c0 + j;
        for (uint32_t t = 0; t < tiles; ++t) {
            uint64_t lo = (uint64_t)t * tile_size;
            uint64_t hi = lo + tile_size < P ? lo + tile_size : P;
            if (lo >= hi) continue;
            for (uint64_t base = lo; base < hi; base += 128) {
                uint64_t cnt = hi - base < 128 ? hi - base : 128;
                uint32_t off0 = (uint32_t)(base - lo);
                if (proj_type == JLO_RADEMACHER) {
                    uint32_t w[4];
                    jlo_stream_block(seed, jlo_stream_name(seed, c, t), off0 / 128u, w);
                    for (uint32_t jj = 0; jj < cnt; ++jj)
                        col[jj] = ((w[jj / 32u] >> (jj % 32u)) & 1u) ? 1.0f : -1.0f;
                } else {
                    for (uint32_t jj = 0; jj < cnt; ++jj)
                        col[jj] = jlo_entry(seed, num_feature_tiles, P, base + jj, c, proj_type);
                }
                for (uint64_t b = 0; b < B; ++b) {
                    const float* g = G + b * ld + base;
                    double acc = 0.0;
                    for (uint32_t jj = 0; jj < cnt; ++jj) acc += (double)g[jj] * (double)col[jj];
                    out[b * nc + j] += acc;
                }
            }
        }
    }
    free(col);
}
