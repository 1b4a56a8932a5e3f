// JL projection  out[b, c] = sum_f G[b, f] * S[f, c]  for gfx950 (MI355X).
//
// Replaces project_kernel / project / fast_jl<> of the reference
// (fast_jl/fast_jl_kernel.cuh:24-132, fast_jl/fast_jl.cu:29-79).  S is never
// stored: every wave generates the entries it needs from the Philox stream
// defined in jl_stream.h directly in the register layout of the B operand of
// v_mfma_f32_32x32x16_{f16,bf16} and contracts them against gradient tiles that
// the workgroup staged in LDS.
//
// Work decomposition
//   workgroup = 8 waves = 1024 JL columns (512 columns when the projection
//               dimension is an odd multiple of 512) x a run of consecutive
//               256-feature chunks of the reference's feature tiles
//               (fts = ceil(P / T) consecutive features each);
//   wave      = 4 (or 2) groups of 32 columns, one 32x32 fp32 accumulator each;
//   lane      = (n = lane % 32, h = lane / 32): column n of each group, and the
//               k-slots 8h..8h+7 of every MFMA.
// The tile is walked in chunks of 256 features.  Lane half h owns features
// [128h, 128h+128) of a chunk: MFMA number q (0..15) of the chunk contracts
// features 128h + 8q + i (i = 0..7), so the 8 Rademacher signs a lane needs for it
// are byte q of ONE Philox block per column per chunk, and the A operand is 16
// contiguous bytes of a gradient row.
//
// A workgroup walks a run of consecutive chunks (across tile boundaries, adding the
// products up in its accumulators) and writes one partial [B, 1024] block; a second
// kernel adds the runs up in order, so results do not depend on scheduling.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>
#include <utility>

#include "jl_stream.h"
#include "store_cast.h"
#include "trakhip_internal.h"

namespace {

using trakhip::store4;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// A workgroup has 8 waves (one workgroup per CU, two waves per SIMD) and stages every gradient
// chunk once for all its columns.
constexpr int kColsMultiple = 512;                    // proj dim granularity (fast_jl_kernel.cuh:113)
constexpr int kPieces = 32 * 32;                      // 16-byte pieces of a [32 x 256] chunk of 16-bit values
constexpr int kChunk = 256;                           // features per staged chunk
constexpr int kLdsRow = kChunk + 8;                   // 16-bit elements; 528 B keeps b128 reads conflict free
constexpr int kPlaneElems = 32 * kLdsRow;
constexpr int kPlaneElems32 = kPlaneElems;

struct __attribute__((packed, aligned(2))) Raw16 {
    uint32_t x, y, z, w;
};
struct __attribute__((packed, aligned(4))) Raw16f {
    uint32_t x, y, z, w;
};

// Gradient data is device (global) memory.  Reading it through a pointer that says so keeps the loads
// from becoming FLAT instructions where the pointer comes out of a segment table: a FLAT load counts as
// an LDS operation too, and every wait for an LDS operand would then wait for all the gradient loads in
// flight.
template <typename T>
__device__ __forceinline__ T gload(const void* p) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const T __attribute__((address_space(1))) * global_ptr;
    return *(global_ptr)(uintptr_t)p;  // (a direct pointer cast is folded back into a generic pointer)
#else
    return *static_cast<const T*>(p);  // host pass of the compiler: never executed
#endif
}

template <int IN>
struct InTraits;
template <>
struct InTraits<TRAKHIP_F16> {
    static constexpr int planes = 1;
    static constexpr bool bf16 = false;
};
template <>
struct InTraits<TRAKHIP_BF16> {
    static constexpr int planes = 1;
    static constexpr bool bf16 = true;
};
template <>
struct InTraits<TRAKHIP_F32> {
    static constexpr int planes = 3;  // x = b1 + b2 + b3 exactly, each a bf16
    static constexpr bool bf16 = true;
};

__device__ __forceinline__ floatx16 mfma16(const uint4& a, const uint4& b, floatx16 c, bool bf16) {
    if (bf16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                  __builtin_bit_cast(half8, b), c, 0, 0, 0);
}

// ---- staging of a [32 x 256] gradient chunk ------------------------------------------------

// 16-bit inputs: every thread moves N = ROWS / (2 W) 16-byte pieces, 2 W rows apart (ROWS = 32, or 64
// for the kernel that multiplies two 32-row blocks by every operand).
template <int W, int ROWS = 32>
struct Stage16 {
    static constexpr int N = ROWS * 32 / (64 * W);
    static constexpr int kThreads = 64 * W;
    uint4 v[N];

    // all ROWS rows and the whole chunk in range: unguarded 16-byte loads
    __device__ __forceinline__ void load_whole(const uint16_t* __restrict__ g, uint64_t ld, uint64_t f_begin, int tid) {
        const uint16_t* p = g + (uint64_t)(tid >> 5) * ld + f_begin + 8u * (tid & 31);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const Raw16 r = gload<Raw16>(p + (uint64_t)(2 * W * i) * ld);
            v[i] = {r.x, r.y, r.z, r.w};
        }
    }
    // the same from the address of the thread's first piece and the distance in bytes to its next one
    __device__ __forceinline__ void load_pieces(const char* p, uint64_t piece_pitch) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const Raw16 r = gload<Raw16>(p + i * piece_pitch);
            v[i] = {r.x, r.y, r.z, r.w};
        }
    }
    __device__ __forceinline__ void load(const uint16_t* __restrict__ g, uint64_t ld, uint32_t rows,
                                         uint64_t f_begin, uint64_t f_end, int tid) {
        if (rows == ROWS && f_begin + kChunk <= f_end) {  // uniform test
            load_whole(g, ld, f_begin, tid);
            return;
        }
        load_edge(g, ld, rows, f_begin, f_end, tid);
    }
    // rows beyond `rows` and features beyond f_end read as zero
    __device__ __forceinline__ void load_edge(const uint16_t* __restrict__ g, uint64_t ld, uint32_t rows,
                                              uint64_t f_begin, uint64_t f_end, int tid) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = tid + kThreads * i;
            const uint32_t row = id >> 5, sg = id & 31;
            const uint64_t f = f_begin + 8u * sg;
            uint4 val = {0u, 0u, 0u, 0u};
            if (row < rows && f < f_end) {
                const uint16_t* p = g + (uint64_t)row * ld + f;
                if (f + 8 <= f_end) {
                    const Raw16 r = gload<Raw16>(p);
                    val = {r.x, r.y, r.z, r.w};
                } else {
                    uint32_t e[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) e[t] = (f + t < f_end) ? (uint32_t)gload<uint16_t>(p + t) : 0u;
                    val = {e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16),
                           e[6] | (e[7] << 16)};
                }
            }
            v[i] = val;
        }
    }
    __device__ __forceinline__ void store(uint16_t* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = tid + kThreads * i;
            const uint32_t row = id >> 5, sg = id & 31;
            *reinterpret_cast<uint4*>(lds + row * kLdsRow + 8 * sg) = v[i];
        }
    }
};

// fp32 inputs: every thread moves N = 32 / W pieces of 4 floats, W rows apart, and splits each float into
// three bf16 terms by truncation (x = b1 + b2 + b3 exactly).
template <int W>
struct Stage32 {
    static constexpr int N = 2 * kPieces / (64 * W);
    static constexpr int kThreads = 64 * W;
    uint4 v[N];

    __device__ __forceinline__ void load(const float* __restrict__ g, uint64_t ld, uint32_t rows,
                                         uint64_t f_begin, uint64_t f_end, int tid) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = tid + kThreads * i;
            const uint32_t row = id >> 6, sg = id & 63;
            const uint64_t f = f_begin + 4u * sg;
            uint4 val = {0u, 0u, 0u, 0u};
            if (row < rows && f < f_end) {
                const float* p = g + (uint64_t)row * ld + f;
                if (f + 4 <= f_end) {
                    const Raw16f r = gload<Raw16f>(p);
                    val = {r.x, r.y, r.z, r.w};
                } else {
                    val.x = gload<uint32_t>(p);
                    val.y = (f + 1 < f_end) ? gload<uint32_t>(p + 1) : 0u;
                    val.z = (f + 2 < f_end) ? gload<uint32_t>(p + 2) : 0u;
                    val.w = 0u;
                }
            }
            v[i] = val;
        }
    }
    __device__ __forceinline__ static void split(uint32_t xb, uint32_t& b1, uint32_t& b2, uint32_t& b3) {
        const float x = __uint_as_float(xb);
        const uint32_t h1 = xb & 0xFFFF0000u;
        const float r1 = x - __uint_as_float(h1);
        const uint32_t h2 = __float_as_uint(r1) & 0xFFFF0000u;
        const float r2 = r1 - __uint_as_float(h2);
        b1 = h1 >> 16;
        b2 = h2 >> 16;
        b3 = __float_as_uint(r2) >> 16;
    }
    __device__ __forceinline__ void store(uint16_t* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = tid + kThreads * i;
            const uint32_t row = id >> 6, sg = id & 63;
            uint32_t a[4][3];
            split(v[i].x, a[0][0], a[0][1], a[0][2]);
            split(v[i].y, a[1][0], a[1][1], a[1][2]);
            split(v[i].z, a[2][0], a[2][1], a[2][2]);
            split(v[i].w, a[3][0], a[3][1], a[3][2]);
#pragma unroll
            for (int pl = 0; pl < 3; ++pl) {
                uint2 o = {a[0][pl] | (a[1][pl] << 16), a[2][pl] | (a[3][pl] << 16)};
                *reinterpret_cast<uint2*>(lds + pl * kPlaneElems + row * kLdsRow + 4 * sg) = o;
            }
        }
    }
};

// ---- gathered input: the gradient is a list of per-parameter tensors --------------------
//
// Segment i holds features [first, first + numel) as a row-major [B, numel] tensor with row
// pitch ld (what TRAK's gradient dict holds per parameter, trak/utils.py:80-110).  A thread's
// pieces of one chunk all start at the same feature, and that feature only grows while the
// workgroup walks its run, so the thread keeps the segment it is in and moves forward when needed.
// ROWS = pieces per thread and chunk (all at the same feature, ROW_STEP rows apart).
template <int ROWS>
struct SegCursor {
    uint32_t idx;
    uint32_t first, end;         // feature range of segs[idx] (P < 2^32)
    const char* base[ROWS];      // base[i] + feature * elem_size = address of (row_i, feature)

    __device__ __forceinline__ void set(const trakhip_segment* segs, uint32_t i, uint32_t row0, uint32_t row_step,
                                        uint32_t esz) {
        const trakhip_segment sg = segs[i];
        idx = i;
        first = (uint32_t)sg.first;
        end = (uint32_t)(sg.first + sg.numel);
        const char* p = static_cast<const char*>(sg.ptr) - sg.first * esz;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) base[r] = p + (uint64_t)(row0 + row_step * r) * sg.ld * esz;
    }
    // segment containing feature f (segments are sorted, contiguous and cover [0, P); f < P)
    __device__ __forceinline__ void seek(const trakhip_segment* segs, uint32_t n, uint32_t f, uint32_t row0,
                                         uint32_t row_step, uint32_t esz) {
        uint32_t lo = 0, hi = n - 1;
        while (lo < hi) {
            const uint32_t mid = (lo + hi + 1) >> 1;
            if (segs[mid].first <= f)
                lo = mid;
            else
                hi = mid - 1;
        }
        set(segs, lo, row0, row_step, esz);
    }
    __device__ __forceinline__ void advance(const trakhip_segment* segs, uint32_t n, uint32_t f, uint32_t row0,
                                            uint32_t row_step, uint32_t esz) {
        while (f >= end && idx + 1 < n) set(segs, idx + 1, row0, row_step, esz);
    }
};

// A piece of COUNT elements that straddles a segment boundary or the end of the tile (slow path,
// kept out of line and rolled up so that the hot loop stays small).
template <typename T, int COUNT>
__device__ __noinline__ uint4 gather_piece(const trakhip_segment* segs, uint32_t n, uint32_t idx, uint32_t row,
                                           uint64_t f, uint64_t f_end) {
    uint32_t e[4] = {0u, 0u, 0u, 0u};
#pragma unroll 1
    for (int t = 0; t < COUNT; ++t) {
        const uint64_t ff = f + t;
        if (ff >= f_end) break;
        while (idx + 1 < n && ff >= segs[idx + 1].first) ++idx;
        const trakhip_segment sg = segs[idx];
        const uint32_t val = (uint32_t)gload<T>(reinterpret_cast<const T*>(sg.ptr) + (uint64_t)row * sg.ld + (ff - sg.first));
        if (sizeof(T) == 2)
            e[t >> 1] |= val << (16 * (t & 1));
        else
            e[t] = val;
    }
    return {e[0], e[1], e[2], e[3]};
}

// The segment the workgroup's current chunk starts in, as uniform values (scalar registers): when the
// whole chunk lies inside it, the chunk is loaded like a chunk of a dense matrix, without the per-thread
// cursors below.
// 16-bit elements; a thread's pieces are at row tid / 32 + row_step * i, features 8 (tid % 32) .. + 7 of the chunk.
struct UniformSeg {
    uint32_t idx;
    uint32_t first, end;   // feature range of segs[idx] (P < 2^32)
    uint64_t piece_pitch;  // bytes from one piece of a thread to its next (row_step rows)
    const char* tbase;     // per thread: tbase + 2 f = address of its first piece of the chunk that starts at feature f
    __device__ __forceinline__ void set(const trakhip_segment* segs, uint32_t i, int tid, uint32_t row_step) {
        const trakhip_segment sg = segs[i];
        // the same values in every lane; said so, they live in scalar registers (a load that follows a
        // barrier is never a scalar load by itself)
        idx = i;
        first = __builtin_amdgcn_readfirstlane((uint32_t)sg.first);
        end = __builtin_amdgcn_readfirstlane((uint32_t)(sg.first + sg.numel));
        const uint64_t pp = (uint64_t)row_step * sg.ld * 2;
        piece_pitch = ((uint64_t)__builtin_amdgcn_readfirstlane((uint32_t)(pp >> 32)) << 32) |
                      __builtin_amdgcn_readfirstlane((uint32_t)pp);
        tbase = static_cast<const char*>(sg.ptr) + ((uint64_t)(tid >> 5) * sg.ld + 8u * (tid & 31)) * 2 - sg.first * 2;
    }
    __device__ __forceinline__ void seek(const trakhip_segment* segs, uint32_t n, uint32_t f, int tid, uint32_t row_step) {
        uint32_t lo = 0, hi = n - 1;
        while (lo < hi) {
            const uint32_t mid = (lo + hi + 1) >> 1;
            if ((uint32_t)segs[mid].first <= f)
                lo = mid;
            else
                hi = mid - 1;
        }
        set(segs, lo, tid, row_step);
    }
    __device__ __forceinline__ void advance(const trakhip_segment* segs, uint32_t n, uint32_t f, int tid, uint32_t row_step) {
        while (f >= end && idx + 1 < n) set(segs, idx + 1, tid, row_step);
    }
};

template <int W, int ROWS = 32>
struct Gather16 : Stage16<W, ROWS> {
    static constexpr int N = Stage16<W, ROWS>::N;
    using Stage16<W, ROWS>::v;
    SegCursor<N> cur;
    __device__ __forceinline__ void init(const trakhip_segment* segs, uint32_t n, uint64_t f_begin, uint64_t P,
                                         int tid) {
        const uint64_t f = f_begin + 8u * (tid & 31);
        cur.seek(segs, n, (uint32_t)(f < P ? f : P - 1), tid >> 5, 2 * W, 2);
    }
    __device__ __forceinline__ void load(const trakhip_segment* segs, uint64_t n64, uint32_t rows, uint64_t f_begin,
                                         uint64_t f_end, int tid) {
        const uint32_t n = (uint32_t)n64;
        const uint64_t f64 = f_begin + 8u * (tid & 31);
        const bool live = f64 < f_end;
        const uint32_t f = (uint32_t)f64;
        if (live) cur.advance(segs, n, f, tid >> 5, 2 * W, 2);
        load_at(segs, n, cur, rows, f64, f_end, live, tid);
    }
    // The same with a cursor that lives for this call only and starts at segment `start`, one that begins
    // at or before f_begin: for a caller that takes this path rarely and saves the registers.
    __device__ __forceinline__ void load_from(const trakhip_segment* segs, uint32_t n, uint32_t start, uint32_t rows,
                                              uint64_t f_begin, uint64_t f_end, int tid) {
        const uint64_t f64 = f_begin + 8u * (tid & 31);
        const bool live = f64 < f_end;
        SegCursor<N> c;
        c.set(segs, start, tid >> 5, 2 * W, 2);
        if (live) c.advance(segs, n, (uint32_t)f64, tid >> 5, 2 * W, 2);
        load_at(segs, n, c, rows, f64, f_end, live, tid);
    }
    __device__ __forceinline__ void load_at(const trakhip_segment* segs, uint32_t n, const SegCursor<N>& c, uint32_t rows,
                                            uint64_t f64, uint64_t f_end, bool live, int tid) {
        const uint32_t f = (uint32_t)f64;
        const uint32_t lim = (uint32_t)f_end < c.end ? (uint32_t)f_end : c.end;  // f_end <= P < 2^32
        const bool whole = live && f + 8u <= lim && f + 8u > f;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const uint32_t row = (tid >> 5) + 2 * W * i;
            uint4 val = {0u, 0u, 0u, 0u};
            if (live && row < rows) {
                if (whole) {
                    const Raw16 r = gload<Raw16>(c.base[i] + (uint64_t)f * 2);
                    val = {r.x, r.y, r.z, r.w};
                } else {
                    val = gather_piece<uint16_t, 8>(segs, n, c.idx, row, f64, f_end);
                }
            }
            v[i] = val;
        }
    }
};

template <int W>
struct Gather32 : Stage32<W> {
    static constexpr int N = Stage32<W>::N;
    using Stage32<W>::v;
    SegCursor<N> cur;
    __device__ __forceinline__ void init(const trakhip_segment* segs, uint32_t n, uint64_t f_begin, uint64_t P,
                                         int tid) {
        const uint64_t f = f_begin + 4u * (tid & 63);
        cur.seek(segs, n, (uint32_t)(f < P ? f : P - 1), tid >> 6, W, 4);
    }
    __device__ __forceinline__ void load(const trakhip_segment* segs, uint64_t n64, uint32_t rows, uint64_t f_begin,
                                         uint64_t f_end, int tid) {
        const uint32_t n = (uint32_t)n64;
        const uint64_t f64 = f_begin + 4u * (tid & 63);
        const bool live = f64 < f_end;
        const uint32_t f = (uint32_t)f64;
        if (live) cur.advance(segs, n, f, tid >> 6, W, 4);
        const uint32_t lim = (uint32_t)f_end < cur.end ? (uint32_t)f_end : cur.end;
        const bool whole = live && f + 4u <= lim && f + 4u > f;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const uint32_t row = (tid >> 6) + W * i;
            uint4 val = {0u, 0u, 0u, 0u};
            if (live && row < rows) {
                if (whole) {
                    const Raw16f r = gload<Raw16f>(cur.base[i] + (uint64_t)f * 4);
                    val = {r.x, r.y, r.z, r.w};
                } else {
                    val = gather_piece<uint32_t, 4>(segs, n, cur.idx, row, f64, f_end);
                }
            }
            v[i] = val;
        }
    }
};

template <int IN, bool GATHER, int W, int ROWS = 32>
struct StageOf {
    typedef Stage16<W, ROWS> type;
    typedef uint16_t elem;
};
template <int W, int ROWS>
struct StageOf<TRAKHIP_F32, false, W, ROWS> {
    typedef Stage32<W> type;
    typedef float elem;
};
template <int W, int ROWS>
struct StageOf<TRAKHIP_F16, true, W, ROWS> {
    typedef Gather16<W, ROWS> type;
    typedef trakhip_segment elem;
};
template <int W, int ROWS>
struct StageOf<TRAKHIP_BF16, true, W, ROWS> {
    typedef Gather16<W, ROWS> type;
    typedef trakhip_segment elem;
};
template <int W, int ROWS>
struct StageOf<TRAKHIP_F32, true, W, ROWS> {
    typedef Gather32<W> type;
    typedef trakhip_segment elem;
};

// ---- Rademacher projection -------------------------------------------------------------------

// Workgroup id -> (column block, run of chunks).  The units u = run * col_blocks + column block are
// numbered so that the column blocks of one run are neighbours, and the 8 XCDs - which are handed
// the workgroups round-robin by linear id - each take a contiguous eighth of them: the column
// blocks of a run then sit on the same XCD at the same time (a run cut by the border between two
// eighths sits on two), so a gradient chunk is fetched from HBM once and then served by that XCD's
// L2.  The launch has 8 * ceil(units / 8) workgroups; false = padding, nothing to do.
__device__ __forceinline__ bool map_workgroup(uint32_t linear, uint32_t col_blocks, uint32_t groups, uint32_t& cb,
                                              uint32_t& group) {
    const uint32_t xcd = linear & 7u, idx = linear >> 3;
    const uint64_t units = (uint64_t)groups * col_blocks;
    const uint32_t lo = (uint32_t)(xcd * units / 8u), hi = (uint32_t)((xcd + 1u) * units / 8u);
    const uint32_t u = lo + idx;
    if (u >= hi) return false;
    group = u / col_blocks;
    cb = u - group * col_blocks;
    return true;
}

// The B operand of one MFMA is eight signs = one byte of a Philox block, looked up in LDS:
// entry e of the table holds the packed 16-bit values (bit i of e set -> +1, clear -> -1) for
// i = 0..7.  There are sixteen copies of every entry, (e * 16 + copy) * 16 bytes from the start
// of LDS, and a lane reads copy lane % 16: the sixteen lanes that the LDS serves in one cycle of a
// 16-byte read then hit all 64 banks whatever their bytes are.
constexpr int kSignCopies = 16;
constexpr int kSignTableBytes = 256 * kSignCopies * 16;  // 64 KB

// Address of the table entry for byte q % 4 of `word`: one v_perm_b32 puts the byte into bits
// 8..15 over lane_base = (lane % 16) * 16.
__device__ __forceinline__ uint32_t sign_entry_address(uint32_t word, int q, uint32_t lane_base) {
    const uint32_t sel = 0x0C0C0000u | ((4u + (uint32_t)(q & 3)) << 8);  // {0, 0, word.byte[q % 4], lane_base.byte[0]}
    return __builtin_amdgcn_perm(word, lane_base, sel);
}

// Half of a Philox round on one column group's state: half 0 is the multiply of c.x (gives z, w
// of the next state), half 1 the multiply of c.z (gives x, y).  The empty asm statements tie the
// instructions to the place in the instruction stream where the call stands: without them the
// compiler moves all the generator arithmetic of a chunk in front of its first MFMA.
//
// In two parts, so that other instructions of the step can stand between the asm that ties down the
// inputs and the multiply: the compiler assumes that a register written by inline asm may not be read
// by the very next vector instruction (one wait state on this target) and would put an s_nop there.
struct PhiloxHalfIn {
    uint32_t m, o;  // the word that is multiplied and the word that is xored into the high half
};
__device__ __forceinline__ PhiloxHalfIn philox_half_in(const jl::u32x4& c, int half) {
    PhiloxHalfIn in = {half == 0 ? c.x : c.z, half == 0 ? c.w : c.y};
    asm volatile("" : "+v"(in.m), "+v"(in.o));
    return in;
}
__device__ __forceinline__ void philox_half_out(const PhiloxHalfIn& in, jl::u32x4& next, int half, uint32_t k0,
                                                uint32_t k1) {
    if (half == 0) {
        const uint64_t p0 = (uint64_t)jl::kPhiloxM0 * in.m;
        next.z = jl::xor3((uint32_t)(p0 >> 32), in.o, k1);
        next.w = (uint32_t)p0;
        asm volatile("" : "+v"(next.z), "+v"(next.w));
    } else {
        const uint64_t p1 = (uint64_t)jl::kPhiloxM1 * in.m;
        next.x = jl::xor3((uint32_t)(p1 >> 32), in.o, k0);
        next.y = (uint32_t)p1;
        asm volatile("" : "+v"(next.x), "+v"(next.y));
    }
}

// f(integral_constant<int, 0>), f(integral_constant<int, 1>), ... in this order
template <class F, int... S>
__device__ __forceinline__ void for_each_step(F& f, std::integer_sequence<int, S...>) {
    (f(std::integral_constant<int, S>{}), ...);
}

// GATHER: g_in is a device array of trakhip_segment and ld their number; otherwise g_in is the
// dense [rows, P] matrix with row pitch ld.  GPW = 32-column groups per wave: 4 (workgroup = 1024
// columns), or for projection dimensions that are an odd multiple of 512: 3 (768 columns) when 768
// divides the dimension, else 2 (512 columns).
//
// The main loop is written out step by step.  A chunk is 16 * GPW steps (q, j): one table lookup
// and one MFMA (three for fp32 gradients) for column group j and features 8q..8q+7 of the lane's
// half of the chunk.  Under them runs the generator for the NEXT chunk, one half round or two per
// step (nine rounds x GPW groups x two halves spread over the steps; the first round has scalar
// operands and is done at the top of the chunk), and the operand reads run kAhead steps ahead of
// the MFMA that uses them.  The matrix pipe stays busy only if the vector instructions between two
// MFMAs of a wave fit into the time of one MFMA of each of the two waves of the SIMD (8 issue
// slots of 4 cycles each, two of them for a 64-bit multiply), which is why the generator is cut
// that fine.
//
// RB = 32-row blocks per pass: 1, or 2 for 16-bit gradients when the batch has more than 32 rows - every
// looked-up operand (and the generator behind it) then feeds two MFMAs.
template <int IN, bool GATHER, int GPW, int RB>
__global__ __launch_bounds__(512) void jl_project_kernel(
    const void* __restrict__ g_in, uint64_t ld, uint32_t rows, uint64_t P, uint32_t k,
    uint32_t seed, uint32_t tiles, uint64_t tile_size, uint32_t chunks_per_tile,
    uint32_t chunks_per_group, uint32_t groups, float* __restrict__ partial) {
    constexpr int W = 8;
    typedef InTraits<IN> Tr;
    typedef typename StageOf<IN, GATHER, W, 32 * RB>::type Stage;
    typedef typename StageOf<IN, GATHER, W, 32 * RB>::elem Elem;
    constexpr int kColsPerWG = W * GPW * 32;
    constexpr bool kBf = Tr::bf16;
    constexpr int kPlanes = Tr::planes;
    static_assert(RB == 1 || kPlanes == 1, "two row blocks: 16-bit gradients only (LDS)");
    // 16-bit inputs: two LDS buffers, one barrier per chunk.  fp32 inputs (three planes) keep one
    // buffer and two barriers: two buffers of three planes do not fit next to the table.
    constexpr int kBuffers = kPlanes == 1 ? 2 : 1;
    constexpr int kPlaneElems = RB * kPlaneElems32;  // this kernel's plane: 32 RB rows
    constexpr int kBufElems = kPlanes * kPlaneElems;
    constexpr int kSteps = 16 * GPW;
    constexpr int kAhead = 3;                       // operand reads in flight
    constexpr int kHalfRounds = 9 * GPW * 2;        // rounds 1..9 of the next chunk's blocks
    static_assert(kSteps % (kAhead + 1) == 0, "the operand ring must close over a chunk");
    static_assert(kHalfRounds >= kSteps && kHalfRounds <= 2 * kSteps, "one or two half rounds per step");

    // the table comes first: a DS instruction adds a 16-bit immediate to the address register, and
    // a table entry's address is built without adding a base
    __shared__ __attribute__((aligned(256))) char smem[kSignTableBytes + kBuffers * kBufElems * 2];
    uint16_t* lds = reinterpret_cast<uint16_t*>(smem + kSignTableBytes);

    const uint32_t col_blocks = k / kColsPerWG;
    uint32_t cb, group;
    if (!map_workgroup(blockIdx.x, col_blocks, groups, cb, group)) return;
    // this workgroup's share of the flattened (tile, chunk) sequence; the streams are counter
    // based, so a workgroup can start in the middle of a tile
    const uint64_t total_chunks = (uint64_t)tiles * chunks_per_tile;
    const uint64_t c_begin = (uint64_t)group * chunks_per_group;
    if (c_begin >= total_chunks) return;  // (the plan leaves no empty run)
    const uint64_t c_end = c_begin + chunks_per_group < total_chunks ? c_begin + chunks_per_group : total_chunks;
    const uint32_t t0 = (uint32_t)(c_begin / chunks_per_tile), s0 = (uint32_t)(c_begin % chunks_per_tile);

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const uint32_t n = lane & 31, h = lane >> 5;
    const uint32_t col0 = cb * kColsPerWG + wave * (GPW * 32) + n;

    {
        const uint32_t plus = kBf ? 0x3F80u : 0x3C00u;
        for (int idx = tid; idx < 256 * kSignCopies; idx += 64 * W) {
            const uint32_t e = (uint32_t)idx / kSignCopies;
            uint32_t v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = plus | (((e >> i) & 1u) ? 0u : 0x8000u);
            *reinterpret_cast<uint4*>(smem + idx * 16) =
                uint4{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
        }
    }

    floatx16 acc[RB][GPW];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int j = 0; j < GPW; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][j][r] = 0.0f;

    const Elem* g = reinterpret_cast<const Elem*>(g_in);
    const uint32_t a_off = n * kLdsRow + 128 * h;  // row block rb: + 32 rb rows
    const uint32_t lane_base = (uint32_t)(lane & 15) << 4;

    // Position of a chunk of the run: tile, chunk in tile, first feature, end of the tile's features and
    // the number of chunks of the tile that lie wholly below that end.  Uniform values (scalar registers)
    // that move from chunk to chunk with a few additions: the 64-bit products are redone only when the
    // tile changes.  Every scalar instruction between the last MFMA of a chunk and the first of the next
    // is paid for with about eight idle cycles of the matrix pipe (all waves are there at the same time).
    struct Cursor {
        uint32_t tile, s, whole;
        uint64_t f, hi;
    };
    auto open_tile = [&](Cursor& c) {
        const uint64_t lo = (uint64_t)c.tile * tile_size;
        c.hi = (lo + tile_size < P) ? lo + tile_size : P;  // may be <= lo (loads give zeros)
        c.whole = c.hi > lo ? (uint32_t)((c.hi - lo) / kChunk) : 0u;
        c.f = lo + (uint64_t)c.s * kChunk;
    };
    auto advance = [&](Cursor& c) {
        if (++c.s == chunks_per_tile) {
            c.s = 0;
            ++c.tile;
            open_tile(c);
        } else {
            c.f += kChunk;
        }
    };
    const bool full_rows = rows == 32u * RB;
    Stage st;
    UniformSeg useg = {0u, 0u, 0u, 0u, nullptr};  // GATHER, 16-bit gradients
    auto load_chunk = [&](const Cursor& c) {
        if constexpr (!GATHER && kPlanes == 1) {
            if (full_rows && c.s < c.whole)
                st.load_whole(g, ld, c.f, tid);
            else
                st.load_edge(g, ld, rows, c.f, c.hi, tid);
        } else if constexpr (GATHER && kPlanes == 1) {
            const uint32_t f32 = (uint32_t)c.f;  // P < 2^32 with segments; beyond P: c.whole is 0
            useg.advance(g, (uint32_t)ld, f32, tid, 2 * W);
            if (full_rows && c.s < c.whole && f32 >= useg.first && f32 + (uint32_t)kChunk <= useg.end)
                st.load_pieces(useg.tbase + 2 * (uint64_t)f32, useg.piece_pitch);
            else  // chunks that cross a segment or tile end: per-thread cursors, set up for this chunk only
                st.load_from(g, (uint32_t)ld, useg.idx, rows, c.f, c.hi, tid);
        } else {
            st.load(g, ld, rows, c.f, c.hi, tid);
        }
    };
    const uint32_t n_chunks = (uint32_t)(c_end - c_begin);

    // Two LDS buffers (16-bit gradients): the chunk loop is one uninterrupted stream of steps.  Chunk
    // i + 1 is stored to the other buffer in the middle of chunk i (it was loaded in the middle of chunk
    // i - 1: one chunk time, about 2 us, in flight), the loads of chunk i + 2 follow the store into the
    // same registers, the one barrier of the chunk stands in front of the first step of its last q -
    // every wave has finished reading the current buffer by then, and the other one is published for the
    // operand reads of the next chunk, which start right there: the rings of A and B operands run on
    // across the chunk boundary.  One buffer (fp32 gradients): store between two barriers at the top of
    // the chunk, the rings start anew.
    constexpr bool kRing = kBuffers == 2;
    constexpr int kSyncStep = 15 * GPW;
    constexpr int kStoreStep = 10 * GPW, kLoadStep = kStoreStep + 1;
    Cursor nx = {t0, s0, 0u, 0u, 0u};  // the chunk after the current one (tile and s: its generator blocks)
    open_tile(nx);
    Cursor ld2 = nx;                   // kRing: the chunk after that (the next one to load)
    if constexpr (GATHER) {
        if constexpr (kPlanes == 1)
            useg.seek(g, (uint32_t)ld, (uint32_t)(nx.f < P ? nx.f : P - 1), tid, 2 * W);
        else
            st.init(g, (uint32_t)ld, nx.f, P, tid);
    }
    load_chunk(nx);
    advance(nx);
    if (kRing) {
        st.store(lds, tid);
        if (n_chunks > 1) load_chunk(nx);
        ld2 = nx;
        advance(ld2);
    }
    __syncthreads();  // publishes the table (and the first chunk)

    // the first two words of a block are bytes 0..7 = MFMA steps q = 0..7, the other two q = 8..15
    uint32_t wd[GPW][4];
#pragma unroll
    for (int j = 0; j < GPW; ++j) {
        const jl::u32x4 w = jl::stream_block(seed, jl::stream_name(seed, col0 + 32u * j, t0), 2u * s0 + h);
        wd[j][0] = w.x, wd[j][1] = w.y, wd[j][2] = w.z, wd[j][3] = w.w;
    }

    uint4 bq[kAhead + 1];       // B operands (sign look-ups), read kAhead steps ahead
    uint4 a[2][RB][kPlanes];    // A operands of this q and of the next one (read one q ahead)
    auto read_a = [&](const uint16_t* base, int slot, int q) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int pl = 0; pl < kPlanes; ++pl)
                a[slot][rb][pl] = *reinterpret_cast<const uint4*>(base + rb * 32 * kLdsRow + pl * kPlaneElems + 8 * q);
    };
    auto lookup = [&](uint32_t word, int q) -> uint4 {
        return *reinterpret_cast<const uint4*>(smem + sign_entry_address(word, q, lane_base));
    };
    if (kRing) {
#pragma unroll
        for (int p = 0; p < kAhead; ++p) bq[p] = lookup(wd[p % GPW][0], p / GPW);
        read_a(lds + a_off, 0, 0);
    }

    // chunk number i of the run; cur_c: its LDS buffer (a constant: immediate offsets in the DS instructions)
    auto chunk = [&](uint32_t i, auto cur_c) __attribute__((always_inline)) {
        constexpr int kCur = decltype(cur_c)::value;
        if (!kRing) {
            __syncthreads();  // everyone is done reading the previous chunk
            st.store(lds, tid);
            __syncthreads();
            if (i + 1 < n_chunks) load_chunk(nx);
        }
        const uint16_t* a_base = lds + kCur * kBufElems + a_off;
        const uint16_t* a_next = lds + (kCur ^ 1) * kBufElems + a_off;

        // The next chunk's blocks: first round now - its counter is (block, stream name, 0, 0) and
        // the block number is the same for the GPW groups, so it is one multiply for all of them
        // and one xor per group - the other nine under the MFMAs below.
        jl::u32x4 pc[GPW], pn[GPW];
        {
            const uint64_t q0 = (uint64_t)jl::kPhiloxM0 * (2u * nx.s + h);
#pragma unroll
            for (int j = 0; j < GPW; ++j) {
                pc[j].x = jl::stream_name(seed, col0 + 32u * j, nx.tile) ^ seed;
                pc[j].y = 0u;
                pc[j].z = (uint32_t)(q0 >> 32);
                pc[j].w = (uint32_t)q0;
            }
        }

        if (!kRing) {
#pragma unroll
            for (int p = 0; p < kAhead; ++p) bq[p] = lookup(wd[p % GPW][(p / GPW) >> 2], p / GPW);
            read_a(a_base, 0, 0);
        }
        // one step; the step number is a constant (the steps are written out through for_each_step, which
        // does not depend on the optimizer's unrolling limits)
        auto do_step = [&](auto step_c) __attribute__((always_inline)) {
            {
                constexpr int step = decltype(step_c)::value;
                constexpr int q = step / GPW, j = step % GPW;
                if constexpr (kRing && step == kSyncStep) __syncthreads();
                // half rounds number first .. first + count - 1 of the kHalfRounds; number
                // i is half i % 2 of round 1 + i / (2 GPW) of group (i / 2) % GPW.  They are
                // spread over the first kSpan steps, one per step and two in every kEvery-th:
                // group g's block must be complete when its first look-up for the next chunk
                // is issued, kAhead steps before the end.
                constexpr int kSpan = GPW == 4 ? kSteps : kSteps - 4;
                constexpr int kExtra = kHalfRounds - kSpan;        // steps that take two
                constexpr int kEvery = kSpan / kExtra;
                static_assert(kExtra * kEvery <= kSpan, "half-round schedule");
                constexpr int twos = (step + kEvery - 1) / kEvery;     // steps < step that took two
                constexpr int first = step + (twos < kExtra ? twos : kExtra);
                constexpr int count = step >= kSpan ? 0 : (step % kEvery == 0 && step / kEvery < kExtra) ? 2 : 1;
                PhiloxHalfIn hin0 = {0u, 0u}, hin1 = {0u, 0u};
                if constexpr (count >= 1) hin0 = philox_half_in(pc[(first / 2) % GPW], first % 2);
                if constexpr (count == 2) hin1 = philox_half_in(pc[((first + 1) / 2) % GPW], (first + 1) % 2);
                {
                    constexpr int t = step + kAhead;  // the look-up issued now; beyond this chunk: the next one's
                    if constexpr (t < kSteps)
                        bq[t % (kAhead + 1)] = lookup(wd[t % GPW][(t / GPW) >> 2], t / GPW);
                    else if constexpr (kRing)
                        bq[t % (kAhead + 1)] = lookup(pc[(t - kSteps) % GPW].x, (t - kSteps) / GPW);
                }
                if constexpr (j == 0) {
                    if constexpr (q + 1 < 16)
                        read_a(a_base, (q + 1) & 1, q + 1);
                    else if constexpr (kRing)
                        read_a(a_next, 0, 0);
                }
                auto half_out = [&](const PhiloxHalfIn& in, int u) {
                    const int r = 1 + u / (2 * GPW), g4 = (u / 2) % GPW;
                    philox_half_out(in, pn[g4], u % 2, seed + (uint32_t)r * jl::kPhiloxW0, (uint32_t)r * jl::kPhiloxW1);
                };
                if constexpr (count >= 1) half_out(hin0, first);
                if constexpr (count == 2) half_out(hin1, first + 1);
#pragma unroll
                for (int u = first; u < first + count; ++u)
                    if (u % 2 == 1) pc[(u / 2) % GPW] = pn[(u / 2) % GPW];
                if constexpr (kRing && step == kStoreStep) {
                    if (i + 1 < n_chunks) st.store(lds + (kCur ^ 1) * kBufElems, tid);
                }
                if constexpr (kRing && step == kLoadStep) {
                    if (i + 2 < n_chunks) load_chunk(ld2);
                    nx.tile = ld2.tile;
                    nx.s = ld2.s;
                    advance(ld2);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                    for (int pl = 0; pl < kPlanes; ++pl)
                        acc[rb][j] = mfma16(a[q & 1][rb][pl], bq[step % (kAhead + 1)], acc[rb][j], kBf);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        for_each_step(do_step, std::make_integer_sequence<int, kSteps>{});
#pragma unroll
        for (int j = 0; j < GPW; ++j) wd[j][0] = pc[j].x, wd[j][1] = pc[j].y, wd[j][2] = pc[j].z, wd[j][3] = pc[j].w;
        if (!kRing) advance(nx);
    };
    for (uint32_t i = 0; i < n_chunks; i += 2) {
        chunk(i, std::integral_constant<int, 0>{});
        if (i + 1 < n_chunks) chunk(i + 1, std::integral_constant<int, kRing ? 1 : 0>{});
    }

    // D[m][n] of a 32x32 MFMA: lane holds column n = lane % 32 and, in register r, row
    // m = 8*(r/4) + 4*(lane/32) + r%4.
    float* out = partial + (uint64_t)group * rows * k;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int j = 0; j < GPW; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = 32u * rb + 8u * (r >> 2) + 4u * h + (r & 3);
                if (m < rows) out[(uint64_t)m * k + col0 + 32u * j] = acc[rb][j][r];
            }
        }
    }
}

// ---- normal (Gaussian) projection ------------------------------------------------------------
//
// Same decomposition as the Rademacher kernel (8 waves, 32-column groups, 256-feature chunks,
// lane half h owns features [128h, 128h + 128) of a chunk), but the cost sits elsewhere: a matrix
// entry is used for 32 multiply-adds only, and making one costs about ten vector instructions
// (Philox4x32-10: one block per eight entries) against 1.5 for a sign, so the kernel is bound by
// the vector ALU, not by the matrix pipe.  What keeps the count that low:
//   * one random word makes a whole Box-Muller pair: the radius R[x] and the signed pair
//     (C[a], S[a]) come out of two LDS tables (32 KB + 64 KB, filled at kernel start from the
//     binary32 sequences of jl_stream.h), each addressed by ONE instruction (the fields of the
//     word sit so that a masked 16-bit half of it is the byte offset), and one v_pk_mul_f16
//     multiplies and rounds both entries: three vector instructions per pair;
//   * the matrix entries are fp16 whatever the gradient type is, so the gradients are brought to
//     fp16 once per chunk at staging time instead of splitting every entry into bf16 terms in the
//     hot loop: bf16 and fp32 chunks are multiplied row by row by the power of two that puts the
//     largest magnitude the row has shown so far into [2^14, 2^15) (bf16: one exact fp16 plane for
//     everything within 2^-31 of it; fp32: two planes h1 + h2, 22 significant bits), the
//     accumulators are scaled down when that maximum grows (v_ldexp_f32, exact) and the factor is
//     taken out again before the partial sums are written.

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));

constexpr int kRadiusEntries = 1 << jl::kRadiusBits;
constexpr int kAngleEntries = 1 << jl::kAngleBits;
#ifndef JL_NORMAL_UNROLL
#define JL_NORMAL_UNROLL 1
#endif
constexpr int kNormalUnroll = JL_NORMAL_UNROLL;  // MFMA steps of the hot loop unrolled together

template <int IN>
struct NormalTraits;
template <>
struct NormalTraits<TRAKHIP_F16> {
    static constexpr int planes = 1, buffers = 2;
    static constexpr bool scaled = false;
};
template <>
struct NormalTraits<TRAKHIP_BF16> {
    static constexpr int planes = 1, buffers = 2;
    static constexpr bool scaled = true;
};
template <>
struct NormalTraits<TRAKHIP_F32> {
    static constexpr int planes = 2, buffers = 1;  // x * 2^sh = h1 + h2 (+ at most 2^-22 of it)
    static constexpr bool scaled = true;
};

// Power of two that brings a row whose largest binary32 exponent field is emax into [2^14, 2^15).
// A row keeps ONE reference exponent that only ever moves towards larger magnitudes: the smallest
// such power over the chunks seen so far (kNoScale until the first chunk that is not all zero).  A
// chunk is converted with the reference, so whatever it holds below 2^-38 of the row's running
// maximum rounds away (it could not change the row's result beyond 2^-38 of its size), and the
// accumulators are only ever scaled down when the reference moves - they cannot overflow.
constexpr int kNoScale = 1 << 20;
struct RowScale {
    int use;    // exponent applied to this chunk
    int delta;  // change against the exponent the accumulators carry (<= 0)
};
__device__ __forceinline__ RowScale next_row_scale(uint32_t emax, int& ref) {
    const int want = emax ? 141 - (int)emax : kNoScale;
    const int prev = ref;
    ref = want < ref ? want : ref;
    RowScale r;
    r.use = ref == kNoScale ? 0 : ref;
    r.delta = prev == kNoScale ? 0 : r.use - prev;
    return r;
}

// Slot of row m in the per-chunk exponent lists: lane half h reads its sixteen accumulator rows
// m = 8*(r/4) + 4*h + r%4 (r = 0..15) as sixteen consecutive ints.
__device__ __forceinline__ int row_slot(uint32_t row) {
    return (int)(row & ~31u) + ((row >> 2) & 1) * 16 + ((row & 31u) >> 3) * 4 + (row & 3);  // 32-row blocks one after another
}

__device__ __forceinline__ uint32_t pack_f16_rne(float a, float b) {
    const half2_t v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, v);
}

// bf16 chunk -> one scaled fp16 plane.  The 32 threads that share tid / 32 hold one row (N rows
// per thread, 2 W apart for a workgroup of W waves); sh_ref[] is the row's reference exponent so far;
// sh_delta / sh_use are the per-row lists of this buffer (2 W N entries each).
template <int W, int N>
__device__ __forceinline__ void store_scaled_bf16(const uint4 (&v)[N], uint16_t* lds, int* sh_delta, int* sh_use,
                                                  int tid, int (&sh_ref)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const uint32_t row = (tid >> 5) + 2 * W * i, sg = tid & 31;
        const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
        ushort2_t m = __builtin_bit_cast(ushort2_t, w[0] & 0x7F807F80u);
#pragma unroll
        for (int t = 1; t < 4; ++t) m = __builtin_elementwise_max(m, __builtin_bit_cast(ushort2_t, w[t] & 0x7F807F80u));
        uint32_t e = m[0] > m[1] ? m[0] : m[1];
#pragma unroll
        for (int d = 1; d < 32; d <<= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)e, d, 64);
            e = o > e ? o : e;
        }
        const RowScale rs = next_row_scale(e >> 7, sh_ref[i]);
        uint32_t h[4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
            h[t] = pack_f16_rne(ldexpf(__uint_as_float(w[t] << 16), rs.use),
                                ldexpf(__uint_as_float(w[t] & 0xFFFF0000u), rs.use));
        *reinterpret_cast<uint4*>(lds + row * kLdsRow + 8 * sg) = uint4{h[0], h[1], h[2], h[3]};
        if (sg == 0) {
            sh_delta[row_slot(row)] = rs.delta;
            sh_use[row_slot(row)] = rs.use;
        }
    }
}

// fp32 chunk -> two scaled fp16 planes.  The 64 threads of a wave hold one row (N = 32 / W rows per
// thread, W apart).
template <int W, int N>
__device__ __forceinline__ void store_scaled_f32(const uint4 (&v)[N], uint16_t* lds, int* sh_delta, int* sh_use, int tid,
                                                 int (&sh_ref)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const uint32_t row = (tid >> 6) + W * i, sg = tid & 63;
        const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
        uint32_t e = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t x = (w[t] >> 23) & 0xFFu;
            e = x > e ? x : e;
        }
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)e, d, 64);
            e = o > e ? o : e;
        }
        const RowScale rs = next_row_scale(e, sh_ref[i]);
        float g[4], r[4];
        _Float16 h1[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            g[t] = ldexpf(__uint_as_float(w[t]), rs.use);
            h1[t] = (_Float16)g[t];
            r[t] = g[t] - (float)h1[t];  // exact
        }
        const half2_t a0 = {h1[0], h1[1]}, a1 = {h1[2], h1[3]};
        *reinterpret_cast<uint2*>(lds + row * kLdsRow + 4 * sg) =
            uint2{__builtin_bit_cast(uint32_t, a0), __builtin_bit_cast(uint32_t, a1)};
        *reinterpret_cast<uint2*>(lds + kPlaneElems + row * kLdsRow + 4 * sg) =
            uint2{pack_f16_rne(r[0], r[1]), pack_f16_rne(r[2], r[3])};
        if (sg == 0) {
            sh_delta[row_slot(row)] = rs.delta;
            sh_use[row_slot(row)] = rs.use;
        }
    }
}

// The Box-Muller pair of one random word as packed fp16 (cosine entry low, sine entry high):
// fields of the word as in jl_stream.h (radius index bits 17..30, angle index bits 2..15).  r_tab
// holds fp16 R[x], cs_tab the packed signed fp16 pairs (C[a], S[a]).  Each byte offset is one
// instruction: the upper half of the word under the mask 0x7FFE (v_and_b32 with a 16-bit sub-word
// select), the lower half under 0xFFFC.
__device__ __forceinline__ uint32_t normal_pair(uint32_t w, const char* r_tab, const char* cs_tab) {
    const _Float16 r = *reinterpret_cast<const _Float16*>(r_tab + ((w >> 16) & 0x7FFEu));
    const uint32_t cs = *reinterpret_cast<const uint32_t*>(cs_tab + (w & 0xFFFCu));
    const half2_t rr = {r, r};
    const half2_t z = rr * __builtin_bit_cast(half2_t, cs);  // v_pk_mul_f16: exact products, rounded once
    return __builtin_bit_cast(uint32_t, z);
}

// GPW = 32-column groups per wave: 4 (workgroup = 1024 columns) or 2 (512 columns, for projection
// dimensions that are an odd multiple of 512).  RB = 32-row blocks per pass: 2 for fp16 / bf16 gradients
// when the batch has more than 32 rows - every generated entry then feeds two MFMAs, which is worth
// almost a factor of two to a kernel bound by the cost of making an entry (one LDS buffer then: two
// do not fit next to the tables).  Always 8 waves; arguments as jl_project_kernel.
template <int IN, bool GATHER, int GPW, int RB, int W>
__global__ __launch_bounds__(64 * W) void jl_project_normal_kernel(
    const void* __restrict__ g_in, uint64_t ld, uint32_t rows, uint64_t P, uint32_t k, uint32_t seed,
    uint32_t tiles, uint64_t tile_size, uint32_t chunks_per_tile, uint32_t chunks_per_group, uint32_t groups,
    float* __restrict__ partial) {
    typedef NormalTraits<IN> Tr;
    typedef typename StageOf<IN, GATHER, W, 32 * RB>::type Stage;
    typedef typename StageOf<IN, GATHER, W, 32 * RB>::elem Elem;
    constexpr int kColsPerWG = W * GPW * 32;
    constexpr int kPlanes = Tr::planes;
    static_assert(RB == 1 || kPlanes == 1, "two row blocks: 16-bit gradients only (LDS)");
    constexpr int kBuffers = RB == 2 ? 1 : Tr::buffers;
    constexpr int kPlaneElems = RB * kPlaneElems32;  // this kernel's plane: 32 RB rows
    constexpr int kBufElems = kPlanes * kPlaneElems;
    constexpr bool kScaled = Tr::scaled;
    constexpr int kRows = 32 * RB;

    // One LDS block, tables first: a DS instruction adds a 16-bit immediate to the address register,
    // so a table that starts below 64 KB is indexed without an extra addition per lookup (the radii
    // at 0, the pairs at 32 KB).
    constexpr int kCsBytes = kAngleEntries * 4, kRBytes = kRadiusEntries * 2;
    static_assert(kRBytes < 65536, "the pair table must start below 64 KB");
    constexpr int kStageBytes = kBuffers * kBufElems * 2;
    __shared__ __attribute__((aligned(16))) char smem[kCsBytes + kRBytes + kStageBytes + kBuffers * 2 * kRows * 4];
    uint16_t* r_tab = reinterpret_cast<uint16_t*>(smem);
    uint32_t* cs_tab = reinterpret_cast<uint32_t*>(smem + kRBytes);
    uint16_t* lds = reinterpret_cast<uint16_t*>(smem + kCsBytes + kRBytes);
    // per buffer and row: change of the row's exponent against the previous chunk, and the exponent
    int (*sh_lds)[2][kRows] = reinterpret_cast<int (*)[2][kRows]>(smem + kCsBytes + kRBytes + kStageBytes);

    const uint32_t col_blocks = k / kColsPerWG;
    uint32_t cb, group;
    if (!map_workgroup(blockIdx.x, col_blocks, groups, cb, group)) return;
    const uint64_t total_chunks = (uint64_t)tiles * chunks_per_tile;
    const uint64_t c_begin = (uint64_t)group * chunks_per_group;
    if (c_begin >= total_chunks) return;  // (the plan leaves no empty run)
    const uint64_t c_end = c_begin + chunks_per_group < total_chunks ? c_begin + chunks_per_group : total_chunks;
    const uint32_t t0 = (uint32_t)(c_begin / chunks_per_tile), s0 = (uint32_t)(c_begin % chunks_per_tile);
    const uint32_t t_last = (uint32_t)((c_end - 1) / chunks_per_tile);
    const uint32_t s_last_end = (uint32_t)((c_end - 1) % chunks_per_tile) + 1;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const uint32_t n = lane & 31, h = lane >> 5;
    const uint32_t col0 = cb * kColsPerWG + wave * (GPW * 32) + n;

    // the two tables; the first barrier below publishes them
    for (int i = tid; i < kRadiusEntries; i += 64 * W) r_tab[i] = jl::f32_to_f16_rne(jl::bm_radius((uint32_t)i));
    for (int i = tid; i < kAngleEntries; i += 64 * W) {
        float c, sn;
        jl::bm_cossin((uint32_t)i, &c, &sn);
        cs_tab[i] = (uint32_t)jl::f32_to_f16_rne(c) | ((uint32_t)jl::f32_to_f16_rne(sn) << 16);
    }
    const char* rt = reinterpret_cast<const char*>(r_tab);
    const char* ct = reinterpret_cast<const char*>(cs_tab);

    floatx16 acc[RB][GPW];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int j = 0; j < GPW; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][j][r] = 0.0f;

    const Elem* g = reinterpret_cast<const Elem*>(g_in);
    const uint32_t a_off = n * kLdsRow + 128 * h;  // row block rb: + 32 rb rows

    Stage st;
    int sh_ref[Stage::N];
#pragma unroll
    for (int i = 0; i < Stage::N; ++i) sh_ref[i] = kNoScale;
    auto stage_store = [&](int buf) {
        if constexpr (IN == TRAKHIP_F16)
            st.store(lds + buf * kBufElems, tid);
        else if constexpr (IN == TRAKHIP_BF16)
            store_scaled_bf16<W>(st.v, lds + buf * kBufElems, sh_lds[buf][0], sh_lds[buf][1], tid, sh_ref);
        else
            store_scaled_f32<W>(st.v, lds + buf * kBufElems, sh_lds[buf][0], sh_lds[buf][1], tid, sh_ref);
    };
    {
        const uint64_t lo = (uint64_t)t0 * tile_size;
        const uint64_t hi = (lo + tile_size < P) ? lo + tile_size : P;
        if constexpr (GATHER) st.init(g, (uint32_t)ld, lo + (uint64_t)s0 * kChunk, P, tid);
        st.load(g, ld, rows, lo + (uint64_t)s0 * kChunk, hi, tid);
    }
    int cur = 0, last = 0;
    if (kBuffers == 2) {
        stage_store(0);
        __syncthreads();
    }

    for (uint32_t tile = t0; tile <= t_last; ++tile) {
        const uint64_t f_lo = (uint64_t)tile * tile_size;
        const uint64_t f_hi = (f_lo + tile_size < P) ? f_lo + tile_size : P;
        const uint32_t s_begin = tile == t0 ? s0 : 0u;
        const uint32_t chunks = tile == t_last ? s_last_end : chunks_per_tile;
        const uint64_t nf_lo = f_lo + tile_size;
        const uint64_t nf_hi = (nf_lo + tile_size < P) ? nf_lo + tile_size : P;

        uint32_t sname[GPW];
#pragma unroll
        for (int j = 0; j < GPW; ++j) sname[j] = jl::stream_name(seed, col0 + 32u * j, tile);

        for (uint32_t s = s_begin; s < chunks; ++s) {
            const bool more_here = s + 1 < chunks;
            const bool more = more_here || tile < t_last;
            if (kBuffers == 1) {
                __syncthreads();  // everyone is done reading the previous chunk
                stage_store(0);
                __syncthreads();
            }
            if (more)
                st.load(g, ld, rows, more_here ? f_lo + (uint64_t)(s + 1) * kChunk : nf_lo, more_here ? f_hi : nf_hi,
                        tid);
            const uint16_t* a_base = lds + cur * kBufElems + a_off;

            if (kScaled) {
                // rows whose reference exponent moved with this chunk: bring their sums along (down only)
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const int4* dp = reinterpret_cast<const int4*>(&sh_lds[cur][0][32 * rb + 16 * h]);
                    int d[16];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int4 x = dp[t];
                        d[4 * t] = x.x, d[4 * t + 1] = x.y, d[4 * t + 2] = x.z, d[4 * t + 3] = x.w;
                    }
#pragma unroll
                    for (int j = 0; j < GPW; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[rb][j][r] = ldexpf(acc[rb][j][r], d[r]);
                }
            }

            // Philox block of (column, offset o): o / 8 with o = 256 s + 128 h + 8 q
            const uint32_t n0 = 32u * s + 16u * h;
#pragma unroll kNormalUnroll
            for (int q = 0; q < 16; ++q) {
                uint4 a[RB][kPlanes];
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                    for (int pl = 0; pl < kPlanes; ++pl)
                        a[rb][pl] = *reinterpret_cast<const uint4*>(a_base + rb * 32 * kLdsRow + pl * kPlaneElems + 8 * q);
#pragma unroll
                for (int j = 0; j < GPW; ++j) {
                    const jl::u32x4 blk = jl::stream_block(seed, sname[j], n0 + (uint32_t)q);
                    const uint4 b = {normal_pair(blk.x, rt, ct), normal_pair(blk.y, rt, ct),
                                     normal_pair(blk.z, rt, ct), normal_pair(blk.w, rt, ct)};
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                        for (int pl = 0; pl < kPlanes; ++pl) acc[rb][j] = mfma16(a[rb][pl], b, acc[rb][j], false);
                }
            }

            last = cur;
            if (kBuffers == 2) {
                if (more) stage_store(cur ^ 1);
                __syncthreads();
                cur ^= 1;
            }
        }
    }

    float* out = partial + (uint64_t)group * rows * k;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        int ex[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) ex[r] = 0;
        if (kScaled) {
            const int4* ep = reinterpret_cast<const int4*>(&sh_lds[last][1][32 * rb + 16 * h]);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int4 x = ep[t];
                ex[4 * t] = x.x, ex[4 * t + 1] = x.y, ex[4 * t + 2] = x.z, ex[4 * t + 3] = x.w;
            }
        }
#pragma unroll
        for (int j = 0; j < GPW; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = 32u * rb + 8u * (r >> 2) + 4u * h + (r & 3);
                if (m < rows)
                    out[(uint64_t)m * k + col0 + 32u * j] = kScaled ? ldexpf(acc[rb][j][r], -ex[r]) : acc[rb][j][r];
            }
        }
    }
}

// out[b, c] = scale * sum over the runs (tile groups) of their partial sums, in a fixed order: eight
// running sums over the runs g = u (mod 8), each in increasing g, combined as
// ((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7)) - the result depends on the shape only.
// Eight neighbouring lanes share one output quad (four consecutive columns of a row), lane u holding
// s_u: a launch has 8 * B * k / 4 threads (with one thread per quad the CPU-runnable configuration had
// eight workgroups on 256 CUs and took 20 us for 8 MB).  kReduceThreads = 64: one wave per workgroup.
constexpr int kReduceThreads = 64;
template <int OUT_DTYPE>
__global__ __launch_bounds__(kReduceThreads) void jl_reduce_kernel(const float* __restrict__ partial,
                                                                   uint32_t groups, uint64_t n4, uint32_t k4,
                                                                   float scale, void* __restrict__ out,
                                                                   uint64_t ld_out) {
    const uint64_t t = (uint64_t)blockIdx.x * kReduceThreads + threadIdx.x;
    const uint64_t i = t >> 3;  // n4 is a multiple of 128 (k of 512): every wave is full
    const uint32_t u = (uint32_t)t & 7u;
    if (i >= n4) return;
    const float4* p = reinterpret_cast<const float4*>(partial) + i;
    float4 s = {0.f, 0.f, 0.f, 0.f};
    uint32_t g = u;
    for (; g + 56 < groups; g += 64) {  // eight loads in flight
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p[(uint64_t)(g + 8 * j) * n4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            s.x += v[j].x;
            s.y += v[j].y;
            s.z += v[j].z;
            s.w += v[j].w;
        }
    }
    {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (g + 8 * j < groups) ? p[(uint64_t)(g + 8 * j) * n4] : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (g + 8 * j < groups) {
                s.x += v[j].x;
                s.y += v[j].y;
                s.z += v[j].z;
                s.w += v[j].w;
            }
        }
    }
    // lane 0 of each eight ends up with the sum in the order stated above (own value first in every step)
#pragma unroll
    for (int d = 1; d < 8; d <<= 1) {
        s.x += __shfl_xor(s.x, d, 64);
        s.y += __shfl_xor(s.y, d, 64);
        s.z += __shfl_xor(s.z, d, 64);
        s.w += __shfl_xor(s.w, d, 64);
    }
    if (u != 0) return;
    float4 r = s;
    r.x *= scale;
    r.y *= scale;
    r.z *= scale;
    r.w *= scale;
    // row pitch of the destination in elements; the result is rounded to fp32 first (as a
    // separate `x *= scale`), then to the store type
    const uint64_t row = i / k4, c4 = i - row * k4;
    const uint64_t e = row * ld_out + c4 * 4;
    store4<OUT_DTYPE>(static_cast<char*>(out) + e * trakhip::out_elem_size(OUT_DTYPE), r);
}

// S[f0 + i, c0 + j] for i < nf, j < nc, written as binary32, row-major [nf, nc].
__global__ __launch_bounds__(256) void jl_materialize_kernel(uint32_t seed, uint64_t tile_size, uint64_t f0,
                                                             uint64_t nf, uint32_t c0, uint32_t nc,
                                                             int proj_type, float* __restrict__ out) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= nf * nc) return;
    const uint64_t f = f0 + idx / nc;
    const uint32_t c = c0 + (uint32_t)(idx % nc);
    const uint32_t tile = (uint32_t)(f / tile_size);
    const uint32_t o = (uint32_t)(f % tile_size);
    out[idx] = proj_type == TRAKHIP_RADEMACHER ? jl::entry_rademacher(seed, c, tile, o)
                                               : jl::entry_normal(seed, c, tile, o);
}

// Compute units of the current device, asked once per device.  256 (MI355X) where no device can be
// asked, so that the workspace functions still answer in a process without a GPU.
constexpr int kMaxDevices = 64;
constexpr uint32_t kDefaultCus = 256;
uint32_t device_cus() {
    static std::atomic<uint32_t> cached[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return kDefaultCus;
    uint32_t n = cached[dev].load(std::memory_order_relaxed);
    if (!n) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
            v = (int)kDefaultCus;
        n = (uint32_t)v;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// How a launch is cut into workgroups.  The (tile, chunk) pairs of all feature tiles form one
// sequence of tiles * chunks_per_tile chunks; every workgroup takes chunks_per_group consecutive
// ones (adding their products in its accumulators) for one block of 1024 columns (512 when the
// projection dimension is an odd multiple of 512).  A workgroup of these kernels has a CU to itself
// (8 waves, 99-133 KB of LDS), so the launch must not have more workgroups than the device has CUs:
// the extra ones would start when the first ones end, and the launch would take two workgroup
// lifetimes.  groups = floor(CUs / column blocks), at least 1.  The split depends on the shape and the
// device's CU count only, so results are reproducible.
struct Plan {
    jl::Tiling tl;
    uint32_t gpw, col_blocks, chunks_per_tile, chunks_per_group, groups;  // gpw: 32-column groups per wave
};

Plan make_plan(uint64_t P, uint32_t k, uint32_t num_feature_tiles) {
    Plan p;
    p.tl = jl::make_tiling(P, num_feature_tiles);
    // columns per workgroup: 1024 (four 32-column groups per wave) when that divides k, else 768 (three),
    // else 512 (two); k is a multiple of 512
    p.gpw = (k % (8 * 4 * 32) == 0) ? 4 : (k % (8 * 3 * 32) == 0) ? 3 : 2;
    p.col_blocks = k / (8 * p.gpw * 32);
    p.chunks_per_tile = (uint32_t)((p.tl.tile_size + kChunk - 1) / kChunk);
    const uint64_t total = (uint64_t)p.tl.tiles * p.chunks_per_tile;
    uint64_t groups = device_cus() / p.col_blocks;
    if (groups > total) groups = total;
    if (groups < 1) groups = 1;
    p.chunks_per_group = (uint32_t)((total + groups - 1) / groups);
    p.groups = (uint32_t)((total + p.chunks_per_group - 1) / p.chunks_per_group);
    return p;
}

// workgroups of a launch: the units rounded up to a multiple of 8 (see map_workgroup)
uint64_t plan_workgroups(const Plan& pl) { return ((uint64_t)pl.groups * pl.col_blocks + 7u) / 8u * 8u; }

template <int IN, bool GATHER, int GPW>
hipError_t launch_rademacher(const void* in, uint64_t ld, uint32_t rows, uint64_t P, uint32_t k, uint32_t seed,
                             const Plan& pl, float* partial, hipStream_t s) {
    const uint64_t wgs = plan_workgroups(pl);
    if (wgs > 0x7FFFFFFFull) return hipErrorInvalidValue;
    if (rows > 32) {
        // two 32-row blocks per pass (16-bit gradients only)
        if constexpr (IN == TRAKHIP_F32) {
            return hipErrorInvalidValue;
        } else {
            hipLaunchKernelGGL((jl_project_kernel<IN, GATHER, GPW, 2>), dim3((uint32_t)wgs), dim3(512), 0, s, in, ld, rows,
                               P, k, seed, pl.tl.tiles, pl.tl.tile_size, pl.chunks_per_tile, pl.chunks_per_group, pl.groups, partial);
        }
    } else {
        hipLaunchKernelGGL((jl_project_kernel<IN, GATHER, GPW, 1>), dim3((uint32_t)wgs), dim3(512), 0, s, in, ld, rows, P,
                           k, seed, pl.tl.tiles, pl.tl.tile_size, pl.chunks_per_tile, pl.chunks_per_group, pl.groups, partial);
    }
    return hipGetLastError();
}

#ifndef JL_NORMAL_WAVES
#define JL_NORMAL_WAVES 16
#endif
#ifndef JL_NORMAL_WAVES_RB2
#define JL_NORMAL_WAVES_RB2 16
#endif
// The normal kernel's workgroup: kNormalWaves waves that share the plan's column block, i.e.
// 8 * GPW / kNormalWaves 32-column groups per wave (kNormalWaves2: the instance with two row blocks).
constexpr int kNormalWaves = JL_NORMAL_WAVES, kNormalWaves2 = JL_NORMAL_WAVES_RB2;

template <int IN, bool GATHER, int GPW>
hipError_t launch_normal(const void* in, uint64_t ld, uint32_t rows, uint64_t P, uint32_t k, uint32_t seed,
                         const Plan& pl, float* partial, hipStream_t s) {
    // same columns per workgroup as the plan's 8 waves x GPW groups; an odd GPW keeps 8 waves
    constexpr int W = (8 * GPW) % kNormalWaves == 0 ? kNormalWaves : 8, G = 8 * GPW / W;
    constexpr int W2 = (8 * GPW) % kNormalWaves2 == 0 ? kNormalWaves2 : 8, G2 = 8 * GPW / W2;
    static_assert(G >= 1 && G * W == 8 * GPW && G2 >= 1 && G2 * W2 == 8 * GPW, "column groups per wave");
    const uint64_t wgs = plan_workgroups(pl);
    if (wgs > 0x7FFFFFFFull) return hipErrorInvalidValue;
    if (rows > 32) {
        if constexpr (IN == TRAKHIP_F32) {
            return hipErrorInvalidValue;
        } else {
            hipLaunchKernelGGL((jl_project_normal_kernel<IN, GATHER, G2, 2, W2>), dim3((uint32_t)wgs), dim3(64 * W2), 0, s, in,
                               ld, rows, P, k, seed, pl.tl.tiles, pl.tl.tile_size, pl.chunks_per_tile,
                               pl.chunks_per_group, pl.groups, partial);
        }
    } else {
        hipLaunchKernelGGL((jl_project_normal_kernel<IN, GATHER, G, 1, W>), dim3((uint32_t)wgs), dim3(64 * W), 0, s, in, ld,
                           rows, P, k, seed, pl.tl.tiles, pl.tl.tile_size, pl.chunks_per_tile, pl.chunks_per_group,
                           pl.groups, partial);
    }
    return hipGetLastError();
}

typedef hipError_t (*LaunchFn)(const void*, uint64_t, uint32_t, uint64_t, uint32_t, uint32_t,
                               const Plan&, float*, hipStream_t);

template <int W>  // 32-column groups per wave
LaunchFn pick_w(int dtype, int proj_type, bool gather) {
    static const LaunchFn table[2][3][2] = {
        {{launch_rademacher<TRAKHIP_F16, false, W>, launch_normal<TRAKHIP_F16, false, W>},
         {launch_rademacher<TRAKHIP_BF16, false, W>, launch_normal<TRAKHIP_BF16, false, W>},
         {launch_rademacher<TRAKHIP_F32, false, W>, launch_normal<TRAKHIP_F32, false, W>}},
        {{launch_rademacher<TRAKHIP_F16, true, W>, launch_normal<TRAKHIP_F16, true, W>},
         {launch_rademacher<TRAKHIP_BF16, true, W>, launch_normal<TRAKHIP_BF16, true, W>},
         {launch_rademacher<TRAKHIP_F32, true, W>, launch_normal<TRAKHIP_F32, true, W>}},
    };
    return table[gather ? 1 : 0][dtype][proj_type];
}

LaunchFn pick(const Plan& pl, int dtype, int proj_type, bool gather) {
    return pl.gpw == 4   ? pick_w<4>(dtype, proj_type, gather)
           : pl.gpw == 3 ? pick_w<3>(dtype, proj_type, gather)
                         : pick_w<2>(dtype, proj_type, gather);
}

}  // namespace

// Scratch of trakhip_project_static (see project_static below): 36 MiB, enough for every shape with
// proj_dim <= 65536.
constexpr size_t kStaticScratchBytes = 36u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void*> static_scratch_ptr[kMaxDevices];

namespace trakhip {

// Rows of one pass of the projection kernels: 16-bit gradients go 64 rows at a time (two 32-row MFMA
// blocks share every generated operand), fp32 gradients 32 (their planes do not fit twice in LDS).
uint32_t project_rows_per_pass(int dtype, int proj_type) {
    (void)proj_type;
    return dtype == TRAKHIP_F16 || dtype == TRAKHIP_BF16 ? 64u : 32u;
}

static size_t workspace_for_rows(uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles, uint64_t pass_rows) {
    if (B == 0 || P == 0 || k == 0 || num_feature_tiles == 0) return 0;
    if (k % kColsMultiple != 0 || P > 0xFFFFFFFFull) return 0;
    const Plan pl = make_plan(P, k, num_feature_tiles);
    const uint64_t rows = B < pass_rows ? B : pass_rows;
    return (size_t)pl.groups * rows * k * sizeof(float);
}

// What a caller should bring: room for passes of 64 rows.  Passes of 32 rows (half of it for B >= 64) are
// the minimum every entry point accepts.
size_t project_workspace_bytes(uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles) {
    return workspace_for_rows(B, P, k, num_feature_tiles, 64);
}
size_t project_workspace_min_bytes(uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles) {
    return workspace_for_rows(B, P, k, num_feature_tiles, 32);
}

static int check_project_args(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, const void* ws,
                              size_t ws_bytes, uint32_t k, uint32_t num_feature_tiles, int proj_type) {
    if (dtype < TRAKHIP_F16 || dtype > TRAKHIP_F32) return TRAKHIP_ERR_DTYPE;
    if (proj_type != TRAKHIP_RADEMACHER && proj_type != TRAKHIP_NORMAL) return TRAKHIP_ERR_PROJ_TYPE;
    if (k == 0 || k % kColsMultiple != 0) return TRAKHIP_ERR_PROJ_DIM;
    if (B == 0 || P == 0 || P > 0xFFFFFFFFull || num_feature_tiles == 0) return TRAKHIP_ERR_SHAPE;
    if (ld < P) return TRAKHIP_ERR_SHAPE;
    if (!in || !ws) return TRAKHIP_ERR_NULL;
    if (ws_bytes < project_workspace_min_bytes(B, P, k, num_feature_tiles)) return TRAKHIP_ERR_WORKSPACE;
    const size_t esz = dtype == TRAKHIP_F32 ? 4 : 2;
    if ((reinterpret_cast<uintptr_t>(in) % esz) || (reinterpret_cast<uintptr_t>(ws) % 16)) return TRAKHIP_ERR_ALIGN;
    return TRAKHIP_OK;
}

int project_partials(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, void* ws, size_t ws_bytes,
                     uint32_t k, uint32_t seed, uint32_t num_feature_tiles, int proj_type, hipStream_t s) {
    const int e = check_project_args(in, dtype, B, P, ld, ws, ws_bytes, k, num_feature_tiles, proj_type);
    if (e) return e;
    if (B > project_rows_per_pass(dtype, proj_type)) return TRAKHIP_ERR_SHAPE;
    if (ws_bytes < workspace_for_rows(B, P, k, num_feature_tiles, 64)) return TRAKHIP_ERR_WORKSPACE;
    const Plan pl = make_plan(P, k, num_feature_tiles);
    if (pick(pl, dtype, proj_type, false)(in, ld, (uint32_t)B, P, k, seed, pl, static_cast<float*>(ws), s) != hipSuccess)
        return TRAKHIP_ERR_LAUNCH;
    return TRAKHIP_OK;
}

int project_gather_partials(const trakhip_segment* segs, uint32_t n_segs, int dtype, uint64_t B, uint64_t P,
                            void* ws, size_t ws_bytes, uint32_t k, uint32_t seed, uint32_t num_feature_tiles,
                            int proj_type, hipStream_t s) {
    // segs is device memory: its contents (sorted, contiguous, covering [0, P)) are the caller's contract
    const int e = check_project_args(segs, dtype, B, P, P, ws, ws_bytes, k, num_feature_tiles, proj_type);
    if (e) return e;
    if (B > project_rows_per_pass(dtype, proj_type) || n_segs == 0) return TRAKHIP_ERR_SHAPE;
    if (ws_bytes < workspace_for_rows(B, P, k, num_feature_tiles, 64)) return TRAKHIP_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(segs) % 8) return TRAKHIP_ERR_ALIGN;
    const Plan pl = make_plan(P, k, num_feature_tiles);
    if (pick(pl, dtype, proj_type, true)(segs, n_segs, (uint32_t)B, P, k, seed, pl, static_cast<float*>(ws), s) !=
        hipSuccess)
        return TRAKHIP_ERR_LAUNCH;
    return TRAKHIP_OK;
}

int project_reduce_store(const void* ws, uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles,
                         float scale, int out_dtype, void* out, uint64_t ld_out, hipStream_t s,
                         bool check_destination) {
    if (k == 0 || k % kColsMultiple != 0) return TRAKHIP_ERR_PROJ_DIM;
    if (B == 0 || B > 64 || P == 0 || P > 0xFFFFFFFFull || num_feature_tiles == 0 || ld_out < k)
        return TRAKHIP_ERR_SHAPE;
    if (out_dtype != TRAKHIP_F16 && out_dtype != TRAKHIP_BF16 && out_dtype != TRAKHIP_F32) return TRAKHIP_ERR_DTYPE;
    if (!ws || !out) return TRAKHIP_ERR_NULL;
    const size_t quad = 4 * out_elem_size(out_dtype);
    if ((reinterpret_cast<uintptr_t>(ws) % 16) || (reinterpret_cast<uintptr_t>(out) % quad) || (ld_out % 4))
        return TRAKHIP_ERR_ALIGN;
    if (check_destination && !kernel_can_write(out)) return TRAKHIP_ERR_POINTER;
    const uint32_t groups = make_plan(P, k, num_feature_tiles).groups;
    const uint64_t n4 = B * k / 4;
    const dim3 grid((uint32_t)((8 * n4 + kReduceThreads - 1) / kReduceThreads)), block(kReduceThreads);
    const float* part = static_cast<const float*>(ws);
    if (out_dtype == TRAKHIP_F32)
        hipLaunchKernelGGL(jl_reduce_kernel<TRAKHIP_F32>, grid, block, 0, s, part, groups, n4, k / 4, scale, out, ld_out);
    else if (out_dtype == TRAKHIP_F16)
        hipLaunchKernelGGL(jl_reduce_kernel<TRAKHIP_F16>, grid, block, 0, s, part, groups, n4, k / 4, scale, out, ld_out);
    else
        hipLaunchKernelGGL(jl_reduce_kernel<TRAKHIP_BF16>, grid, block, 0, s, part, groups, n4, k / 4, scale, out, ld_out);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

int project_reduce(const void* ws, uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles, float scale,
                   float* out, hipStream_t s) {
    if (out && reinterpret_cast<uintptr_t>(out) % 16) return TRAKHIP_ERR_ALIGN;
    return project_reduce_store(ws, B, P, k, num_feature_tiles, scale, TRAKHIP_F32, out, k, s, false);
}

int project(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, float* out, void* ws,
            size_t ws_bytes, uint32_t k, uint32_t seed, uint32_t num_feature_tiles, int proj_type,
            hipStream_t s) {
    const int e = check_project_args(in, dtype, B, P, ld, ws, ws_bytes, k, num_feature_tiles, proj_type);
    if (e) return e;
    if (!out) return TRAKHIP_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(out) % 16) return TRAKHIP_ERR_ALIGN;
    const size_t esz = dtype == TRAKHIP_F32 ? 4 : 2;
    // rows are walked 64 or 32 at a time (the reference walks 8, 16 or 32 at a time: fast_jl/fast_jl.cu:44-76);
    // a workspace sized for 32-row passes only is accepted and used that way
    uint64_t pass = project_rows_per_pass(dtype, proj_type);
    if (pass > 32 && ws_bytes < workspace_for_rows(B, P, k, num_feature_tiles, pass)) pass = 32;
    for (uint64_t b0 = 0; b0 < B; b0 += pass) {
        const uint64_t rows = (B - b0) < pass ? (B - b0) : pass;
        const char* src = static_cast<const char*>(in) + b0 * ld * esz;
        int r = project_partials(src, dtype, rows, P, ld, ws, ws_bytes, k, seed, num_feature_tiles, proj_type, s);
        if (!r) r = project_reduce(ws, rows, P, k, num_feature_tiles, 1.0f, out + b0 * k, s);
        if (r) return r;
    }
    return TRAKHIP_OK;
}

// ---- projection without any allocation ------------------------------------------------------
//
// For callers that cannot provide or allocate a workspace (code under HIP graph capture, tight
// serving loops): the partial sums go to a file-scope device array instead.  Every device the
// library runs on holds its own copy of the array, at its own address, until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress: the address that kernels
// and copies use is looked up once per device (with that device current) and kept in
// static_scratch_ptr[]; the name itself is never passed to a kernel.

size_t project_static_limit_bytes() { return kStaticScratchBytes; }

// Address of the current device's copy of `scratch` (nullptr + error code on failure).
static int static_scratch(void** ptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TRAKHIP_ERR_NO_DEVICE;
    void* p = static_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // two threads racing here look up the same address; the store is idempotent
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return TRAKHIP_ERR_NO_DEVICE;
        static_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return TRAKHIP_OK;
}

int project_static(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, float* out, uint32_t k,
                   uint32_t seed, uint32_t num_feature_tiles, int proj_type, hipStream_t s) {
    // host-only validation first (a dummy non-null, aligned workspace of unlimited size)
    const int e = check_project_args(in, dtype, B, P, ld, reinterpret_cast<const void*>(uintptr_t(256)), SIZE_MAX, k,
                                     num_feature_tiles, proj_type);
    if (e) return e;
    if (!out) return TRAKHIP_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(out) % 16) return TRAKHIP_ERR_ALIGN;
    if (project_workspace_min_bytes(B, P, k, num_feature_tiles) > kStaticScratchBytes) return TRAKHIP_ERR_STATIC_LIMIT;
    void* ws = nullptr;
    const int d = static_scratch(&ws);
    if (d) return d;
    // every partial block that the reduction reads is written by the projection kernel of the same
    // call, so nothing in the array has to start at zero
    return project(in, dtype, B, P, ld, out, ws, kStaticScratchBytes, k, seed, num_feature_tiles, proj_type, s);
}

int materialize_device(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                       uint32_t c0, uint32_t nc, int proj_type, float* out, hipStream_t s) {
    if (proj_type != TRAKHIP_RADEMACHER && proj_type != TRAKHIP_NORMAL) return TRAKHIP_ERR_PROJ_TYPE;
    if (P == 0 || P > 0xFFFFFFFFull || num_feature_tiles == 0 || f0 + nf > P) return TRAKHIP_ERR_SHAPE;
    if (nf == 0 || nc == 0) return TRAKHIP_OK;
    if (!out) return TRAKHIP_ERR_NULL;
    const jl::Tiling tl = jl::make_tiling(P, num_feature_tiles);
    const uint64_t total = nf * nc;
    if ((total + 255) / 256 > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    hipLaunchKernelGGL(jl_materialize_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, seed,
                       tl.tile_size, f0, nf, c0, nc, proj_type, out);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

int materialize_host(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                     uint32_t c0, uint32_t nc, int proj_type, float* out) {
    if (proj_type != TRAKHIP_RADEMACHER && proj_type != TRAKHIP_NORMAL) return TRAKHIP_ERR_PROJ_TYPE;
    if (P == 0 || P > 0xFFFFFFFFull || num_feature_tiles == 0 || f0 + nf > P) return TRAKHIP_ERR_SHAPE;
    if (nf == 0 || nc == 0) return TRAKHIP_OK;
    if (!out) return TRAKHIP_ERR_NULL;
    const jl::Tiling tl = jl::make_tiling(P, num_feature_tiles);
    for (uint64_t i = 0; i < nf; ++i) {
        const uint64_t f = f0 + i;
        const uint32_t tile = (uint32_t)(f / tl.tile_size), o = (uint32_t)(f % tl.tile_size);
        for (uint32_t j = 0; j < nc; ++j) {
            out[i * nc + j] = proj_type == TRAKHIP_RADEMACHER ? jl::entry_rademacher(seed, c0 + j, tile, o)
                                                              : jl::entry_normal(seed, c0 + j, tile, o);
        }
    }
    return TRAKHIP_OK;
}

}  // namespace trakhip
