// Device-side building blocks shared by the kernels for float values (pl_kernels.hip) and for
// double values (pl_kernels_f64.hip): the packed vertex key and its hash, the simplex of a point,
// the point <-> thread mapping, the wavefront election, the walk over vertex blocks, and the
// host helpers that size grids.
//
// Translation units that include this must be compiled with -ffp-contract=off: the integer results
// (nearest lattice point, rank permutation, vertex keys) are only equal to those of the reference
// CPU path (src/PermutohedralLatticeCPU.h:220-304 of the reference tree) if every floating-point
// operation of the embedding is a single IEEE operation.
#ifndef PL_DEVICE_H
#define PL_DEVICE_H

#include <hip/hip_runtime.h>

#include <cstdint>

#include "pl_kernels.h"

namespace plk {
namespace device {

constexpr int kBlock = 256;
constexpr unsigned kXcds = 8;  // MI355X: 8 accelerator dies, each with its own L2

// Workgroups are handed to the XCDs round-robin (workgroup b runs on XCD b % 8).  Points that are
// close in memory share lattice vertices, so the kernels that update shared cells or values
// atomically give each XCD one contiguous range of points: the contended lines then stay in
// one L2 instead of migrating between dies.
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned b, unsigned nb, int enabled) {
    if (!enabled) return b;
    const unsigned q = nb / kXcds, rem = nb % kXcds;
    const unsigned xcd = b % kXcds, i = b / kXcds;
    return xcd * q + (xcd < rem ? xcd : rem) + i;
}

template <int PD>
struct KeyCodec {
    static constexpr int kBits = (60 / PD) > 16 ? 16 : (60 / PD);
    static constexpr int kBias = 1 << (kBits - 1);
    // one step of margin on both sides so that a neighbour's coordinate never leaves its field
    static constexpr int kMinQ = -kBias + 1;
    static constexpr int kMaxQ = kBias - 2;
    static constexpr uint64_t kFieldMask = (1ull << kBits) - 1ull;

    template <int N>
    __device__ static uint64_t pack(const int (&q)[N], int r) {
        static_assert(N >= PD, "one q per stored coordinate");
        uint64_t k = (uint64_t)(uint32_t)r << 60;
#pragma unroll
        for (int i = 0; i < PD; ++i) k |= (uint64_t)(uint32_t)(q[i] + kBias) << (i * kBits);
        return k;
    }
    __device__ static void unpack(uint64_t k, int (&q)[PD], int &r) {
        r = (int)(k >> 60);
#pragma unroll
        for (int i = 0; i < PD; ++i) q[i] = (int)((k >> (i * kBits)) & kFieldMask) - kBias;
    }
};

// One 32-bit multiplication: the two words of the key folded with a rotation (the fields that
// differ between the keys of one neighbourhood lie at different bit positions of the fold), a
// multiplicative hash of that, and its high bits brought down, since the cell of a key is taken
// from the low bits and the LDS slot of a tile from the nine highest.  Spreads the vertex keys of
// an image over the table, and a tile's keys over its 512 slots, as evenly as a finalizer of three
// multiplications did (keys beyond their first pair of cells: 1.6 % either way at load 0.17; 0.12
// further slot probes per key either way), at a third of its cost: a 32-bit multiplication takes
// the vector unit four times as long as an addition.
__device__ __forceinline__ uint32_t hash_key(uint64_t k) {
    const uint32_t lo = (uint32_t)k, hi = (uint32_t)(k >> 32);
    uint32_t x = lo ^ ((hi << 13) | (hi >> 19));
    x *= 0x9E3779B1u;
    x ^= x >> 15;
    return x;
}
constexpr int kTileSlotShift = 23;   // LDS slot of a key: hash_key(key) >> kTileSlotShift (512 slots)

// Wide keys.  The packed 64-bit key leaves pd >= 5 less than the 16 bits per coordinate that the
// reference's keys have (short key[pd], src/PermutohedralLatticeCPU.h:297-304): a lattice whose
// coordinates do not fit is built again with keys of two words, 16 bits per field (15 for pd = 8,
// whose fields need 13), r in the top four bits of the second word.  A biased field is never all
// ones and r is at most 8, so neither word of a key is all ones, the mark of an empty word.
struct Key128 {
    uint64_t a, b;
};
__device__ __forceinline__ bool operator==(const Key128 &x, const Key128 &y) {
    return x.a == y.a && x.b == y.b;
}
template <int PD>
struct WideCodec {
    static constexpr int kBits = (124 / PD) > 16 ? 16 : (124 / PD);
    static constexpr int kBias = 1 << (kBits - 1);
    template <int N>
    __device__ static Key128 pack(const int (&q)[N], int r) {
        static_assert(N >= PD, "one q per stored coordinate");
        unsigned __int128 k = (unsigned __int128)(unsigned)r << 124;
#pragma unroll
        for (int i = 0; i < PD; ++i) k |= (unsigned __int128)(uint32_t)(q[i] + kBias) << (i * kBits);
        return Key128{(uint64_t)k, (uint64_t)(k >> 64)};
    }
    __device__ static void unpack(const Key128 &key, int (&q)[PD], int &r) {
        const unsigned __int128 k = ((unsigned __int128)key.b << 64) | key.a;
        r = (int)(key.b >> 60);
#pragma unroll
        for (int i = 0; i < PD; ++i)
            q[i] = (int)((uint32_t)(k >> (i * kBits)) & ((1u << kBits) - 1u)) - kBias;
    }
};
__device__ __forceinline__ uint32_t hash_key(const Key128 &k) {
    return hash_key(k.a ^ (k.b * 0x9E3779B97F4A7C15ull) ^ (k.b >> 31));
}
// Keys spread over the table by where they lie along feature 0.  Every XCD has an L2 of its own,
// and the kernels deal their work out so that an XCD handles one band of image rows (one
// contiguous eighth of the tiles, of the vertices): if a vertex's cell is taken from the eighth of
// the table that belongs to its band, what an XCD looks up -- its own vertices and their
// neighbours -- lies in an eighth of the table instead of all over it.  Feature 0 can be read off a
// key: the first two coordinates of an elevated point differ by twice its scaled feature 0, and a
// vertex is within pd+1 of the points that touch it.
// Only the first two cells of a key's probe sequence are in its band's part (an aligned pair, so
// one 16-byte piece of a line); after them the sequence is the plain one, from the key's hash over
// the whole table.  With the table a fifth full that places 19 keys of 20 in their band, and an
// input whose vertices crowd into one band (an image that is flat but for a few rows) costs every
// key two more probe steps and nothing else.
struct KeyRegions {
    float lo, per_unit;   // band = (scaled feature 0 - lo) * per_unit, clamped to 0..7; per_unit 0: one band
};
__device__ __forceinline__ KeyRegions key_regions(const RegionSource &src) {
    KeyRegions regions{0.0f, 0.0f};
    if (!src.enabled || src.N < 2) return regions;
    float a = src.first, b = src.last;
    if (src.range0) {
        a = src.range0[0];
        b = src.range0[1];
    } else if (src.positions) {
        a = src.positions[0];
        b = src.positions[(size_t)(src.N - 1) * src.pd];
    } else if (src.positions64) {
        a = (float)src.positions64[0];
        b = (float)src.positions64[(size_t)(src.N - 1) * src.pd];
    }
    a *= src.scale0;
    b *= src.scale0;
    const float lo = fminf(a, b), span = fmaxf(a, b) - lo;
    // bands narrower than a few lattice steps would scatter a point's vertices over several
    if (!(span >= 32.0f * (float)(src.pd + 1))) return regions;
    regions.lo = lo;
    regions.per_unit = 8.0f / span;
    return regions;
}
template <int PD>
__device__ __forceinline__ uint32_t cell_of_key(uint64_t key, uint32_t mask, const KeyRegions &regions) {
    const uint32_t h = hash_key(key);
    if (regions.per_unit == 0.0f) return h & mask & ~1u;
    int q[PD], r;
    KeyCodec<PD>::unpack(key, q, r);
    // scaled feature 0 of the points around this vertex: half the difference of its first two
    // coordinates (for pd = 1 the second coordinate is minus the first)
    const float c = PD >= 2 ? 0.5f * (float)((q[0] - q[PD >= 2 ? 1 : 0]) * (PD + 1))
                            : (float)(q[0] * (PD + 1) + r);
    int band = (int)((c - regions.lo) * regions.per_unit);
    band = band < 0 ? 0 : (band > 7 ? 7 : band);
    const uint32_t low = mask >> 3;   // the table has at least 4096 cells
    return (((uint32_t)band * (low + 1u)) | (h & low)) & ~1u;
}
// A probe sequence is a sequence of aligned pairs of cells (16 bytes, one load), walked first cell
// first.  The cell after `cell`, the step-th of key's sequence (step counts from 0):
__device__ __forceinline__ uint32_t next_cell(uint32_t cell, uint32_t step, uint64_t key, uint32_t mask,
                                             const KeyRegions &regions) {
    if (regions.per_unit != 0.0f && step == 1u) return hash_key(key) & mask & ~1u;
    return (cell + 1u) & mask;
}
// and the pair after the pair that starts at `cell`, the index-th pair of the sequence
__device__ __forceinline__ uint32_t next_pair(uint32_t cell, uint32_t index, uint64_t key, uint32_t mask,
                                             const KeyRegions &regions) {
    if (regions.per_unit != 0.0f && index == 0u) return hash_key(key) & mask & ~1u;
    return (cell + 2u) & mask;
}

// ------------------------------------------------------------------------------------------------
// Per-point arithmetic: same operations, in the same precision and order, as
// x[0] >= x[1] >= ... in place.  Six values take the 12-comparator network; other counts an
// odd-even transposition sort.
template <typename S>
__device__ __forceinline__ void order_pair(S &hi, S &lo) {
    const bool swap = hi < lo;
    const S a = swap ? lo : hi, b = swap ? hi : lo;
    hi = a;
    lo = b;
}
template <int N, typename S>
__device__ __forceinline__ void sort_descending(S (&x)[N]) {
    if constexpr (N == 6) {
        order_pair(x[0], x[5]); order_pair(x[1], x[3]); order_pair(x[2], x[4]);
        order_pair(x[1], x[2]); order_pair(x[3], x[4]);
        order_pair(x[0], x[3]); order_pair(x[2], x[5]);
        order_pair(x[0], x[1]); order_pair(x[2], x[3]); order_pair(x[4], x[5]);
        order_pair(x[1], x[2]); order_pair(x[3], x[4]);
    } else {
#pragma unroll
        for (int round = 0; round < N; ++round) {
#pragma unroll
            for (int i = round & 1; i + 1 < N; i += 2) order_pair(x[i], x[i + 1]);
        }
    }
}

// embed_position_vector / find_enclosing_simplex / compute_barycentric_coordinates of the
// reference CPU path.  q[i] is rem0[i] / (pd+1).
// ------------------------------------------------------------------------------------------------
// T is the reference's value type
template <int PD, typename T = float>
struct Simplex {
    int q[PD + 1];
    int rank[PD + 1];
    T weight[PD + 1];
};

template <int PD>
__device__ __forceinline__ void enclosing_simplex(const float (&pos)[PD], const ScaleFactor &scale,
                                                  Simplex<PD> &s) {
    constexpr int D1 = PD + 1;
    const double inv_d1 = 1.0 / (double)D1;

    // elevate onto the hyperplane sum(x) = 0 (float, unfused)
    float el[D1];
    float running = 0.0f;
#pragma unroll
    for (int i = PD; i >= 1; --i) {
        const float c = pos[i - 1] * scale.v[i - 1];
        const float ic = (float)i * c;
        el[i] = running - ic;
        running = running + c;
    }
    el[0] = running;

    // nearest remainder-0 point: round each coordinate to a multiple of pd+1, ties go down
    float rem[D1];
    int qsum = 0;
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        // (The reference rounds between ceil(v) and floor(v) times pd+1.  The ceiling is the
        // floor plus one unless v is whole, and then both of its candidates are the same point:
        // one step above the floor's multiple decides the same, without a second rounding.)
        const float v = (float)((double)el[i] * inv_d1);
        const float fl = floorf(v);
        const float below = fl * (float)D1, above = below + (float)D1;
        const bool up = (above - el[i]) < (el[i] - below);
        rem[i] = up ? above : below;
        s.q[i] = (int)fl + (up ? 1 : 0);
        qsum += s.q[i];
    }

    // rank[i] = number of coordinates with a larger residual.  One strict < per pair i < j decides
    // ties exactly as the sequential loop does: true counts for i, false for j, so rank[i] starts
    // at i (the pairs below it, all taken as false) and every true moves one count from j to i.
    // The rounded point is qsum steps off the plane, which rotates the ranks by qsum.
    float d[D1];
    int rk[D1];
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        d[i] = el[i] - rem[i];
        rk[i] = i + qsum;
    }
#pragma unroll
    for (int i = 0; i < D1; ++i) {
#pragma unroll
        for (int j = i + 1; j < D1; ++j) {
            const int lt = (d[i] < d[j]) ? 1 : 0;
            rk[i] += lt;
            rk[j] -= lt;
        }
    }
    // ranks that left 0..pd wrap round, and their coordinate moves one step
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        const int step = rk[i] < 0 ? 1 : (rk[i] > PD ? -1 : 0);
        s.rank[i] = rk[i] + step * D1;
        s.q[i] += step;
        rem[i] += (float)(step * D1);
    }

    // barycentric weights.  by_rank[k] is the scaled residual of the coordinate of rank k; the
    // reference's scatter b[pd-rank] += delta, b[pd-rank+1] -= delta gives
    // b[k] = by_rank[pd-k] - by_rank[pd-k+1] with one rounding, in either order of the two updates.
    // The ranks order the coordinates by falling residual (a coordinate that wrapped moved a whole
    // step, past all that did not), so by_rank is the residuals sorted, largest first; equal
    // residuals are equal in either place.  Sorted by a network of compare-and-swaps.
    float by_rank[D1];
#pragma unroll
    for (int i = 0; i < D1; ++i) by_rank[i] = (float)((double)(el[i] - rem[i]) * inv_d1);
    sort_descending<D1>(by_rank);
#pragma unroll
    for (int k = 1; k < D1; ++k) s.weight[k] = by_rank[PD - k] - by_rank[PD - k + 1];
    s.weight[0] = (float)((double)by_rank[PD] + (1.0 + (double)(-by_rank[0])));
}

// The same for T = double.  All of it is double arithmetic except, as in the reference, the scaled
// coordinate and its product with the index, which are floats for every T (`float cf`,
// src/PermutohedralLatticeCPU.h:226).
template <int PD>
__device__ __forceinline__ void enclosing_simplex(const double (&pos)[PD], const ScaleFactor64 &scale,
                                                  Simplex<PD, double> &s) {
    constexpr int D1 = PD + 1;
    const double inv_d1 = 1.0 / (double)D1;

    double el[D1];
    double running = 0.0;
#pragma unroll
    for (int i = PD; i >= 1; --i) {
        const float c = (float)(pos[i - 1] * scale.v[i - 1]);
        const float ic = (float)i * c;
        el[i] = running - (double)ic;
        running = running + (double)c;
    }
    el[0] = running;

    double rem[D1];
    int qsum = 0;
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        const double v = el[i] * inv_d1;
        const double cu = ceil(v), fl = floor(v);
        const double above = cu * (double)D1, below = fl * (double)D1;
        const bool up = (above - el[i]) < (el[i] - below);
        rem[i] = up ? above : below;
        s.q[i] = (int)(up ? cu : fl);
        qsum += s.q[i];
    }

    double d[D1];
    int rk[D1];
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        d[i] = el[i] - rem[i];
        rk[i] = i + qsum;
    }
#pragma unroll
    for (int i = 0; i < D1; ++i) {
#pragma unroll
        for (int j = i + 1; j < D1; ++j) {
            const int lt = (d[i] < d[j]) ? 1 : 0;
            rk[i] += lt;
            rk[j] -= lt;
        }
    }
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        const int step = rk[i] < 0 ? 1 : (rk[i] > PD ? -1 : 0);
        s.rank[i] = rk[i] + step * D1;
        s.q[i] += step;
        rem[i] += (double)(step * D1);
    }

    // (the residuals sorted, largest first, as in the float version)
    double by_rank[D1];
#pragma unroll
    for (int i = 0; i < D1; ++i) by_rank[i] = (el[i] - rem[i]) * inv_d1;
    sort_descending<D1>(by_rank);
#pragma unroll
    for (int k = 1; k < D1; ++k) s.weight[k] = by_rank[PD - k] - by_rank[PD - k + 1];
    s.weight[0] = by_rank[PD] + (1.0 + (-by_rank[0]));
}

// q-coordinates of simplex vertex r: the coordinates ranked above pd-r drop by one step
template <int PD, typename T>
__device__ __forceinline__ void vertex_q(const Simplex<PD, T> &s, int r, int (&q)[PD]) {
#pragma unroll
    for (int i = 0; i < PD; ++i) q[i] = s.q[i] - ((s.rank[i] > PD - r) ? 1 : 0);
}

// The packed keys of all pd+1 vertices of a simplex.  From vertex r-1 to vertex r exactly one
// coordinate drops by one step, the one of rank pd-r+1 (the ranks are a permutation of 0..pd), so
// a key follows from the one before it: its field of that coordinate (if it is one of the pd that
// are stored) one lower, its remainder one higher.  No field can borrow from the next: a simplex
// in key range has every biased field at least 1 after the step (simplex_in_key_range).  Same
// bits as KeyCodec<PD>::pack(vertex_q(s, r), r).
template <int PD, typename T>
__device__ __forceinline__ void vertex_keys_of(const Simplex<PD, T> &s, uint64_t (&key)[PD + 1]) {
    constexpr int kBits = KeyCodec<PD>::kBits;
    key[0] = KeyCodec<PD>::pack(s.q, 0);
#pragma unroll
    for (int r = 1; r <= PD; ++r) {
        uint32_t step_lo = 0, step_hi = 0;
#pragma unroll
        for (int i = 0; i < PD; ++i) {
            const bool drops = s.rank[i] == PD - r + 1;
            if (i * kBits < 32)
                step_lo = drops ? (1u << ((i * kBits) & 31)) : step_lo;
            else
                step_hi = drops ? (1u << ((i * kBits - 32) & 31)) : step_hi;
        }
        key[r] = key[r - 1] - (((uint64_t)step_hi << 32) | step_lo) + (1ull << 60);
    }
}

template <int PD, typename T>
__device__ __forceinline__ bool simplex_in_key_range(const Simplex<PD, T> &s) {
    bool ok = true;
#pragma unroll
    for (int i = 0; i < PD; ++i)
        ok = ok && (s.q[i] - 1 >= KeyCodec<PD>::kMinQ) && (s.q[i] <= KeyCodec<PD>::kMaxQ);
    return ok;
}

// Every coordinate of every vertex of the simplex is a short, as the reference's keys are
// (q_i - 1 is the lowest a vertex takes, and the remainder is at most pd)
template <int PD, typename T>
__device__ __forceinline__ bool simplex_in_short_range(const Simplex<PD, T> &s) {
    bool ok = true;
#pragma unroll
    for (int i = 0; i < PD; ++i)
        ok = ok && ((s.q[i] - 1) * (PD + 1) >= -32768) && (s.q[i] * (PD + 1) + PD <= 32767) &&
             s.q[i] > -40000 && s.q[i] < 40000;
    return ok;
}
template <int PD, typename T>
__device__ __forceinline__ void wide_keys_of(const Simplex<PD, T> &s, Key128 (&key)[PD + 1]) {
#pragma unroll
    for (int r = 0; r <= PD; ++r) {
        int q[PD];
        vertex_q<PD>(s, r, q);
        key[r] = WideCodec<PD>::pack(q, r);
    }
}

// ------------------------------------------------------------------------------------------------
// Which point a thread works on.  Points that are neighbours in the image share lattice vertices,
// and every duplicate that meets inside one wavefront is merged before it reaches memory, so a
// wavefront should cover a compact tile of the image, not a run of 64 points of one row.  With a
// grid hint (the op knows its spatial extents) a workgroup takes a 16x16 tile of a 2-D grid
// (wavefronts 8x8) or a 4x8x8 tile of a 3-D grid (wavefronts 4x4x4); without one it takes 256
// consecutive points.  The mapping only changes the order of work, never a result.
// Per-point scratch (the replay arrays) is stored in thread order, so it stays coalesced.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ int point_of_thread(const PointMap &m, unsigned vblock, unsigned tid) {
    if (m.mode == 0) {
        const size_t n = (size_t)vblock * kBlock + tid;
        return n < (size_t)m.N ? (int)n : -1;
    }
    if (m.mode == 1) {
        if (vblock >= *m.n_tiles || vblock >= m.n_blocks) return -1;
        const int p = m.order[(size_t)vblock * kBlock + tid];
        return (unsigned)p < (unsigned)m.N ? p : -1;
    }
    const unsigned wave = tid >> 6, lane = tid & 63;
    const unsigned tiles_yx = (unsigned)m.tiles[1] * (unsigned)m.tiles[2];
    const unsigned tz = vblock / tiles_yx;
    const unsigned rest = vblock - tz * tiles_yx;
    const unsigned ty = rest / (unsigned)m.tiles[2];
    const unsigned tx = rest - ty * (unsigned)m.tiles[2];
    unsigned z, y, x;
    if (m.mode == 2) {
        z = tz;
        y = ty * 16 + (wave >> 1) * 8 + (lane >> 3);
        x = tx * 16 + (wave & 1) * 8 + (lane & 7);
    } else {
        z = tz * 4 + (lane >> 4);
        y = ty * 8 + (wave >> 1) * 4 + ((lane >> 2) & 3);
        x = tx * 8 + (wave & 1) * 4 + (lane & 3);
    }
    if (z >= (unsigned)m.dims[0] || y >= (unsigned)m.dims[1] || x >= (unsigned)m.dims[2]) return -1;
    return (int)(((size_t)z * m.dims[1] + y) * m.dims[2] + x);
}

// The share of the points this workgroup takes (vblock; each XCD a contiguous range of shares when
// xcd_aware), false when it has none: the workgroups behind the last that holds points of an
// ordered list.  Those keep their own number as vblock, so that every workgroup of the grid has
// one of its own.
__device__ __forceinline__ bool block_of_points(const PointMap &m, int xcd_aware, unsigned &vblock) {
    unsigned nb = gridDim.x;
    if (m.mode == 1) {
        const unsigned tiles = *m.n_tiles;
        nb = tiles < nb ? tiles : nb;
        if (blockIdx.x >= nb) {
            vblock = blockIdx.x;
            return false;
        }
    }
    vblock = xcd_contiguous_block(blockIdx.x, nb, xcd_aware);
    return true;
}

// Mask of the lanes whose predicate holds (the compare result itself, no detour through 0/1)
__device__ __forceinline__ uint64_t wave_ballot(bool predicate) {
    return __builtin_amdgcn_ballot_w64(predicate);
}

// Mask of the (executing) lanes whose x equals the wavefront-uniform k, straight from the compare
__device__ __forceinline__ uint64_t lanes_equal(uint64_t x, uint64_t k) {
    return __builtin_amdgcn_uicmpl(x, k, 32 /* ICMP_EQ */);
}
__device__ __forceinline__ uint64_t lanes_equal(int x, int k) {
    return __builtin_amdgcn_uicmp((unsigned)x, (unsigned)k, 32 /* ICMP_EQ */);
}
// A lane mask as a per-lane predicate
__device__ __forceinline__ bool lane_in(uint64_t mask) {
    return __builtin_amdgcn_inverse_ballot_w64(mask);
}

__device__ __forceinline__ int lane_value(int x, int lane) { return __builtin_amdgcn_readlane(x, lane); }
__device__ __forceinline__ uint64_t lane_value(uint64_t x, int lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)x, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(x >> 32), lane);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ Key128 lane_value(const Key128 &x, int lane) {
    return Key128{lane_value(x.a, lane), lane_value(x.b, lane)};
}
__device__ __forceinline__ uint64_t lanes_equal(const Key128 &x, const Key128 &k) {
    return lanes_equal(x.a, k.a) & lanes_equal(x.b, k.b);
}

// x := value (the same in all lanes) in the lanes of `lanes`, which must be among the executing
// ones.  One v_mov under a narrowed exec mask: as `lanes ? value : x` the compiler spends a move of
// the value into a vector register and a select.
__device__ __forceinline__ void set_in_lanes(int &x, uint64_t lanes, int value) {
    uint64_t saved;
    asm volatile(
        "s_mov_b64 %1, exec\n\t"
        "s_mov_b64 exec, %2\n\t"
        "v_mov_b32 %0, %3\n\t"
        "s_mov_b64 exec, %1"
        : "+v"(x), "=&s"(saved)
        : "s"(lanes), "s"(value));
}
// Lanes in a mask, as a 32-bit scalar (the compiler's count of 64 bits is carried as a 64-bit
// number, and a comparison with it then runs on the vector unit; two 32-bit counts and an addition
// stay on the scalar unit but are three instructions)
__device__ __forceinline__ int lanes_in(uint64_t mask) {
    int n;
    asm("s_bcnt1_i32_b64 %0, %1" : "=s"(n) : "s"(mask) : "scc");
    return n;
}

// Lanes that hold the same value of `x` elect the lowest of them as leader.  Returns the leader's
// lane; inactive lanes get their own.  One iteration per distinct value in the wavefront, each a
// v_readlane of the first unassigned lane's value, a compare and a ballot.
template <typename T>
__device__ __forceinline__ int wave_leader_of_equal(T x, bool active, int lane) {
    int leader = lane;
    const uint64_t among = wave_ballot(active);
    uint64_t remaining = among;
    while (remaining) {
        const int first = __builtin_ctzll(remaining);
        const uint64_t same = lanes_equal(x, lane_value(x, first)) & among;
        set_in_lanes(leader, same, first);
        remaining &= ~same;
    }
    return leader;
}
// The same, and the mask of the lanes whose group has at most small_size members.
template <typename T>
__device__ __forceinline__ int wave_leader_of_equal(T x, bool active, int lane, int small_size, uint64_t &small) {
    int leader = lane;
    small = 0;
    const uint64_t among = wave_ballot(active);
    uint64_t remaining = among;
    while (remaining) {
        const int first = __builtin_ctzll(remaining);
        const uint64_t same = lanes_equal(x, lane_value(x, first)) & among;
        set_in_lanes(leader, same, first);
        remaining &= ~same;
        if (lanes_in(same) <= small_size) small |= same;
    }
    return leader;
}

// What a build counts in, as the build after next must find it
__device__ __forceinline__ void reset_counters(Counters *c) {
    c->vertices = 0;
    c->flags = 0;
    for (int k = 0; k < kMaxSegments; ++k) c->segment_count[k].n = 0;   // (n_segments: set by every build)
    c->foreign_rows_sampled.n = 0;
}

// The passes over the vertices.  The vertex counts are only known on the device, so these kernels
// are launched for an estimate (the counts of the lattice's previous build, with a margin) and
// every workgroup walks blocks of 256 items in strides: a launch for the most vertices the table
// can hold would spend more time dispatching empty workgroups than the passes spend working.
// Workgroup b runs on XCD b % 8 and each XCD has its own L2, so XCD x walks the vertices of the
// eighth x of the image (the grid is a multiple of 8): the segments that XCD's workgroups
// numbered, when the build numbered them (Counters::n_segments != 0); else the x-th eighth of
// the numbers 0 .. vertices-1, which follow the image too.  What a workgroup gathers from is then
// mostly what its own XCD works on.
struct SegmentWalk {
    unsigned first, count;     // the run of numbers being walked (one of this XCD's)
    unsigned cursor, step;     // next block among the blocks of that run, stride
    // the runs this XCD walks: the segments run_first .. run_first + runs - 1 (runs == 0: one run
    // that is no segment, set up by the constructor)
    const Counters *counters;
    unsigned run, runs, run_first, stride;
    __device__ void load_run() {
        const unsigned n = counters->segment_count[run_first + run].n;
        first = (run_first + run) * stride;
        count = n < stride ? n : stride;
    }
    // grid_blocks: workgroups of the grid that walk (a multiple of 8), workgroup: index among them
    __device__ SegmentWalk(const Counters *counters_, int max_vertices, unsigned workgroup,
                           unsigned grid_blocks)
        : counters(counters_) {
        const unsigned xcd = workgroup % kXcds;
        const Counters::PaddedCount mine = counters->segment_count[xcd];
        run = 0;
        if (mine.n_segments >= (int)kXcds) {
            // (eight segments: XCD x walks segment x; sixty-four: segments 8x .. 8x + 7)
            runs = (unsigned)mine.n_segments / kXcds;
            run_first = xcd * runs;
            stride = segment_stride((uint32_t)max_vertices, mine.n_segments);
            if (runs == 1) {
                // (the XCD's one segment is the line just read: no second round trip to memory)
                first = xcd * stride;
                count = mine.n < stride ? mine.n : stride;
            } else {
                load_run();
            }
        } else {
            // (one run: after the numbering pass every line holds the total, after a build
            // with one segment the first)
            runs = 0;
            run_first = 0;
            stride = 0;
            const unsigned all = mine.n_segments == 1 ? counters->segment_count[0].n : mine.n;
            const unsigned m = all < (unsigned)max_vertices ? all : (unsigned)max_vertices;
            const unsigned per_xcd = ((m + kBlock - 1) / kBlock + kXcds - 1) / kXcds * kBlock;
            first = xcd * per_xcd;
            count = m > first ? (m - first < per_xcd ? m - first : per_xcd) : 0u;
        }
        cursor = workgroup / kXcds;
        step = grid_blocks / kXcds;
    }
    // This workgroup's next block b of 256 items of the run (first, count), a vertex being
    // items_per_vertex items, in a pass that visits every block `visits` times
    __device__ bool next(unsigned items_per_vertex, unsigned visits, unsigned &b) {
        for (;;) {
            const unsigned n =
                (unsigned)(((size_t)count * items_per_vertex + kBlock - 1) / kBlock) * visits;
            if (cursor < n) {
                b = cursor;
                cursor += step;
                return true;
            }
            if (run + 1 >= runs) return false;
            cursor -= n;       // (the stride carries over into the XCD's next run)
            run += 1;
            load_run();
        }
    }
};

inline unsigned blocks_for(size_t n, int block = kBlock) { return (unsigned)((n + block - 1) / block); }
// grids of the kernels that walk their items with ItemBlocks: a multiple of 8
inline unsigned vertex_blocks(size_t n_items) {
    const unsigned b = (blocks_for(n_items) + 7u) & ~7u;
    return b ? b : 8u;
}

// ------------------------------------------------------------------------------------------------
// Wavefront sums of doubles (the splat of a lattice of doubles)
// ------------------------------------------------------------------------------------------------
// The double of another lane (by DPP control; both words moved alike)
template <int CTRL>
__device__ __forceinline__ double from_lane_f64(double x) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(x), CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(x), CTRL, 0xf, 0xf, false);
    return __hiloint2double(hi, lo);
}
// Sums over the wavefront of four terms per lane (zero where `member` is false), delivered to
// every quad of lanes: lane q of a quad returns the sum of channel channel_of_quad_lane(q).  The
// terms are reduce-scattered inside each quad (two exchanges, after which a lane holds one
// channel), then summed across the quads of a row by rotations and across the rows with
// v_permlane16_swap and v_permlane32_swap (given x twice, the first result holds the even rows /
// lower half in both places and the second the odd rows / upper half: their sum is the pair's).
__device__ __forceinline__ int channel_of_quad_lane(int lane) {
    return ((lane & 1) << 1) | ((lane >> 1) & 1);
}
__device__ __forceinline__ double wave_sums_to_quads_f64(bool member, const double (&term)[4],
                                                         int lane) {
    const bool bit0 = lane & 1, bit1 = lane & 2;
    const double keep_a = member ? (bit0 ? term[2] : term[0]) : 0.0;
    const double keep_b = member ? (bit0 ? term[3] : term[1]) : 0.0;
    const double send_a = member ? (bit0 ? term[0] : term[2]) : 0.0;
    const double send_b = member ? (bit0 ? term[1] : term[3]) : 0.0;
    const double ya = keep_a + from_lane_f64<0xB1>(send_a);   // quad_perm:[1,0,3,2]
    const double yb = keep_b + from_lane_f64<0xB1>(send_b);
    double x = (bit1 ? yb : ya) + from_lane_f64<0x4E>(bit1 ? ya : yb);   // quad_perm:[2,3,0,1]
    x += from_lane_f64<0x124>(x);   // row_ror:4
    x += from_lane_f64<0x128>(x);   // row_ror:8
    {
        const unsigned lo = (unsigned)__double2loint(x), hi = (unsigned)__double2hiint(x);
        const auto l = __builtin_amdgcn_permlane16_swap(lo, lo, false, false);
        const auto h = __builtin_amdgcn_permlane16_swap(hi, hi, false, false);
        x = __hiloint2double((int)h[0], (int)l[0]) + __hiloint2double((int)h[1], (int)l[1]);
    }
    {
        const unsigned lo = (unsigned)__double2loint(x), hi = (unsigned)__double2hiint(x);
        const auto l = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
        const auto h = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
        x = __hiloint2double((int)h[0], (int)l[0]) + __hiloint2double((int)h[1], (int)l[1]);
    }
    return x;
}

// (keys of two words exist for the dimensions whose packed key has fields of less than 16 bits)
#define PLK_DISPATCH_WIDE_PD(pd, CALL)            \
    switch (pd) {                                 \
        case 5: { constexpr int PD = 5; CALL; } break; \
        case 6: { constexpr int PD = 6; CALL; } break; \
        case 7: { constexpr int PD = 7; CALL; } break; \
        case 8: { constexpr int PD = 8; CALL; } break; \
        default: return hipErrorInvalidValue;     \
    }

#define PLK_DISPATCH_PD(pd, CALL)                 \
    switch (pd) {                                 \
        case 1: { constexpr int PD = 1; CALL; } break; \
        case 2: { constexpr int PD = 2; CALL; } break; \
        case 3: { constexpr int PD = 3; CALL; } break; \
        case 4: { constexpr int PD = 4; CALL; } break; \
        case 5: { constexpr int PD = 5; CALL; } break; \
        case 6: { constexpr int PD = 6; CALL; } break; \
        case 7: { constexpr int PD = 7; CALL; } break; \
        case 8: { constexpr int PD = 8; CALL; } break; \
        default: return hipErrorInvalidValue;     \
    }


}  // namespace device
}  // namespace plk

#endif
