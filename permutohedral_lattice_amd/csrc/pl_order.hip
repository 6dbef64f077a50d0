// An order for a plain list of points in which neighbours in space are neighbours in the list
// (plk::order_by_locality): what lets the merging build, which counts on the 256 points of a
// workgroup sharing most of their lattice vertices, work for points that are not an image.
// No counterpart in the reference, whose GPU path inserts every key of every point into the
// global table on its own (src/PermutohedralLatticeGPU.cuh:151-208).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "pl_device.h"
#include "pl_kernels.h"

namespace plk {

namespace {

using namespace device;

constexpr int kScanBlock = 1024;
// more bins than this (lists of more than two million points) are scanned by many workgroups
constexpr unsigned kOneWorkgroupScans = 65536;

// The bins are laid over the bounding box of the first three features of a sample of the points
// (kBoxSamples of them, in runs of kSampleRun at places a multiplicative hash picks, so that no
// pattern of the list falls between them; single points all over the list cost 16 us, most of it
// address translation: every sample in a page of its own): one small workgroup finds it and
// leaves the bins for the other kernels.
// Points outside the sample's box land in the bins at its edge; a far outlier no longer
// stretches the bins of all the others.  (A pass over all points cost 7 us for a million points
// and 41 us for 8.4 million, and its 512 partial boxes had to be folded by every workgroup that
// needed them; atomic maxima on a few words instead were some ten thousand atomics on one cache
// line, one after the other, 0.4 ms.)
constexpr int kBoxSamples = 4096;
constexpr unsigned kSampleRun = 16;
constexpr float kNoValue = -3.4e38f;
constexpr int kBoxFeatures = 3;
struct Box {
    float hi[kBoxFeatures], neg_lo[kBoxFeatures];
};
// A bin is meant to be a wavefront's share: when every bin starts a wavefront of its own, the 64
// lanes hold points of one bin as they hold 8x8 pixels of an image, and share as many vertices.
// (The build of a 1024x1024 image given as a list, bins following each other without gaps, so
// that a wavefront takes parts of two: 85 us; every bin a wavefront: 60 us.  Bins of 16 points
// along a Hilbert curve, without gaps, changed nothing: a wavefront then takes parts of two small
// bins plus four whole ones, and the count and the scan of four times the bins cost 10 us more.)
// Points in a regular pattern fill bins of this size with at most 64 each: 7 or 8 rows of 7 or 8
// (56: 0.317 ms per step for the 1024x1024 image as a list, 60: 0.310, 63: 0.307, but the nearer to
// 64, the less unevenness it takes for bins to need a second wavefront).
constexpr float kPointsPerBin = 60.0f;
// The third feature takes part when its extent is at least this fraction of the larger of the
// first two: the depth of a volume does, the first colour channel of an image under a wide colour
// kernel does not (its few bins would only cut the tiles of the image in layers).
constexpr float kThirdFeatureExtent = 0.125f;

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x = fmaxf(x, __shfl_xor(x, d));
    return x;
}

__device__ __forceinline__ void widen(Box &b, const Box &o) {
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f) {
        b.hi[f] = fmaxf(b.hi[f], o.hi[f]);
        b.neg_lo[f] = fmaxf(b.neg_lo[f], o.neg_lo[f]);
    }
}
__device__ __forceinline__ Box empty_box() {
    Box b;
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f) b.hi[f] = b.neg_lo[f] = kNoValue;
    return b;
}
// The box of the boxes of all threads of the workgroup, in every thread.  (fmaxf drops NaNs.)
__device__ __forceinline__ Box block_box(Box v, Box *wave_part) {
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f) {
        v.hi[f] = wave_max(v.hi[f]);
        v.neg_lo[f] = wave_max(v.neg_lo[f]);
    }
    const int wave = threadIdx.x >> 6, n_waves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) wave_part[wave] = v;
    __syncthreads();
    Box all = wave_part[0];
    for (int w = 1; w < n_waves; ++w) widen(all, wave_part[w]);
    return all;
}

// The bins for the box; the same in every thread of every kernel of one call.
struct LocalityBins {
    float lo[kBoxFeatures], per_unit;   // bin along feature i = (feature i - lo_i) * per_unit
    int n[kBoxFeatures];                // bins along the features (1 along one that takes no part)
    unsigned n_bins;                    // numbers in use: 2x2 bins along the first two features stay together
    float hi0;
};
static_assert(sizeof(LocalityBins) <= kLocalityBinsBytes, "the record the kernels pass the bins in");
__device__ __forceinline__ LocalityBins *bins_record(const LocalityScratch &scratch) {
    return static_cast<LocalityBins *>(scratch.bins);
}
__device__ __forceinline__ uint64_t bin_numbers(int n0, int n1, int n2) {
    return (uint64_t)((n0 + 1) >> 1) * (uint64_t)((n1 + 1) >> 1) * 4u * (uint64_t)n2;
}
__device__ __forceinline__ LocalityBins bins_over(const Box &box, int N, int pd, unsigned max_bins) {
    LocalityBins b{{0.0f, 0.0f, 0.0f}, 0.0f, {1, 1, 1}, 4u, 0.0f};
    float r[kBoxFeatures];
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f) {
        const bool there = f < pd;
        b.lo[f] = there ? -box.neg_lo[f] : 0.0f;
        r[f] = there ? box.hi[f] + box.neg_lo[f] : 0.0f;
    }
    b.hi0 = box.hi[0];
    // (a box with a NaN or an infinity in it: one bin, the order of the list)
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f)
        if (!(r[f] >= 0.0f && r[f] < 3.0e38f)) return b;
    const float flat = fmaxf(r[0], r[1]);
    const bool third = r[2] > 0.0f && r[2] >= kThirdFeatureExtent * flat;
    if (!third) r[2] = 0.0f;
    // the side of a square (cubic) bin that holds kPointsPerBin points if they are spread evenly
    // over the box (over its longer side if it is a line)
    const float per_point = kPointsPerBin / (float)N;
    float side;
    if (third && r[0] > 0.0f && r[1] > 0.0f) {
        side = cbrtf(r[0] * r[1] * (r[2] * per_point));
    } else if (third && flat > 0.0f) {
        side = sqrtf(flat * (r[2] * per_point));
    } else if (r[0] > 0.0f && r[1] > 0.0f && r[0] * r[1] > 0.0f) {
        side = sqrtf(r[0] * (r[1] * per_point));
    } else {
        side = fmaxf(flat, r[2]) * per_point;
    }
    if (!(side > 0.0f)) return b;
    for (int turn = 0; turn < 256; ++turn) {
        const float f0 = r[0] / side + 1.0f, f1 = r[1] / side + 1.0f, f2 = r[2] / side + 1.0f;
        if (f0 < 1.0e6f && f1 < 1.0e6f && f2 < 1.0e6f) {
            const int n0 = (int)f0, n1 = (int)f1, n2 = (int)f2;
            const uint64_t numbers = bin_numbers(n0, n1, n2);
            if (numbers <= (uint64_t)max_bins) {
                b.n[0] = n0;
                b.n[1] = n1;
                b.n[2] = n2;
                b.n_bins = (unsigned)numbers;
                b.per_unit = 1.0f / side;
                return b;
            }
        }
        side *= 1.25f;
    }
    return b;
}
__device__ __forceinline__ unsigned bin_of(const LocalityBins &b, const float (&p)[kBoxFeatures]) {
    // (fminf and fmaxf drop a NaN operand: such a point lands in bin 0)
    int c[kBoxFeatures];
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f)
        c[f] = (int)fminf(fmaxf((p[f] - b.lo[f]) * b.per_unit, 0.0f), (float)(b.n[f] - 1));
    const unsigned pair = (unsigned)(c[0] >> 1) * (unsigned)((b.n[1] + 1) >> 1) + (unsigned)(c[1] >> 1);
    // The four bins of a 2x2 block in the order down, across, up: each bin touches the one before
    // it, and the last touches the first of the block to its right, so that any 256 consecutive
    // points (a workgroup of the build, wherever its share starts) lie in bins that hang together.
    // The bins along the third feature follow each other inside each of those.
    const unsigned down = (unsigned)(c[0] & 1), across = (unsigned)(c[1] & 1);
    return (pair * 4u + (across ? 3u - down : down)) * (unsigned)b.n[2] + (unsigned)c[2];
}

template <typename T>
__device__ __forceinline__ void first_features(const T *__restrict__ positions, size_t n, int pd,
                                               float (&p)[kBoxFeatures]) {
    const T *row = positions + n * (size_t)pd;
#pragma unroll
    for (int f = 0; f < kBoxFeatures; ++f) p[f] = f < pd ? (float)row[f] : 0.0f;
}

// The bins for this list: the box of the sampled points, the bins over it, left in memory for the
// kernels that follow (one workgroup)
template <typename T>
__global__ __launch_bounds__(kScanBlock) void k_locality_bins(const T *__restrict__ positions, int N, int pd,
                                                               LocalityScratch scratch) {
    __shared__ Box wave_part[kScanBlock / 64];
    // (all the loads first, none behind a branch: a sample past the end reads the last point)
    constexpr int kPerThread = kBoxSamples / kScanBlock;
    float p[kPerThread][kBoxFeatures];
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
        const unsigned sample = (unsigned)(k * kScanBlock) + threadIdx.x;
        // (every point when there are no more than samples)
        const unsigned run = sample / kSampleRun, in_run = sample % kSampleRun;
        unsigned n = N <= kBoxSamples
                         ? sample
                         : (unsigned)((((uint64_t)run * 0x9E3779B97F4A7C15ull) >> 32) * (uint64_t)(unsigned)N >> 32) + in_run;
        n = n < (unsigned)N ? n : (unsigned)N - 1u;
        first_features(positions, (size_t)n, pd, p[k]);
    }
    Box v = empty_box();
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
#pragma unroll
        for (int f = 0; f < kBoxFeatures; ++f) {
            v.hi[f] = fmaxf(v.hi[f], p[k][f]);
            v.neg_lo[f] = fmaxf(v.neg_lo[f], -p[k][f]);
        }
    }
    v = block_box(v, wave_part);
    if (threadIdx.x == 0) {
        const LocalityBins bins = bins_over(v, N, pd, scratch.max_bins);
        *bins_record(scratch) = bins;
        scratch.range0[0] = bins.lo[0];
        scratch.range0[1] = bins.hi0;
    }
}

// Every point draws its rank in its bin.  The lanes of a wavefront that share a bin (in a list
// that has any order at all, most of them) draw their ranks with one atomic.  A thread takes
// kCountPoints points, 256 apart, so that their loads and their atomics are in flight together.
// (Also: every place of the order set to "no point".)
constexpr int kCountPoints = 2;
template <typename T>
__global__ __launch_bounds__(kBlock) void k_locality_count(const T *__restrict__ positions, int N, int pd,
                                                            LocalityScratch scratch, int *__restrict__ order,
                                                            size_t order_entries) {
    const int lane = threadIdx.x & 63;
    // (the places of the order that the scatter will leave empty)
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < order_entries;
         i += (size_t)gridDim.x * kBlock)
        order[i] = -1;
    const LocalityBins bins = *bins_record(scratch);
    size_t n[kCountPoints];
    bool valid[kCountPoints];
    float p[kCountPoints][kBoxFeatures];
#pragma unroll
    for (int k = 0; k < kCountPoints; ++k) {
        n[k] = ((size_t)blockIdx.x * kCountPoints + k) * kBlock + threadIdx.x;
        valid[k] = n[k] < (size_t)N;
#pragma unroll
        for (int f = 0; f < kBoxFeatures; ++f) p[k][f] = 0.0f;
        if (valid[k]) first_features(positions, n[k], pd, p[k]);
    }
    int bin[kCountPoints], leader[kCountPoints];
    unsigned size[kCountPoints], index[kCountPoints], first_rank[kCountPoints];
#pragma unroll
    for (int k = 0; k < kCountPoints; ++k) {
        bin[k] = valid[k] ? (int)bin_of(bins, p[k]) : 0;
        // after 16 different bins the lanes that are left draw their ranks one by one
        uint64_t todo = wave_ballot(valid[k]);
        leader[k] = lane;
        size[k] = 1;
        index[k] = 0;
        for (int turn = 0; todo != 0 && turn < 16; ++turn) {
            const int first = __builtin_ctzll(todo);
            const int b = __builtin_amdgcn_readlane(bin[k], first);
            const uint64_t same = lanes_equal(bin[k], b) & todo;
            if (lane_in(same)) {
                leader[k] = first;
                size[k] = (unsigned)__builtin_popcountll(same);
                index[k] = __builtin_amdgcn_mbcnt_hi((unsigned)(same >> 32),
                                                     __builtin_amdgcn_mbcnt_lo((unsigned)same, 0u));
            }
            todo &= ~same;
        }
    }
#pragma unroll
    for (int k = 0; k < kCountPoints; ++k) {
        first_rank[k] = 0;
        if (valid[k] && leader[k] == lane) first_rank[k] = atomicAdd(&scratch.bin_count[bin[k]], size[k]);
    }
#pragma unroll
    for (int k = 0; k < kCountPoints; ++k) {
        first_rank[k] = __shfl(first_rank[k], leader[k]);
        if (valid[k]) scratch.bin_rank[n[k]] = make_uint2((unsigned)bin[k], first_rank[k] + index[k]);
    }
}

// bin_first = the place of each bin's first point in the order; the counts go back to zero for
// the next call.  If giving every bin wavefronts of its own (its count rounded up to 64s) takes no
// more workgroups than the order has room for, the bins are laid out so; else one behind the
// other.  One workgroup: every thread takes a run of bins, four at a time (the arrays are as long
// as max_bins, a multiple of four, and the counts behind the bins in use are zero).
constexpr unsigned kScanHeld = 8;   // fours of counts a thread holds in registers between its two passes
__device__ __forceinline__ unsigned wavefronts_for(unsigned points) { return (points + 63u) >> 6; }
__global__ __launch_bounds__(kScanBlock) void k_locality_scan(LocalityScratch scratch, int N) {
    __shared__ unsigned wave_total[kScanBlock / 64];
    __shared__ unsigned wave_padded[kScanBlock / 64];
    uint4 *__restrict__ count4 = reinterpret_cast<uint4 *>(scratch.bin_count);
    uint4 *__restrict__ first4 = reinterpret_cast<uint4 *>(scratch.bin_first);
    unsigned n_bins = bins_record(scratch)->n_bins;
    if (n_bins > scratch.max_bins) n_bins = scratch.max_bins;
    const unsigned n_fours = (n_bins + 3u) / 4u;
    const unsigned per = (n_fours + kScanBlock - 1) / kScanBlock;
    const unsigned begin = threadIdx.x * per;
    const unsigned end = begin + per < n_fours ? begin + per : n_fours;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint4 held[kScanHeld];
    unsigned points = 0, padded = 0;   // of this thread's bins: points, and wavefronts if each bin has its own
    auto add = [&](const uint4 &c) {
        points += (c.x + c.y) + (c.z + c.w);
        padded += (wavefronts_for(c.x) + wavefronts_for(c.y)) + (wavefronts_for(c.z) + wavefronts_for(c.w));
    };
#pragma unroll
    for (unsigned k = 0; k < kScanHeld; ++k) {
        held[k] = begin + k < end ? count4[begin + k] : make_uint4(0u, 0u, 0u, 0u);
        add(held[k]);
    }
    for (unsigned i = begin + kScanHeld; i < end; ++i) add(count4[i]);
    // which layout: all the wavefronts of the second must fit
    unsigned all_padded = padded;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) all_padded += __shfl_xor(all_padded, d);
    if (lane == 0) wave_padded[wave] = all_padded;
    __syncthreads();
    all_padded = 0;
    for (int w = 0; w < kScanBlock / 64; ++w) all_padded += wave_padded[w];
    const bool own_wavefronts = all_padded <= 4u * scratch.max_tiles;
    // the sums before this thread: within the wavefront, then over the wavefronts
    const unsigned sum = own_wavefronts ? padded : points;
    unsigned inclusive = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const unsigned other = __shfl_up(inclusive, d);
        if (lane >= d) inclusive += other;
    }
    if (lane == 63) wave_total[wave] = inclusive;
    __syncthreads();
    unsigned before = inclusive - sum;
    for (int w = 0; w < wave; ++w) before += wave_total[w];
    if (own_wavefronts) before *= 64u;
    auto room = [&](unsigned c) { return own_wavefronts ? wavefronts_for(c) * 64u : c; };
    auto place = [&](unsigned i, const uint4 &c) {
        uint4 f;
        f.x = before;
        f.y = f.x + room(c.x);
        f.z = f.y + room(c.y);
        f.w = f.z + room(c.z);
        before = f.w + room(c.w);
        first4[i] = f;
        count4[i] = make_uint4(0u, 0u, 0u, 0u);
    };
#pragma unroll
    for (unsigned k = 0; k < kScanHeld; ++k)
        if (begin + k < end) place(begin + k, held[k]);
    for (unsigned i = begin + kScanHeld; i < end; ++i) place(i, count4[i]);
    if (threadIdx.x == 0) {
        const unsigned wavefronts = own_wavefronts ? all_padded : wavefronts_for((unsigned)N);
        const unsigned tiles = (wavefronts + 3u) / 4u;
        *scratch.n_tiles = tiles < scratch.max_tiles ? tiles : scratch.max_tiles;
    }
}

// The same in three launches, for more bins than one workgroup scans in a few microseconds: every
// workgroup takes kScanChunk fours of bins (a thread kScanRun of them, next to each other), the
// first launch leaves each chunk's two sums, one workgroup chooses the layout and turns the chosen
// sums into the places before each chunk, the third launch places the bins.
constexpr unsigned kScanRun = 4, kScanChunk = kScanRun * kBlock;
__device__ __forceinline__ void chunk_counts(const LocalityScratch &scratch, uint4 (&c)[kScanRun],
                                             unsigned &points, unsigned &padded) {
    const uint4 *__restrict__ count4 = reinterpret_cast<const uint4 *>(scratch.bin_count);
    const unsigned n_fours = scratch.max_bins / 4u;
    const unsigned begin = blockIdx.x * kScanChunk + threadIdx.x * kScanRun;
    points = padded = 0;
#pragma unroll
    for (unsigned k = 0; k < kScanRun; ++k) {
        c[k] = begin + k < n_fours ? count4[begin + k] : make_uint4(0u, 0u, 0u, 0u);
        points += (c[k].x + c[k].y) + (c[k].z + c[k].w);
        padded += (wavefronts_for(c[k].x) + wavefronts_for(c[k].y)) +
                  (wavefronts_for(c[k].z) + wavefronts_for(c[k].w));
    }
}
__global__ __launch_bounds__(kBlock) void k_locality_chunk_sums(LocalityScratch scratch) {
    __shared__ unsigned part[2][kBlock / 64];
    uint4 c[kScanRun];
    unsigned points, padded;
    chunk_counts(scratch, c, points, padded);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        points += __shfl_xor(points, d);
        padded += __shfl_xor(padded, d);
    }
    if ((threadIdx.x & 63) == 0) {
        part[0][threadIdx.x >> 6] = points;
        part[1][threadIdx.x >> 6] = padded;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned a = 0, b = 0;
        for (int w = 0; w < kBlock / 64; ++w) {
            a += part[0][w];
            b += part[1][w];
        }
        scratch.chunk_sums[2 * blockIdx.x] = a;
        scratch.chunk_sums[2 * blockIdx.x + 1] = b;
    }
}
// (one wavefront: the chunks are few)
__global__ __launch_bounds__(64) void k_locality_chunk_places(LocalityScratch scratch, int N, unsigned n_chunks) {
    unsigned all_padded = 0;
    for (unsigned i = threadIdx.x; i < n_chunks; i += 64) all_padded += scratch.chunk_sums[2 * i + 1];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) all_padded += __shfl_xor(all_padded, d);
    const bool own_wavefronts = all_padded <= 4u * scratch.max_tiles;
    unsigned before = 0;
    for (unsigned i0 = 0; i0 < n_chunks; i0 += 64) {
        const unsigned i = i0 + threadIdx.x;
        const unsigned sum = i < n_chunks ? scratch.chunk_sums[2 * i + (own_wavefronts ? 1 : 0)] : 0u;
        unsigned inclusive = sum;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const unsigned other = __shfl_up(inclusive, d);
            if ((int)threadIdx.x >= d) inclusive += other;
        }
        if (i < n_chunks) scratch.chunk_first[i] = (before + inclusive - sum) * (own_wavefronts ? 64u : 1u);
        before += __shfl(inclusive, 63);
    }
    if (threadIdx.x == 0) {
        scratch.chunk_first[n_chunks] = own_wavefronts ? 1u : 0u;
        const unsigned wavefronts = own_wavefronts ? all_padded : wavefronts_for((unsigned)N);
        const unsigned tiles = (wavefronts + 3u) / 4u;
        *scratch.n_tiles = tiles < scratch.max_tiles ? tiles : scratch.max_tiles;
    }
}
__global__ __launch_bounds__(kBlock) void k_locality_chunk_scan(LocalityScratch scratch, unsigned n_chunks) {
    __shared__ unsigned wave_total[kBlock / 64];
    uint4 *__restrict__ count4 = reinterpret_cast<uint4 *>(scratch.bin_count);
    uint4 *__restrict__ first4 = reinterpret_cast<uint4 *>(scratch.bin_first);
    const unsigned n_fours = scratch.max_bins / 4u;
    const unsigned begin = blockIdx.x * kScanChunk + threadIdx.x * kScanRun;
    const bool own_wavefronts = scratch.chunk_first[n_chunks] != 0u;
    uint4 c[kScanRun];
    unsigned points, padded;
    chunk_counts(scratch, c, points, padded);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned sum = own_wavefronts ? padded * 64u : points;
    unsigned inclusive = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const unsigned other = __shfl_up(inclusive, d);
        if (lane >= d) inclusive += other;
    }
    if (lane == 63) wave_total[wave] = inclusive;
    __syncthreads();
    unsigned before = scratch.chunk_first[blockIdx.x] + inclusive - sum;
    for (int w = 0; w < wave; ++w) before += wave_total[w];
    auto room = [&](unsigned n) { return own_wavefronts ? wavefronts_for(n) * 64u : n; };
#pragma unroll
    for (unsigned k = 0; k < kScanRun; ++k) {
        if (begin + k >= n_fours) break;
        uint4 f;
        f.x = before;
        f.y = f.x + room(c[k].x);
        f.z = f.y + room(c[k].y);
        f.w = f.z + room(c[k].z);
        before = f.w + room(c[k].w);
        first4[begin + k] = f;
        count4[begin + k] = make_uint4(0u, 0u, 0u, 0u);
    }
}

__global__ __launch_bounds__(kBlock) void k_locality_scatter(LocalityScratch scratch, int N,
                                                              int *__restrict__ order) {
    const size_t n = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (n >= (size_t)N) return;
    const uint2 br = scratch.bin_rank[n];
    const unsigned place = scratch.bin_first[br.x] + br.y;
    // (ranks come from atomics on counts that started at zero, so the place is the point's own)
    if ((size_t)place < (size_t)scratch.max_tiles * kBlock) order[place] = (int)n;
}

template <typename T>
hipError_t order_points(const T *positions, int N, int pd, const LocalityScratch &scratch, int *order,
                        hipStream_t s) {
    const unsigned blocks = (unsigned)(((size_t)N + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((k_locality_bins<T>), dim3(1), dim3(kScanBlock), 0, s, positions, N, pd, scratch);
    const unsigned count_blocks = (blocks + kCountPoints - 1) / kCountPoints;
    hipLaunchKernelGGL((k_locality_count<T>), dim3(count_blocks), dim3(kBlock), 0, s, positions, N, pd, scratch,
                       order, (size_t)scratch.max_tiles * kBlock);
    if (scratch.max_bins <= kOneWorkgroupScans) {
        hipLaunchKernelGGL(k_locality_scan, dim3(1), dim3(kScanBlock), 0, s, scratch, N);
    } else {
        // (over all max_bins: the counts behind the bins in use are zero)
        const unsigned n_chunks = locality_scan_chunks(scratch.max_bins);
        hipLaunchKernelGGL(k_locality_chunk_sums, dim3(n_chunks), dim3(kBlock), 0, s, scratch);
        hipLaunchKernelGGL(k_locality_chunk_places, dim3(1), dim3(64), 0, s, scratch, N, n_chunks);
        hipLaunchKernelGGL(k_locality_chunk_scan, dim3(n_chunks), dim3(kBlock), 0, s, scratch, n_chunks);
    }
    hipLaunchKernelGGL(k_locality_scatter, dim3(blocks), dim3(kBlock), 0, s, scratch, N, order);
    return hipGetLastError();
}

}  // namespace

hipError_t order_by_locality(const float *positions, const double *positions64, int N, int pd,
                             const LocalityScratch &scratch, int *order, hipStream_t s) {
    if (N <= 0) return hipSuccess;
    if (!scratch.bins || !scratch.range0 || !scratch.bin_count || !scratch.bin_first ||
        !scratch.bin_rank || !order || !scratch.n_tiles || !scratch.chunk_sums || !scratch.chunk_first ||
        scratch.max_bins < 4u ||
        (size_t)scratch.max_tiles * kBlock < (size_t)N || scratch.max_bins % 4u != 0u ||
        (reinterpret_cast<uintptr_t>(scratch.bin_count) | reinterpret_cast<uintptr_t>(scratch.bin_first)) % 16u != 0u ||
        pd < 1)
        return hipErrorInvalidValue;
    if (positions64) return order_points<double>(positions64, N, pd, scratch, order, s);
    if (positions) return order_points<float>(positions, N, pd, scratch, order, s);
    return hipErrorInvalidValue;
}

}  // namespace plk
