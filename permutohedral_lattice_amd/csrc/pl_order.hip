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

// The bounding box of the first two features is found in two steps: kBoxBlocks workgroups each
// write the box of their share of the points (largest feature 0, largest -feature 0, the same of
// feature 1), and every workgroup that needs the box folds those rows itself.  (Atomic maxima on
// four words instead: some ten thousand atomics on one cache line, one after the other, 0.4 ms.)
constexpr int kBoxBlocks = kLocalityBoxRows;
constexpr float kNoValue = -3.4e38f;
// A bin is meant to be a wavefront's share: when every bin starts a wavefront of its own, the 64
// lanes hold points of one bin as they hold 8x8 pixels of an image, and share as many vertices.
// (The build of a 1024x1024 image given as a list, bins following each other without gaps, so
// that a wavefront takes parts of two: 85 us; every bin a wavefront: 60 us.  Bins of 16 points
// along a Hilbert curve, without gaps, changed nothing: a wavefront then takes parts of two small
// bins plus four whole ones, and the count and the scan of four times the bins cost 10 us more.)
// Points in a regular pattern fill bins of this size with at most 64 each: 7 or 8 rows of 7 or 8.
constexpr float kPointsPerBin = 56.0f;

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x = fmaxf(x, __shfl_xor(x, d));
    return x;
}

// The largest of each component over the workgroup, in every thread.
// (fmaxf drops NaNs.)
__device__ __forceinline__ float4 block_max(float4 v, float4 *wave_part) {
    v.x = wave_max(v.x);
    v.y = wave_max(v.y);
    v.z = wave_max(v.z);
    v.w = wave_max(v.w);
    const int wave = threadIdx.x >> 6, n_waves = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) wave_part[wave] = v;
    __syncthreads();
    float4 all = wave_part[0];
    for (int w = 1; w < n_waves; ++w) {
        const float4 o = wave_part[w];
        all.x = fmaxf(all.x, o.x);
        all.y = fmaxf(all.y, o.y);
        all.z = fmaxf(all.z, o.z);
        all.w = fmaxf(all.w, o.w);
    }
    return all;
}

// The bins for the box; the same in every thread of every kernel of one call.
struct LocalityBins {
    float lo0, lo1, per_unit;   // bin along feature i = (feature i - lo_i) * per_unit
    int n0, n1;                 // bins along the two features
    unsigned n_bins;            // numbers in use: pairs of bins along each feature stay together
    float hi0;
};
__device__ __forceinline__ LocalityBins locality_bins(const float4 *partial_boxes, float4 *wave_part,
                                                      int N, int pd, unsigned max_bins) {
    float4 mine{kNoValue, kNoValue, kNoValue, kNoValue};
    for (int i = threadIdx.x; i < kBoxBlocks; i += blockDim.x) {
        const float4 o = partial_boxes[i];
        mine.x = fmaxf(mine.x, o.x);
        mine.y = fmaxf(mine.y, o.y);
        mine.z = fmaxf(mine.z, o.z);
        mine.w = fmaxf(mine.w, o.w);
    }
    const float4 box = block_max(mine, wave_part);
    LocalityBins b{0.0f, 0.0f, 0.0f, 1, 1, 4u, 0.0f};
    const float hi0 = box.x, lo0 = -box.y;
    const float hi1 = pd >= 2 ? box.z : 0.0f;
    const float lo1 = pd >= 2 ? -box.w : 0.0f;
    b.lo0 = lo0;
    b.lo1 = lo1;
    b.hi0 = hi0;
    const float r0 = hi0 - lo0, r1 = hi1 - lo1;
    // (a box with a NaN or an infinity in it: one bin, the order of the list)
    if (!(r0 >= 0.0f && r0 < 3.0e38f && r1 >= 0.0f && r1 < 3.0e38f)) return b;
    // the side of a square bin that holds kPointsPerBin points if they are spread evenly over the
    // box (over its longer side if it is a line)
    float side;
    if (r0 > 0.0f && r1 > 0.0f && r0 * r1 > 0.0f) {
        side = sqrtf(r0 * (r1 * kPointsPerBin / (float)N));
    } else {
        side = fmaxf(r0, r1) * kPointsPerBin / (float)N;
    }
    if (!(side > 0.0f)) return b;
    for (int turn = 0; turn < 256; ++turn) {
        const float f0 = r0 / side + 1.0f, f1 = r1 / side + 1.0f;
        if (f0 < 1.0e6f && f1 < 1.0e6f) {
            const int n0 = (int)f0, n1 = (int)f1;
            const uint64_t numbers = (uint64_t)((n0 + 1) >> 1) * (uint64_t)((n1 + 1) >> 1) * 4u;
            if (numbers <= (uint64_t)max_bins) {
                b.n0 = n0;
                b.n1 = n1;
                b.n_bins = (unsigned)numbers;
                b.per_unit = 1.0f / side;
                return b;
            }
        }
        side *= 1.25f;
    }
    return b;
}
__device__ __forceinline__ unsigned bin_of(const LocalityBins &b, float p0, float p1) {
    // (fminf and fmaxf drop a NaN operand: such a point lands in bin 0)
    const int b0 = (int)fminf(fmaxf((p0 - b.lo0) * b.per_unit, 0.0f), (float)(b.n0 - 1));
    const int b1 = (int)fminf(fmaxf((p1 - b.lo1) * b.per_unit, 0.0f), (float)(b.n1 - 1));
    const unsigned pair = (unsigned)(b0 >> 1) * (unsigned)((b.n1 + 1) >> 1) + (unsigned)(b1 >> 1);
    // The four bins of a 2x2 block in the order down, across, up: each bin touches the one before
    // it, and the last touches the first of the block to its right, so that any 256 consecutive
    // points (a workgroup of the build, wherever its share starts) lie in bins that hang together.
    const unsigned down = (unsigned)(b0 & 1), across = (unsigned)(b1 & 1);
    return pair * 4u + (across ? 3u - down : down);
}

template <typename T>
__device__ __forceinline__ void first_two_features(const T *__restrict__ positions, int n, int pd,
                                                   float &p0, float &p1) {
    const T *row = positions + (size_t)n * pd;
    p0 = (float)row[0];
    p1 = pd >= 2 ? (float)row[1] : 0.0f;
}

// The box of every kBoxBlocks-th run of 256 points, one row of partial_boxes per workgroup; and
// every place of the order set to "no point"
template <typename T>
__global__ __launch_bounds__(kBlock) void k_locality_box(const T *__restrict__ positions, int N, int pd,
                                                          float4 *partial_boxes, int *__restrict__ order,
                                                          size_t order_entries) {
    __shared__ float4 wave_part[kBlock / 64];
    // (the places of the order that the scatter will leave empty)
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < order_entries;
         i += (size_t)gridDim.x * kBlock)
        order[i] = -1;
    float4 v{kNoValue, kNoValue, kNoValue, kNoValue};
#pragma unroll 4
    for (size_t n = (size_t)blockIdx.x * kBlock + threadIdx.x; n < (size_t)N;
         n += (size_t)gridDim.x * kBlock) {
        float p0, p1;
        first_two_features(positions, (int)n, pd, p0, p1);
        v.x = fmaxf(v.x, p0);
        v.y = fmaxf(v.y, -p0);
        v.z = fmaxf(v.z, p1);
        v.w = fmaxf(v.w, -p1);
    }
    v = block_max(v, wave_part);
    if (threadIdx.x == 0) partial_boxes[blockIdx.x] = v;
}

// Every point draws its rank in its bin.  The lanes of a wavefront that share a bin (in a list
// that has any order at all, most of them) draw their ranks with one atomic.  A thread takes
// kCountPoints points, 256 apart, so that their loads and their atomics are in flight together.
constexpr int kCountPoints = 2;
template <typename T>
__global__ __launch_bounds__(kBlock) void k_locality_count(const T *__restrict__ positions, int N, int pd,
                                                            LocalityScratch scratch) {
    const int lane = threadIdx.x & 63;
    __shared__ float4 wave_part[kBlock / 64];
    // (the loads of the points are on their way while the boxes are folded)
    size_t n[kCountPoints];
    bool valid[kCountPoints];
    float p0[kCountPoints], p1[kCountPoints];
#pragma unroll
    for (int k = 0; k < kCountPoints; ++k) {
        n[k] = ((size_t)blockIdx.x * kCountPoints + k) * kBlock + threadIdx.x;
        valid[k] = n[k] < (size_t)N;
        p0[k] = p1[k] = 0.0f;
        if (valid[k]) first_two_features(positions, (int)n[k], pd, p0[k], p1[k]);
    }
    const LocalityBins bins = locality_bins(scratch.partial_boxes, wave_part, N, pd, scratch.max_bins);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        // what the scan needs of them
        scratch.range0[0] = bins.lo0;
        scratch.range0[1] = bins.hi0;
        reinterpret_cast<unsigned *>(scratch.range0)[2] = bins.n_bins;
    }
    int bin[kCountPoints], leader[kCountPoints];
    unsigned size[kCountPoints], index[kCountPoints], first_rank[kCountPoints];
#pragma unroll
    for (int k = 0; k < kCountPoints; ++k) {
        bin[k] = valid[k] ? (int)bin_of(bins, p0[k], p1[k]) : 0;
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
    unsigned n_bins = reinterpret_cast<const unsigned *>(scratch.range0)[2];
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
    hipLaunchKernelGGL((k_locality_box<T>), dim3(kBoxBlocks), dim3(kBlock), 0, s, positions, N, pd,
                       scratch.partial_boxes, order, (size_t)scratch.max_tiles * kBlock);
    const unsigned count_blocks = (blocks + kCountPoints - 1) / kCountPoints;
    hipLaunchKernelGGL((k_locality_count<T>), dim3(count_blocks), dim3(kBlock), 0, s, positions, N, pd, scratch);
    hipLaunchKernelGGL(k_locality_scan, dim3(1), dim3(kScanBlock), 0, s, scratch, N);
    hipLaunchKernelGGL(k_locality_scatter, dim3(blocks), dim3(kBlock), 0, s, scratch, N, order);
    return hipGetLastError();
}

}  // namespace

hipError_t order_by_locality(const float *positions, const double *positions64, int N, int pd,
                             const LocalityScratch &scratch, int *order, hipStream_t s) {
    if (N <= 0) return hipSuccess;
    if (!scratch.partial_boxes || !scratch.range0 || !scratch.bin_count || !scratch.bin_first ||
        !scratch.bin_rank || !order || !scratch.n_tiles || scratch.max_bins < 4u ||
        (size_t)scratch.max_tiles * kBlock < (size_t)N || scratch.max_bins % 4u != 0u ||
        (reinterpret_cast<uintptr_t>(scratch.bin_count) | reinterpret_cast<uintptr_t>(scratch.bin_first)) % 16u != 0u ||
        pd < 1)
        return hipErrorInvalidValue;
    if (positions64) return order_points<double>(positions64, N, pd, scratch, order, s);
    if (positions) return order_points<float>(positions, N, pd, scratch, order, s);
    return hipErrorInvalidValue;
}

}  // namespace plk
