// gfx950 kernels of the permutohedral-lattice filter for T = double, the other value type the
// reference registers (src/LatticeFilterKernel.cpp:196-208).
//
// The lattice itself (keys, hash table, vertex numbering, neighbour table) is what the float path
// builds: the build kernel is instantiated for double positions in pl_kernels.hip, and the
// numbering and neighbour passes do not look at values.  What is here are the passes that touch
// values: splat, blur and slice on rows of doubles, the feature builder and the per-point dump.
// The splat here serves pl_apply_f64 and more than four channels (with up to four, pl_filter_f64
// splats in the merging build kernel, as the float path does); the blur kernels here serve more
// than four channels (up to four use the float path's row kernels over the value type).
//
// Arithmetic follows the reference CPU path with T = double: the three-tap blur and the reciprocal
// of the slice are double expressions there for every T.  The splat adds in a different order
// than the sequential CPU loop, so values agree to rounding (1e-16 relative per addition), not
// bit for bit; the integers of the lattice agree exactly.
#include "pl_device.h"
#include "pl_kernels.h"

namespace plk {

namespace {

using namespace device;

// Splat.  As in the float path the contributions of a wavefront to one vertex are summed before
// they leave it (points that are neighbours in the image share vertices, and what bounds a splat
// is the number of atomic requests): for each distinct vertex of the wavefront and each channel
// four channels at a time are summed over the members, and the first four lanes add the four
// sums to the vertex row with one atomic instruction.  replay rows and weights are stored in thread order, [r][t],
// like the float path's.
template <int D1>
__global__ __launch_bounds__(kBlock) void k_splat_f64(int vd, PointMap map,
                                                       const double *__restrict__ input,
                                                       int in_channels, ReplayEntry *replay,
                                                       const double *__restrict__ weights,
                                                       const int *__restrict__ cell_vertex,
                                                       double *values, int xcd_aware) {
    unsigned vblock;
    if (!block_of_points(map, xcd_aware, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t n_slots = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    const int lane = threadIdx.x & 63;
    // every lane stays for the sums; lanes without a point, or whose keys the build could not
    // place (it has said so), carry vertex -1 and belong to no group
    int vertex[D1];
    double weight[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        vertex[r] = n >= 0 ? replay[(size_t)r * n_slots + t].index : -1;
        weight[r] = weights[(size_t)r * n_slots + t];
    }
    if (cell_vertex) {
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            if (vertex[r] >= 0) {
                vertex[r] = cell_vertex[vertex[r]];
                replay[(size_t)r * n_slots + t].index = vertex[r];
            }
        }
    }
    const double *value = input + (size_t)(n >= 0 ? n : 0) * in_channels;
    // four channels at a time: their values are loaded once, then every corner's groups are
    // walked with the four sums of a group going to lanes 0..3 and out in one instruction
    for (int first_channel = 0; first_channel < vd; first_channel += 4) {
        const int channels = vd - first_channel < 4 ? vd - first_channel : 4;
        double val[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int j = first_channel + c;
            // the homogeneous channel is the bare weight when vd-1 channels are given
            val[c] = (n >= 0 && j < in_channels) ? value[j] : 1.0;
        }
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            const int v = vertex[r];
            const double w = weight[r];
            const double term[4] = {w * val[0], w * val[1], w * val[2], w * val[3]};
            const int my_channel = channel_of_quad_lane(lane);
            uint64_t remaining = wave_ballot(v >= 0);
            while (remaining) {
                const int first = __builtin_ctzll(remaining);
                const int k = lane_value(v, first);
                const uint64_t group = lanes_equal(v, k);
                remaining &= ~group;
                const double sum = wave_sums_to_quads_f64(lane_in(group), term, lane);
                if (lane < 4 && my_channel < channels)
                    atomicAdd(values + (size_t)k * vd + first_channel + my_channel, sum);
            }
        }
    }
}

// Slice, up to eight channels: one thread per point, the row sums in registers.
template <int D1>
__global__ __launch_bounds__(kBlock) void k_slice_point_f64(int vd, PointMap map,
                                                             const ReplayEntry *__restrict__ replay,
                                                             const double *__restrict__ weights,
                                                             const int *__restrict__ cell_vertex,
                                                             const double *__restrict__ values,
                                                             double *__restrict__ output,
                                                             int normalize) {
    constexpr int kMaxChannels = 8;
    // each XCD takes one contiguous range of the tiles, whose vertices' rows are then in its L2
    unsigned vblock;
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t n_slots = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    if (n < 0) return;
    int vertex[D1];
    double weight[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        vertex[r] = replay[(size_t)r * n_slots + t].index;
        weight[r] = weights[(size_t)r * n_slots + t];
    }
    if (cell_vertex) {
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (vertex[r] >= 0) vertex[r] = cell_vertex[vertex[r]];
    }
    double sum[kMaxChannels];
#pragma unroll
    for (int j = 0; j < kMaxChannels; ++j) sum[j] = 0.0;
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        if (vertex[r] < 0) continue;
        const double *row = values + (size_t)vertex[r] * vd;
#pragma unroll
        for (int j = 0; j < kMaxChannels; ++j)
            if (j < vd) sum[j] += weight[r] * row[j];
    }
    if (normalize) {
        double homogeneous = 0.0;
#pragma unroll
        for (int j = 0; j < kMaxChannels; ++j)
            if (j == vd - 1) homogeneous = sum[j];
        const double scale = 1.0 / homogeneous;
#pragma unroll
        for (int j = 0; j < kMaxChannels; ++j)
            if (j < vd - 1) output[(size_t)n * (vd - 1) + j] = sum[j] * scale;
    } else {
#pragma unroll
        for (int j = 0; j < kMaxChannels; ++j)
            if (j < vd) output[(size_t)n * vd + j] = sum[j];
    }
}

// More channels: one thread per point and output channel, its channel's sum and the homogeneous
// channel's.
template <int D1>
__global__ __launch_bounds__(kBlock) void k_slice_f64(int vd, PointMap map,
                                                       const ReplayEntry *__restrict__ replay,
                                                       const double *__restrict__ weights,
                                                       const int *__restrict__ cell_vertex,
                                                       const double *__restrict__ values,
                                                       double *__restrict__ output, int normalize) {
    const int out_channels = normalize ? vd - 1 : vd;
    // each XCD takes one contiguous range of the tiles, whose vertices' rows are then in its L2
    unsigned vblock;
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t n_slots = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    if (n < 0) return;
    const int j = blockIdx.y;
    double sum = 0.0, homogeneous = 0.0;
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        int v = replay[(size_t)r * n_slots + t].index;
        if (v < 0) continue;
        if (cell_vertex) v = cell_vertex[v];
        const double w = weights[(size_t)r * n_slots + t];
        const double *row = values + (size_t)v * vd;
        sum += w * row[j];
        homogeneous += w * row[vd - 1];
    }
    output[(size_t)n * out_channels + j] = normalize ? sum * (1.0 / homogeneous) : sum;
}

template <int PD>
__global__ __launch_bounds__(kBlock) void k_debug_simplex_f64(const double *__restrict__ positions,
                                                               int N, ScaleFactor64 scale,
                                                               short *rem0, short *rank, short *keys,
                                                               double *barycentric) {
    constexpr int D1 = PD + 1;
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= N) return;
    double pos[PD];
#pragma unroll
    for (int i = 0; i < PD; ++i) pos[i] = positions[(size_t)n * PD + i];
    Simplex<PD, double> s;
    enclosing_simplex<PD>(pos, scale, s);
#pragma unroll
    for (int i = 0; i < D1; ++i) {
        if (rem0) rem0[(size_t)n * D1 + i] = (short)(s.q[i] * D1);
        if (rank) rank[(size_t)n * D1 + i] = (short)s.rank[i];
        if (barycentric) barycentric[(size_t)n * D1 + i] = s.weight[i];
    }
    if (keys) {
#pragma unroll
        for (int r = 0; r < D1; ++r) {
            int q[PD];
            vertex_q<PD>(s, r, q);
#pragma unroll
            for (int i = 0; i < PD; ++i)
                keys[((size_t)n * D1 + r) * PD + i] = (short)(q[i] * D1 + r);
        }
    }
}

// reference: compute_kernel_cpu<double>, src/PermutohedralLatticeCPU.h:452-474
__global__ __launch_bounds__(kBlock) void k_positions_f64(const double *__restrict__ reference,
                                                           double *__restrict__ positions, int N,
                                                           int rc, int nsd, SpatialDims dims,
                                                           double spatial_std, double feature_std) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= N) return;
    const int pd = nsd + rc;
    double *row = positions + (size_t)n * pd;
    int stride = 1;
    for (int s = nsd - 1; s >= 0; --s) {
        const int coord = (n / stride) % dims.v[s];
        row[s] = (double)coord / spatial_std;
        stride *= dims.v[s];
    }
    for (int c = 0; c < rc; ++c) row[nsd + c] = reference[(size_t)n * rc + c] / feature_std;
}

}  // namespace

hipError_t splat_f64(int pd, int vd, const PointMap &map, const double *input, int in_channels,
                     ReplayEntry *replay, const double *weights, const int *cell_vertex,
                     double *values, int xcd_aware, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL(k_splat_f64<PD + 1>, dim3(map.n_blocks), dim3(kBlock), 0,
                                           s, vd, map, input, in_channels, replay, weights,
                                           cell_vertex, values, xcd_aware));
    return hipGetLastError();
}

hipError_t slice_f64(int pd, int vd, const PointMap &map, const ReplayEntry *replay,
                     const double *weights, const int *cell_vertex, const double *values,
                     double *output, int normalize, hipStream_t s) {
    if (map.n_blocks == 0) return hipSuccess;
    if (vd >= 2 && vd <= 4)
        return slice_rows_f64(pd, vd, map, replay, weights, cell_vertex, values, output, normalize, s);
    if (vd <= 8) {
        PLK_DISPATCH_PD(pd, hipLaunchKernelGGL(k_slice_point_f64<PD + 1>, dim3(map.n_blocks),
                                               dim3(kBlock), 0, s, vd, map, replay, weights,
                                               cell_vertex, values, output, normalize));
        return hipGetLastError();
    }
    const unsigned out_channels = (unsigned)(normalize ? vd - 1 : vd);
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL(k_slice_f64<PD + 1>, dim3(map.n_blocks, out_channels),
                                           dim3(kBlock), 0, s, vd, map, replay, weights,
                                           cell_vertex, values, output, normalize));
    return hipGetLastError();
}

hipError_t debug_simplex_f64(int pd, const double *positions, int N, const ScaleFactor64 &scale,
                             short *rem0, short *rank, short *keys, double *barycentric,
                             hipStream_t s) {
    if (N <= 0) return hipSuccess;
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL(k_debug_simplex_f64<PD>, dim3(blocks_for((size_t)N)),
                                           dim3(kBlock), 0, s, positions, N, scale, rem0, rank,
                                           keys, barycentric));
    return hipGetLastError();
}

hipError_t compute_positions_f64(const double *reference, double *positions, int N,
                                 int n_ref_channels, int n_spatial_dims, const SpatialDims &dims,
                                 double spatial_std, double feature_std, hipStream_t s) {
    if (N <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_positions_f64, dim3(blocks_for((size_t)N)), dim3(kBlock), 0, s, reference,
                       positions, N, n_ref_channels, n_spatial_dims, dims, spatial_std,
                       feature_std);
    return hipGetLastError();
}

}  // namespace plk
