// The splat of a lattice that is applied many times, as a gather.
//
// The reference splats point by point (src/PermutohedralLatticeCPU.h:306-326; its CUDA path with
// atomics, src/PermutohedralLatticeGPU.cuh:273-333).  The splat kernels of pl_kernels.hip do the
// same per wavefront: they find, on every call, which of a wavefront's points share a vertex, sum
// those in registers and add the sums with one atomic request per wavefront and vertex.  For a
// lattice that is built once and applied many times (pl_build, then pl_apply) none of that changes
// between the calls, so the build can write the transpose of the replay matrix once: for every
// vertex the list of (point, weight) that touch it, one run of a single array in vertex order
// (compressed rows).  The splat is then a gather per vertex: no election, no atomics, no zero fill
// of the value table, and sums that are added in the same order on every call.
//
// Lists differ in length by orders of magnitude (a wide kernel over a flat part of an image gives
// one vertex ten thousand rows while most have twenty), so the unit of work is a chunk of at most
// ListChunks::rows rows of one list (list_chunk_rows): a list of one chunk is summed straight into
// the value table, the chunks of a longer list into partial rows that a second, small launch adds
// up.
//
// This translation unit needs no -ffp-contract=off (nothing here decides an integer), but is
// compiled with the same flags as the others.
#include "pl_kernels.h"
#include "pl_device.h"

namespace plk {

namespace {

using namespace device;

// ------------------------------------------------------------------------------------------------
// Lists, step 1: every (point, corner) draws its place in its vertex's list.  The lanes of a
// wavefront that name the same vertex are found as in the splat (one turn per distinct vertex,
// no memory access in it); then the lowest lane of each group adds the group's size to the
// vertex's count with one returning atomic -- all of a wavefront's in flight together -- and a
// lane's place is what came back plus its rank in the group.  Rows that still hold hash cells are
// translated to vertices and written back, as the first splat after a build does.
// ------------------------------------------------------------------------------------------------
template <int D1>
__global__ __launch_bounds__(kBlock) void k_list_places(PointMap map, ReplayEntry *replay,
                                                         const int *__restrict__ cell_vertex,
                                                         unsigned *count, unsigned *places,
                                                         int max_vertices) {
    unsigned vblock;
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    const int lane = threadIdx.x & 63;

    int vertex[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) vertex[r] = n >= 0 ? replay[(size_t)r * T + t].index : -1;
    if (cell_vertex) {
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (vertex[r] >= 0) vertex[r] = cell_vertex[vertex[r]];
#pragma unroll
        for (int r = 0; r < D1; ++r)
            if (n >= 0) replay[(size_t)r * T + t].index = vertex[r];
    }
    int leader[D1], rank[D1], size[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        // (a vertex number beyond the table cannot come out of a build that fitted; such a row
        // would take no part)
        if ((unsigned)vertex[r] >= (unsigned)max_vertices) vertex[r] = -1;
        leader[r] = lane;
        rank[r] = 0;
        size[r] = 0;
        uint64_t remaining = wave_ballot(vertex[r] >= 0);
        while (remaining) {
            const int first = __builtin_ctzll(remaining);
            const uint64_t group = lanes_equal(vertex[r], lane_value(vertex[r], first)) & remaining;
            remaining &= ~group;
            if (lane_in(group)) {
                leader[r] = first;
                rank[r] = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(group >> 32),
                                                         __builtin_amdgcn_mbcnt_lo((uint32_t)group, 0u));
                size[r] = lanes_in(group);
            }
        }
    }
    unsigned base[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r)
        base[r] = (vertex[r] >= 0 && leader[r] == lane) ? atomicAdd(&count[vertex[r]], (unsigned)size[r]) : 0u;
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const unsigned b = (unsigned)__shfl((int)base[r], leader[r]);
        if (vertex[r] >= 0) places[(size_t)r * T + t] = b + (unsigned)rank[r];
    }
}

// ------------------------------------------------------------------------------------------------
// Lists, step 2: where every vertex's list starts, and where its chunks start: exclusive prefix
// sums over all n vertex numbers of the table (numbers without a vertex count zero) of the counts
// and of the chunks the counts make, both in one pass of two launches: sums of blocks of
// kScanItems items; then the scan inside each block, every workgroup adding up the sums of the
// blocks before its own.  The second launch also describes the first chunk of every list and
// names the lists that have several (workgroup by workgroup in the order the atomics give; each
// of those is summed on its own); their further chunks are described in step 3.  start[n],
// chunk_start[n]: the totals.
// ------------------------------------------------------------------------------------------------
constexpr int kScanPerThread = 8;
constexpr int kScanItems = kBlock * kScanPerThread;

// c := a thread's kScanPerThread counts from count[first ..], 0 beyond n: two loads of four where
// all exist (first is a multiple of 8), else each from an element that exists
__device__ __forceinline__ void load_counts(const unsigned *__restrict__ count, size_t first, unsigned n,
                                            unsigned (&c)[kScanPerThread]) {
    static_assert(kScanPerThread == 8, "two loads of four");
    if (first + kScanPerThread <= n) {
        const uint4 lo = *reinterpret_cast<const uint4 *>(count + first);
        const uint4 hi = *reinterpret_cast<const uint4 *>(count + first + 4);
        c[0] = lo.x, c[1] = lo.y, c[2] = lo.z, c[3] = lo.w;
        c[4] = hi.x, c[5] = hi.y, c[6] = hi.z, c[7] = hi.w;
    } else {
        unsigned x[kScanPerThread];
#pragma unroll
        for (int i = 0; i < kScanPerThread; ++i) x[i] = count[first + i < n ? first + i : 0];
#pragma unroll
        for (int i = 0; i < kScanPerThread; ++i) c[i] = first + i < n ? x[i] : 0u;
    }
}

// (rows: a power of two)
__host__ __device__ inline unsigned chunks_of(unsigned count, unsigned rows) {
    return (count + rows - 1u) >> __builtin_ctz(rows);
}

// exclusive prefix sums of one pair of values per thread over the workgroup; *total: the sums of all
__device__ __forceinline__ uint2 block_exclusive_scan(uint2 x, uint2 *total) {
    __shared__ uint2 wave_sum[kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint2 inclusive = x;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned a = (unsigned)__shfl_up((int)inclusive.x, off);
        const unsigned b = (unsigned)__shfl_up((int)inclusive.y, off);
        if (lane >= off) {
            inclusive.x += a;
            inclusive.y += b;
        }
    }
    __syncthreads();   // (wave_sum may still be read by a previous call)
    if (lane == 63) wave_sum[wave] = inclusive;
    __syncthreads();
    uint2 before = make_uint2(0u, 0u), all = make_uint2(0u, 0u);
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) {
        const uint2 s = wave_sum[w];
        before.x += w < wave ? s.x : 0u;
        before.y += w < wave ? s.y : 0u;
        all.x += s.x;
        all.y += s.y;
    }
    *total = all;
    return make_uint2(before.x + inclusive.x - x.x, before.y + inclusive.y - x.y);
}

// (also zeroes info[0], the number of long lists, which the last launch of the pass counts)
__global__ __launch_bounds__(kBlock) void k_scan_block_sums(const unsigned *__restrict__ count,
                                                             unsigned n, uint2 *block_sums,
                                                             unsigned *info, unsigned rows) {
    if (blockIdx.x == 0 && threadIdx.x == 0) info[0] = 0u;
    const size_t first = (size_t)blockIdx.x * kScanItems + (size_t)threadIdx.x * kScanPerThread;
    unsigned c[kScanPerThread];
    load_counts(count, first, n, c);
    uint2 sum = make_uint2(0u, 0u);
#pragma unroll
    for (int i = 0; i < kScanPerThread; ++i) {
        sum.x += c[i];
        sum.y += chunks_of(c[i], rows);
    }
    uint2 total;
    (void)block_exclusive_scan(sum, &total);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

// Every workgroup adds up the sums of the blocks before its own (a few hundred pairs: cheaper than
// a launch that scans them), scans its block from there, and writes per vertex the start of its
// list and of its chunks and the descriptor of its first chunk; a list of several chunks is also
// recorded in long_lists (the workgroup's long lists take one run of places there, drawn with one
// atomic: an atomic per list would queue up on the one counter).  The counts are left at
// zero, as the next build's k_list_places must find them.
__global__ __launch_bounds__(kBlock) void k_scan_starts(unsigned *count, unsigned n,
                                                         const uint2 *__restrict__ block_sums,
                                                         unsigned *start, ListChunks chunks) {
    const size_t first = (size_t)blockIdx.x * kScanItems + (size_t)threadIdx.x * kScanPerThread;
    unsigned c[kScanPerThread];
    load_counts(count, first, n, c);
    uint2 before_block = make_uint2(0u, 0u);
    for (unsigned i = threadIdx.x; i < blockIdx.x; i += kBlock) {
        const uint2 s = block_sums[i];
        before_block.x += s.x;
        before_block.y += s.y;
    }
    uint2 base;
    (void)block_exclusive_scan(before_block, &base);
    uint2 sum = make_uint2(0u, 0u);
    unsigned long_here = 0;
#pragma unroll
    for (int i = 0; i < kScanPerThread; ++i) {
        const unsigned of_v = chunks_of(c[i], chunks.rows);
        sum.x += c[i];
        sum.y += of_v;
        long_here += of_v > 1u ? 1u : 0u;
    }
    uint2 total;
    const uint2 before = block_exclusive_scan(sum, &total);
    uint2 long_total;
    const uint2 long_before = block_exclusive_scan(make_uint2(long_here, 0u), &long_total);
    __shared__ unsigned long_base;
    if (threadIdx.x == 0) long_base = long_total.x ? atomicAdd(&chunks.info[0], long_total.x) : 0u;
    __syncthreads();
    unsigned long_at = long_base + long_before.x;
    unsigned entry = base.x + before.x, chunk = base.y + before.y;
#pragma unroll
    for (int i = 0; i < kScanPerThread; ++i) {
        if (first + i < n) {
            const unsigned v = (unsigned)(first + i);
            start[v] = entry;
            chunks.chunk_start[v] = chunk;
            if (c[i]) count[v] = 0u;
            const unsigned of_v = chunks_of(c[i], chunks.rows);
            if (of_v == 1u && chunk < chunks.max_chunks) {
                chunks.chunk[chunk] = ListChunk{entry, entry + c[i], v, 1u};
            } else if (of_v > 1u) {
                if (long_at < chunks.max_long)
                    chunks.long_lists[long_at] = LongList{v, chunk, entry, entry + c[i]};
                long_at += 1u;
                // (its first chunk; the others are described by the rows that open them, in
                // k_list_fill)
                if (chunk < chunks.max_chunks)
                    chunks.chunk[chunk] = ListChunk{entry, entry + chunks.rows, v, 0u};
            }
            entry += c[i];
            chunk += of_v;
        }
    }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) {
        const uint2 all = make_uint2(base.x + total.x, base.y + total.y);
        start[n] = all.x;
        chunks.chunk_start[n] = all.y;
        chunks.info[1] = all.y < chunks.max_chunks ? all.y : chunks.max_chunks;
    }
}

// ------------------------------------------------------------------------------------------------
// Lists, step 3: every (point, corner) writes (point, weight) to its place in its vertex's list.
// ------------------------------------------------------------------------------------------------
template <int D1>
__global__ __launch_bounds__(kBlock) void k_list_fill(PointMap map,
                                                       const ReplayEntry *__restrict__ replay,
                                                       const unsigned *__restrict__ places,
                                                       const unsigned *__restrict__ start,
                                                       ListEntry *entries, int max_vertices,
                                                       size_t capacity, ListChunks chunks,
                                                       unsigned *host_info, unsigned sequence) {
    // (the last launch of the pass: how many lists have several chunks, and the chunks in all, for
    // the host, which sizes every apply's launches by them; then, behind a system-wide fence, the
    // number of the build they belong to, which the host polls for)
    if (host_info && blockIdx.x == 0 && threadIdx.x == 0) {
        host_info[0] = chunks.info[0];
        host_info[1] = chunks.info[1];
        __threadfence_system();
        __hip_atomic_store(&host_info[2], sequence, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    unsigned vblock;
    if (!block_of_points(map, 1, vblock)) return;
    const size_t t = (size_t)vblock * kBlock + threadIdx.x;
    const size_t T = (size_t)gridDim.x * kBlock;
    const int n = point_of_thread(map, vblock, threadIdx.x);
    if (n < 0) return;
    ReplayEntry e[D1];
    unsigned place[D1], first[D1];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        e[r] = replay[(size_t)r * T + t];
        place[r] = places[(size_t)r * T + t];
    }
#pragma unroll
    for (int r = 0; r < D1; ++r)
        first[r] = start[(unsigned)e[r].index < (unsigned)max_vertices ? e[r].index : 0];
#pragma unroll
    for (int r = 0; r < D1; ++r) {
        const size_t at = (size_t)first[r] + place[r];
        if ((unsigned)e[r].index < (unsigned)max_vertices && at < capacity) {
            entries[at] = ListEntry{n, e[r].weight};
            // the row that opens a further chunk of its list describes that chunk
            if (place[r] != 0u && (place[r] & (chunks.rows - 1u)) == 0u) {
                const unsigned v = (unsigned)e[r].index;
                const unsigned c = chunks.chunk_start[v] + (place[r] >> __builtin_ctz(chunks.rows));
                const unsigned from = (unsigned)at, end = start[v + 1u];
                if (c < chunks.max_chunks)
                    chunks.chunk[c] = ListChunk{from, end - from < chunks.rows ? end : from + chunks.rows, v, 0u};
            }
        }
    }
}

// The rows of a chunk and where its sums go: the vertex's row of the value table when the chunk
// is the whole list, else the chunk's partial row.  One 16-byte load.
struct ChunkWork {
    unsigned from, to;     // entries
    float *row;            // vd floats, or nullptr: no chunk
};
__device__ __forceinline__ ChunkWork chunk_work(unsigned c, unsigned n_chunks, const ListChunks &chunks,
                                                int vd, float *values) {
    ChunkWork w{0u, 0u, nullptr};
    if (c >= n_chunks) return w;
    const uint4 d = reinterpret_cast<const uint4 *>(chunks.chunk)[c];   // {from, to, vertex, whole}
    w.from = d.x;
    w.to = d.y;
    w.row = d.w ? values + (size_t)d.z * vd : chunks.partial_rows + (size_t)c * vd;
    return w;
}

// ------------------------------------------------------------------------------------------------
// The splat as a gather, up to four channels: kLanes lanes per chunk take every kLanes-th of its
// rows, four each per turn with all their loads in flight (the entries, then the input rows they
// name, each row one request), and the lanes' sums are added across the group.  The row of every
// vertex is written whole, so the value table needs no zero fill.
// ------------------------------------------------------------------------------------------------
constexpr int kLanes = 8;      // lanes per chunk
constexpr int kInFlight = 4;   // entries per lane and turn

// An input row of IN floats, read with one request (rows of three floats are only aligned to four
// bytes, which a 12-byte load allows)
template <int IN>
struct alignas(IN == 3 ? 4 : 4 * IN) InputRow {
    float c[IN];
};

// IN: channels of an input row, VD - 1 (the last channel of the vertex row is the sum of the bare
// weights) or VD
template <int VD, int IN>
__global__ __launch_bounds__(kBlock) void k_splat_gather(ListChunks chunks, unsigned n_chunks,
                                                          const ListEntry *__restrict__ entries,
                                                          const float *__restrict__ input,
                                                          float *values) {
    static_assert(VD >= 2 && VD <= 4 && (IN == VD || IN == VD - 1), "the rows are gathered in registers");
    const unsigned sub = threadIdx.x % kLanes;
    constexpr unsigned per_block = kBlock / kLanes;
    constexpr unsigned kTurn = kLanes * kInFlight;
    // (chunks follow the vertex numbers, which follow the image: every XCD takes one contiguous
    // range of them, so that the input rows its chunks share stay in its L2)
    const unsigned first_block = xcd_contiguous_block(blockIdx.x, gridDim.x, 1);
    for (unsigned c0 = first_block * per_block; c0 < n_chunks; c0 += gridDim.x * per_block) {
        const ChunkWork work = chunk_work(c0 + threadIdx.x / kLanes, n_chunks, chunks, VD, values);
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        // A turn's entries are asked for one turn ahead, together with the rows of the turn before:
        // a turn then waits for one round trip to memory, not two.  (An entry past the end of the
        // chunk reads the chunk's first and counts with weight zero.)
        ListEntry e[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            const unsigned i = work.from + (unsigned)u * kLanes + sub;
            e[u] = entries[i < work.to ? i : work.from];
        }
        // (the lanes of a chunk leave the loop together: what they exchange below is complete)
        for (unsigned turn = work.from; turn < work.to; turn += kTurn) {
            InputRow<IN> x[kInFlight];
            float w[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                x[u] = reinterpret_cast<const InputRow<IN> *>(input)[e[u].point];
                w[u] = turn + (unsigned)u * kLanes + sub < work.to ? e[u].weight : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const unsigned i = turn + kTurn + (unsigned)u * kLanes + sub;
                e[u] = entries[i < work.to ? i : work.from];
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
#pragma unroll
                for (int j = 0; j < VD; ++j) acc[j] += w[u] * (j < IN ? x[u].c[j] : 1.0f);
            }
        }
#pragma unroll
        for (int j = 0; j < VD; ++j) {
#pragma unroll
            for (int off = 1; off < kLanes; off <<= 1) acc[j] += __shfl_xor(acc[j], off);
        }
        if (work.row && sub == 0) {
#pragma unroll
            for (int j = 0; j < VD; ++j) work.row[j] = acc[j];
        }
    }
}

// More than four channels: L lanes per chunk (4, 8 or 16), lane i on the channels 4i .. 4i+3 of
// every row of the chunk.  What bounds a gather of rows of many channels is the number of load
// instructions (the memory pipeline takes 16 cycles to look at the 64 addresses of one, whatever
// their width), so a lane reads its four channels of an input row with one 16-byte load; rows
// need only be aligned to four bytes for that.  The lane on the row's last channels reads the
// row's last four instead (no load leaves the row) and its sums are shifted back at the end.  The
// lanes first read the whole chunk's entries, kChannelChunk / L each, and hand them round.
// Channels past the input are the homogeneous one: the sum of the bare weights.
constexpr int kChannelChunk = (int)kListChunkManyChannels;   // rows of a chunk at most (vd > 4)


struct alignas(4) FourFloats {
    float c[4];
};
__device__ __forceinline__ float pick(const float (&x)[4], int i) {
    return i == 0 ? x[0] : i == 1 ? x[1] : i == 2 ? x[2] : x[3];
}

template <int L>
__global__ __launch_bounds__(kBlock) void k_splat_gather_channels(ListChunks chunks, unsigned n_chunks,
                                                                   int vd,
                                                                   const ListEntry *__restrict__ entries,
                                                                   const float *__restrict__ input,
                                                                   int in_channels, float *values) {
    constexpr unsigned per_block = kBlock / L;
    constexpr int E = kChannelChunk / L;          // entries per lane
    constexpr int kBatch = 16;                    // rows in flight (8: 6 % slower, 32: 2 %)
    const int sub = threadIdx.x % L;
    const unsigned first_block = xcd_contiguous_block(blockIdx.x, gridDim.x, 1);
    for (unsigned c0 = first_block * per_block; c0 < n_chunks; c0 += gridDim.x * per_block) {
        const ChunkWork work = chunk_work(c0 + threadIdx.x / L, n_chunks, chunks, vd, values);
        const unsigned rows = work.to - work.from;
        // (entries past the end of the chunk: its first row, weight zero)
        ListEntry e[E];
#pragma unroll
        for (int u = 0; u < E; ++u) {
            const unsigned mine = work.from + (unsigned)(u * L + sub);
            e[u] = entries[mine < work.to ? mine : work.from];
            if (mine >= work.to) e[u].weight = 0.0f;
        }
        for (int ch0 = 0; ch0 < vd; ch0 += 4 * L) {
            const int c = ch0 + 4 * sub;
            const int start = c < in_channels ? (c < in_channels - 4 ? c : in_channels - 4) : 0;
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f}, weights = 0.0f;
#pragma unroll
            for (int row0 = 0; row0 < kChannelChunk; row0 += kBatch) {
                if ((unsigned)row0 < rows) {
                    FourFloats x[kBatch];
                    float w[kBatch];
#pragma unroll
                    for (int k = 0; k < kBatch; ++k) {
                        // (row row0 + k of the chunk is entry (row0 + k) / L of lane (row0 + k) % L)
                        const int p = __shfl(e[(row0 + k) / L].point, (row0 + k) % L, L);
                        w[k] = __shfl(e[(row0 + k) / L].weight, (row0 + k) % L, L);
                        x[k] = *reinterpret_cast<const FourFloats *>(
                            input + (size_t)p * in_channels + start);
                    }
#pragma unroll
                    for (int k = 0; k < kBatch; ++k) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) acc[j] += w[k] * x[k].c[j];
                        weights += w[k];
                    }
                }
            }
            if (work.row) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (c + j < vd)
                        work.row[c + j] = c + j < in_channels ? pick(acc, c - start + j) : weights;
            }
        }
    }
}

// The lists of more than one chunk: the vertex's row := the sum of its chunks' partial rows.  A
// wavefront per list and block of 32 channels: lane (h, c) adds channel c of every second chunk,
// kSumInFlight loads in flight (one round of loads for a list of up to 2 * kSumInFlight chunks),
// and the two halves are added at the end.  Which lane adds which chunks depends on the list
// alone: the same order on every call.
constexpr int kSumInFlight = 16;

__global__ __launch_bounds__(kBlock) void k_sum_partial_rows(ListChunks chunks, unsigned n_long, int vd,
                                                              float *values) {
    const int lane = threadIdx.x & 63, half = lane >> 5, sub = lane & 31;
    const unsigned waves = gridDim.x * (kBlock / 64);
    for (unsigned i = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); i < n_long; i += waves) {
        const LongList list = chunks.long_lists[i];
        const unsigned from = list.chunk_from;
        unsigned to = from + chunks_of(list.to - list.from, chunks.rows);
        if (to > chunks.max_chunks) to = chunks.max_chunks;
        for (int c0 = 0; c0 < vd; c0 += 32) {
            const int c = c0 + sub;
            float acc[kSumInFlight];
#pragma unroll
            for (int u = 0; u < kSumInFlight; ++u) acc[u] = 0.0f;
            for (unsigned k = from + (unsigned)half; k < to; k += 2u * kSumInFlight) {
#pragma unroll
                for (int u = 0; u < kSumInFlight; ++u) {
                    // (every load is issued, from a row that exists, and counted or not
                    // afterwards: loads under a condition would wait for one another)
                    const unsigned ku = k + 2u * (unsigned)u;
                    const bool counts = ku < to && c < vd;
                    const float x = chunks.partial_rows[(size_t)(ku < to ? ku : from) * vd +
                                                        (c < vd ? c : 0)];
                    acc[u] += counts ? x : 0.0f;
                }
            }
#pragma unroll
            for (int width = kSumInFlight / 2; width >= 1; width /= 2)
#pragma unroll
                for (int u = 0; u < width; ++u) acc[u] += acc[u + width];
            float sum = acc[0];
            sum += __shfl_xor(sum, 32);
            if (half == 0 && c < vd) values[(size_t)list.vertex * vd + c] = sum;
        }
    }
}

}  // namespace

size_t vertex_list_scan_blocks(int max_vertices) {
    return ((size_t)max_vertices + kScanItems - 1) / kScanItems;
}
size_t vertex_list_max_chunks(int max_vertices, size_t rows) {
    // (every vertex's list ends in a chunk that may be short; the rest are full ones)
    return (size_t)max_vertices + rows / kListChunkManyChannels + 1;
}
size_t vertex_list_max_long(size_t rows) { return rows / kListChunkManyChannels + 1; }

hipError_t build_vertex_lists(int pd, const PointMap &map, ReplayEntry *replay, const int *cell_vertex,
                              int max_vertices, const VertexLists &lists, unsigned *host_info,
                              unsigned sequence, hipStream_t s) {
    if (max_vertices <= 0 || map.n_blocks == 0) return hipSuccess;
    // (lists.count is all zeros: filled so when it was allocated, left so by every k_scan_starts)
    const dim3 block(kBlock), grid(map.n_blocks);
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_list_places<PD + 1>), grid, block, 0, s, map, replay,
                                           cell_vertex, lists.count, lists.places, max_vertices));
    const unsigned n = (unsigned)max_vertices;
    const unsigned scan_blocks = (unsigned)vertex_list_scan_blocks(max_vertices);
    uint2 *block_sums = reinterpret_cast<uint2 *>(lists.block_sums);
    hipLaunchKernelGGL(k_scan_block_sums, dim3(scan_blocks), block, 0, s, lists.count, n, block_sums,
                       lists.chunks.info, lists.chunks.rows);
    hipLaunchKernelGGL(k_scan_starts, dim3(scan_blocks), block, 0, s, lists.count, n, block_sums,
                       lists.start, lists.chunks);
    PLK_DISPATCH_PD(pd, hipLaunchKernelGGL((k_list_fill<PD + 1>), grid, block, 0, s, map, replay,
                                           lists.places, lists.start, lists.entries, max_vertices,
                                           lists.capacity, lists.chunks, host_info, sequence));
    return hipGetLastError();
}

hipError_t splat_gather(int vd, const VertexLists &lists, unsigned n_chunks, unsigned n_long,
                        const float *input, int in_channels, float *values, hipStream_t s) {
    if (n_chunks == 0) return hipSuccess;
    const dim3 block(kBlock);
#define PLK_GATHER(VD)                                                                               \
    case VD:                                                                                        \
        if (in_channels == VD)                                                                      \
            hipLaunchKernelGGL((k_splat_gather<VD, VD>), dim3(blocks_for(n_chunks, kBlock / kLanes)),\
                               block, 0, s, lists.chunks, n_chunks, lists.entries, input, values);\
        else if (in_channels == VD - 1)                                                             \
            hipLaunchKernelGGL((k_splat_gather<VD, VD - 1>),                                         \
                               dim3(blocks_for(n_chunks, kBlock / kLanes)), block, 0, s,            \
                               lists.chunks, n_chunks, lists.entries, input, values);  \
        else                                                                                        \
            return hipErrorInvalidValue;                                                            \
        break;
    switch (vd) {
        PLK_GATHER(2) PLK_GATHER(3) PLK_GATHER(4)
        default:
            if (lists.chunks.rows > (unsigned)kChannelChunk) return hipErrorInvalidValue;
            if (in_channels < 4) return hipErrorInvalidValue;
            if (vd <= 16)
                hipLaunchKernelGGL(k_splat_gather_channels<4>, dim3(blocks_for(n_chunks, kBlock / 4)),
                                   block, 0, s, lists.chunks, n_chunks, vd, lists.entries, input,
                                   in_channels, values);
            else if (vd <= 32)
                hipLaunchKernelGGL(k_splat_gather_channels<8>, dim3(blocks_for(n_chunks, kBlock / 8)),
                                   block, 0, s, lists.chunks, n_chunks, vd, lists.entries, input,
                                   in_channels, values);
            else
                hipLaunchKernelGGL(k_splat_gather_channels<16>, dim3(blocks_for(n_chunks, kBlock / 16)),
                                   block, 0, s, lists.chunks, n_chunks, vd, lists.entries, input,
                                   in_channels, values);
            break;
    }
#undef PLK_GATHER
    if (n_long)
        hipLaunchKernelGGL(k_sum_partial_rows, dim3(blocks_for(n_long, kBlock / 64)), block, 0, s,
                           lists.chunks, n_long, vd, values);
    return hipGetLastError();
}

}  // namespace plk
