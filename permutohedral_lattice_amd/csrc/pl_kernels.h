// Internal launch interface between the host-side lattice object (pl_api.cpp) and the gfx950
// kernels (pl_kernels.hip for float values, pl_kernels_f64.hip for double values).  Not part of the public ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace plk {

constexpr int kMaxPd = 8;          // feature dimensions the build/neighbour kernels are instantiated for
constexpr int kMaxSpatialDims = 8;
constexpr uint64_t kEmptyCell = ~0ull;
constexpr uint32_t kMaxCells = 1u << 28;   // cells are addressed by 32-bit byte offsets (8 bytes each)

// bits of Counters::flags
enum : int {
    kFlagTableFull = 1,   // a probe sequence wrapped, or more vertices were created than the table may hold
    kFlagKeyRange = 2,    // a lattice coordinate does not fit its field of the key (packed key: the build
                          // is repeated with keys of two words; those: it is no short)
    kFlagTileFull = 4,    // a workgroup of the merging build has more distinct keys than its LDS table holds
};

// Device-side state of one build.  Kernels after the build read the vertex counts from here, so
// the host never has to wait for them between launches.
//
// Vertex numbers.  The merging build can number its vertices itself: a workgroup draws a run of
// numbers for the vertices it created from the counter of its segment (one atomic per workgroup;
// the segment is the eighth of the image the workgroup lies in, which one XCD builds and later
// walks), and segment x owns the numbers from x * segment_stride(max_vertices, 8) on: eight dense
// runs in the order in which the workgroups of an eighth got there, n_segments == 8.  A small
// table has one segment.  An atomic on one address takes about 50 ns and the next one waits for
// it, so this is for builds of a few thousand workgroups.  Otherwise the numbering is left to
// number_vertices, which gives the numbers 0 .. vertices-1 (n_segments == 0).
constexpr int kMaxSegments = 64;
struct Counters {
    unsigned int vertices;   // total (may exceed what the table can hold)
    int flags;
    // how the build spread its keys over the table (KeyRegions in pl_device.h), written by the
    // build for the passes that look keys up after it: they must not read the caller's positions
    // again, which only have to stay valid until the build has run
    float region_lo, region_per_unit;
    int n_segments;
    // (a counter per 128 bytes: atomics on one line queue up in one memory channel, whatever
    // address in the line they name.  Each line also says how the vertices are numbered, and
    // after the numbering pass every line holds the total: a pass over the vertices learns what
    // its XCD walks from one line.)
    struct alignas(128) PaddedCount {
        unsigned int n;
        int n_segments;
    };
    PaddedCount segment_count[kMaxSegments];
    // rows of sums for vertices of other workgroups (CreatedLists), counted by every eighth
    // workgroup of a build that numbers its vertices
    PaddedCount foreign_rows_sampled;
};
constexpr unsigned kForeignSampling = 8;
__host__ __device__ inline uint32_t segment_stride(uint32_t max_vertices, int n_segments) {
    return max_vertices / (uint32_t)(n_segments > 0 ? n_segments : 1);
}
// Segments a merging build of `workgroups` workgroups that numbers its vertices uses with a table
// for max_vertices: none smaller than 2048 numbers (a workgroup can create 512 vertices); eight,
// or sixty-four when a segment of eight would serve more than a thousand workgroups.
inline int segments_for(uint32_t max_vertices, unsigned workgroups) {
    if (max_vertices / 8u < 2048u) return 1;
    return workgroups > 8192u && max_vertices / (uint32_t)kMaxSegments >= 2048u ? kMaxSegments : 8;
}

// What the build (or the numbering pass) writes to pinned host memory about the build.
struct HostStatus {
    int num_vertices;
    int flags;
    int max_segment;   // vertices in the fullest segment (num_vertices when there are none)
    int n_segments;
    int foreign_rows;  // CreatedLists rows of a build that numbered its vertices (an estimate)
    // written last, behind a system-wide fence: the number of the build the fields above belong
    // to.  The host, which holds the struct in pinned memory, polls this word instead of waiting
    // for an event behind the kernel (an event between two kernels of a stream keeps the second
    // from starting for some microseconds).
    unsigned sequence;
};
// Where a build reports to, and as which build.
struct HostReport {
    HostStatus *status;
    unsigned sequence;
};

// Per-vertex and per-cell tables of a lattice (all sized by the hash table): vertex v has key
// vertex_keys[v] and sits in hash cell vertex_cell[v]; cell_vertex[cell] is the inverse;
// neighbours[a*max_vertices + v] holds v's two neighbours along blur axis a (-1: none).
struct VertexTables {
    int *cell_vertex;
    uint64_t *vertex_keys;
    int *vertex_cell;
    int2 *neighbours;
    int max_vertices;
};

// Vertices a table of n_cells may hold (load factor 3/4): beyond that probe sequences get long,
// below 1/3 the table no longer fits the L2 next to everything else.
__host__ __device__ inline uint32_t max_vertices_for(uint32_t n_cells) { return n_cells / 4u * 3u; }

// One row of the replay matrix (reference: MatrixEntry, src/PermutohedralLatticeCPU.h:187-190):
// which vertex a point's simplex corner is (hash cell until the first splat) and its weight.
struct ReplayEntry {
    int index;
    float weight;
};

struct ScaleFactor {
    float v[kMaxPd];
};
struct ScaleFactor64 {
    double v[kMaxPd];
};
// What the build reads and writes for double values: positions N x pd, and the barycentric
// weights in the layout of the replay rows.
struct Points64 {
    const double *positions;
    double *weights;
    ScaleFactor64 scale;
};

struct SpatialDims {
    int v[kMaxSpatialDims];
};

// Per-workgroup lists, `stride` uint4 per workgroup of the build (in the build's virtual order).
// A build that leaves the numbering to number_vertices lists what it created: workgroup b has
// block_count[b] new vertices, one uint4 each: (key low word, key high word, hash cell, 0);
// chunk_count[c] is the sum over the kBlocksPerChunk workgroups of chunk c and must be zero
// before the build.
// A merging build that numbers its vertices itself lists, when it splats, the rows of sums it
// holds for vertices that another workgroup created (their numbers are not known yet):
// block_count[b] of them, the rows (four values each) from the start of the workgroup's part and
// their hash cells, as ints, behind kTileSlots rows.  neighbours() adds them to the value table.
constexpr int kBlocksPerChunk = 64;
constexpr int kTileSlots = 512;    // LDS slots of a workgroup of the merging build
struct CreatedLists {
    uint4 *entries;
    int *block_count;
    int *chunk_count;
    int stride;
};
// uint4 a workgroup's part must hold: its 256 * (pd+1) possible vertices, or kTileSlots rows of
// four values and as many cells
inline int created_list_stride(int pd, bool f64) {
    const int vertices = 256 * (pd + 1);
    const int rows = kTileSlots * (f64 ? 2 : 1) + kTileSlots / 4;
    return vertices > rows ? vertices : rows;
}

// What the merging build needs to number its vertices: the per-vertex tables and the value table
// (rows of value_words floats: the rows of the vertices a workgroup created receive its sums when
// the build splats, zeros when not).  n_segments == 0: it does not number them but lists them and
// adds its sums to the rows of the hash cells, like the plain build, and number_vertices follows.
struct InBuildNumbering {
    int *cell_vertex;
    uint64_t *vertex_keys;
    int *vertex_cell;
    int2 *neighbours;
    int max_vertices;
    void *values;
    int value_words;
    int n_segments;       // 0, 1, 8 or 64 (segments_for)
};

// Where the feature vector of a point comes from: the row of a positions array, or, with
// positions == nullptr, the point's grid coordinates divided by spatial_std followed by its
// reference channels divided by feature_std (what compute_positions would have written).
struct PointFeatures {
    const float *positions;   // N x pd
    const float *reference;   // N x n_reference_channels
    int n_spatial_dims, n_reference_channels;
    SpatialDims dims;         // slowest first, the last runs fastest
    float spatial_std, feature_std;
};

// How threads are laid over the points (see point_of_thread in pl_kernels.hip).
struct PointMap {
    int N;
    int mode;        // 0: 256 consecutive points per workgroup; 1: 256 consecutive entries of
                     // `order`; 2: 16x16 tiles; 3: 4x8x8 tiles
    int dims[3];     // grid extents, slowest first (leading extents folded into dims[0])
    int tiles[3];    // workgroup tiles along each extent
    unsigned n_blocks;
    // mode 1 (order_by_locality): n_blocks * 256 entries, the points with neighbours in space next
    // to each other, -1 where a place is left empty; and how many of the workgroups have any
    // (in device memory: the launch is enqueued before the order is known)
    const int *order;
    const unsigned *n_tiles;
};

// Where feature 0 of the first and of the last point can be read (one of the two pointers, or
// the two values themselves when the features are built on the fly), for spreading the keys over
// the hash table by it: see KeyRegions in pl_device.h.  enabled == 0: plain hashing.
struct RegionSource {
    const float *positions;
    const double *positions64;
    const float *range0;   // or: the smallest and the largest feature 0 of all points, in device memory
    float first, last;
    float scale0;          // scale factor of feature 0
    int N, pd;
    int enabled;
};

// Bits per lattice coordinate in the packed 64-bit key, and the coordinate range that fits.
int key_field_bits(int pd);

// n_dims < 2 or dims == nullptr: no grid, consecutive points.
PointMap make_point_map(int N, int n_dims, const int *dims);

// Hash cells := empty.
hipError_t clear_table(uint64_t *cell_keys, uint32_t n_cells, hipStream_t s);

// Stage 1+2: per point embed, enclosing simplex, barycentric weights, then insertion of the pd+1
// vertex keys.  The replay arrays hold (pd+1) rows of T = map.n_blocks*256 entries in thread
// order: replay[r*T+t] := hash cell of vertex r of the point of thread t (-1: no point) and its
// barycentric weight.  The lane whose insertion created a vertex appends its cell and key to
// its workgroup's list in created_lists.
// splat_vd != 0 (allowed when build_can_splat(vd)): the kernel also splats `input`
// (in_channels per point) into cell_values[cell*vd ..], rows addressed by hash cell;
// number_vertices then moves them into the dense value table.
// numbering != nullptr: the merging build (the points are a grid).  With numbering->n_segments
// != 0 it numbers its vertices itself (Counters, CreatedLists, InBuildNumbering): no
// number_vertices follows it, cell_values is not used, and neighbours() must be given the lists
// when the build splatted.
// wide_keys (pd >= 5, plain build only): keys of two words, for lattices whose coordinates do not
// fit the packed key but are shorts, as the reference's keys are: cell_keys then holds two words
// per cell (both all ones when empty), the lists two entries per vertex, and number_vertices,
// neighbours and export_keys must be told.
bool build_can_splat(int vd);
hipError_t build(int pd, const PointFeatures &features, const PointMap &map, const ScaleFactor &scale,
                 uint64_t *cell_keys, uint32_t n_cells, Counters *counters, ReplayEntry *replay,
                 int xcd_aware, int splat_vd, const float *input,
                 int in_channels, float *cell_values, const CreatedLists &created_lists,
                 const RegionSource &regions, const InBuildNumbering *numbering, bool wide_keys,
                 hipStream_t s);

// The build for double values: the same kernel on points.positions with points.scale; replay[]
// receives the cells (and the weights rounded to float), points.weights[r*T+t] the weights.
hipError_t build_f64(int pd, const Points64 &points, const PointMap &map, uint64_t *cell_keys,
                     uint32_t n_cells, Counters *counters, ReplayEntry *replay, int xcd_aware,
                     const CreatedLists &created_lists, const RegionSource &regions,
                     const InBuildNumbering *numbering, int splat_vd, const double *input,
                     int in_channels, double *cell_values, bool wide_keys, hipStream_t s);

// Dense vertex numbers in the order of the build's workgroups (same map as the build):
// cell_vertex[cell] := v, vertex_keys[v] := key, vertex_cell[v] := cell,
// neighbours[a][v] := (-1, -1) for a <= pd, counters->vertices := M, and the vertex's row of
// `values` := 0, or, with cell_values != nullptr, := the row cell_values[cell*vd ..], which is
// zeroed.  Copies M and the flags to *host_status, zeroes *next_counters and
// next_chunk_count[0 .. n_chunks).
hipError_t number_vertices(int pd, const PointMap &map, const CreatedLists &lists,
                           int *next_chunk_count, unsigned n_chunks, const VertexTables &vertices,
                           float *values, int vd, float *cell_values, Counters *counters, Counters *next_counters,
                           HostReport host_report, bool wide_keys, hipStream_t s);

// neighbours[a*max_vertices+v] := vertex indices of v's two neighbours along blur axis a, for v
// below the vertex count; entries of absent neighbours keep their -1.
// launch_vertices (here and below): the vertex count the grid is sized for; any count is
// covered, a wrong estimate only costs time.
// Keys are looked for where the build put them: counters->region_* as the build left them.
// foreign_rows != nullptr (after a merging build that numbered its vertices and splatted): the
// launch also adds the rows the build's n_lists workgroups listed to `values` (rows of vd floats
// or doubles).
// report != nullptr (after a merging build that numbered its vertices): the launch also sums the
// segments' counts in *report (the build's counters, == counters), copies them and the flags to
// *host_status and zeroes *next_counters, as number_vertices does otherwise.
hipError_t neighbours(int pd, const VertexTables &vertices, const Counters *counters,
                      const uint64_t *cell_keys, uint32_t n_cells, int launch_vertices,
                      const CreatedLists *foreign_rows, unsigned n_lists, void *values, int vd,
                      bool values_are_double, Counters *report, Counters *next_counters,
                      HostReport host_report, bool wide_keys, hipStream_t s);

hipError_t fill_zero(float *p, size_t n, hipStream_t s);

// Stage 3.  in_channels is vd-1 (the homogeneous channel is the bare weight) or vd.
// cell_vertex != nullptr: the replay rows still hold hash cells; they are translated to vertex
// indices and written back.
hipError_t splat(int pd, int vd, const PointMap &map, const float *input, int in_channels,
                 ReplayEntry *replay, const int *cell_vertex, float *values,
                 int xcd_aware, hipStream_t s);

// The transpose of the replay matrix, for lattices that are applied many times (pl_gather.hip):
// the rows that name vertex v are entries[start[v] .. start[v+1]), each the point and its weight.
// Vertices must be numbered densely (number_vertices).  The unit of work of the splat that
// gathers is a chunk of at most ListChunks::rows rows of one list: the chunks of vertex v are
// chunk_start[v] .. chunk_start[v+1], chunk c is described by chunk[c]; a list of several chunks is
// summed into the partial rows of its chunks first (partial_rows[c * vd ..]) and is named in
// long_lists.  info: {long lists, chunks in all}.
// (a chunk of 256 rows for rows of up to four values, where no list of an image like the
// benchmark's is longer; 128 for rows of many channels, whose chunks cost more per row)
constexpr unsigned kListChunkFewChannels = 256, kListChunkManyChannels = 128;
inline unsigned list_chunk_rows(int vd) { return vd <= 4 ? kListChunkFewChannels : kListChunkManyChannels; }
struct ListEntry {
    int point;
    float weight;
};
struct alignas(16) ListChunk {
    unsigned from, to;       // its rows: entries[from .. to)
    unsigned vertex;
    unsigned whole;          // 1: the chunk is all of its vertex's list
};
struct alignas(16) LongList {   // a list of several chunks
    unsigned vertex;
    unsigned chunk_from;     // its first chunk
    unsigned from, to;       // its rows: entries[from .. to)
};
struct ListChunks {
    unsigned *chunk_start;   // [max_vertices + 1]
    ListChunk *chunk;        // [max_chunks]
    LongList *long_lists;    // [max_long]
    float *partial_rows;     // [max_chunks * vd]
    unsigned *info;          // [2], the two words behind VertexLists::count
    unsigned max_chunks, max_long;
    unsigned rows;           // rows of a chunk at most (list_chunk_rows)
};
struct VertexLists {
    unsigned *start;       // [max_vertices + 1]
    ListEntry *entries;    // [capacity]: one per replay row
    unsigned *count;       // [max_vertices + 2] scratch of the build of the lists (and info)
    unsigned *places;      // [capacity] scratch, in the layout of the replay rows
    unsigned *block_sums;  // [2 * (vertex_list_scan_blocks(max_vertices) + 1)] scratch, 8-byte aligned
    size_t capacity;
    ListChunks chunks;
};
size_t vertex_list_scan_blocks(int max_vertices);
size_t vertex_list_max_chunks(int max_vertices, size_t rows);
size_t vertex_list_max_long(size_t rows);
// cell_vertex != nullptr: the replay rows still hold hash cells; they are translated and written
// back.  When the stream has run this, lists.chunks.info holds the numbers splat_gather wants,
// and so do the first two of the three words at host_info (pinned memory the host reads); the
// third is `sequence`, written last by the pass's last launch as that launch starts.
hipError_t build_vertex_lists(int pd, const PointMap &map, ReplayEntry *replay, const int *cell_vertex,
                              int max_vertices, const VertexLists &lists, unsigned *host_info,
                              unsigned sequence, hipStream_t s);
// Stage 3 from the lists: values[v] := sum over v's entries of weight * input row (every vertex's
// row is written whole; no zero fill needed).  n_chunks, n_long: lists.chunks.info as the build of
// the lists left it (a second launch adds up the lists of several chunks when there are any).
hipError_t splat_gather(int vd, const VertexLists &lists, unsigned n_chunks, unsigned n_long,
                        const float *input, int in_channels, float *values, hipStream_t s);

// Stage 4, one axis: dst[v] = 1/4 src[n1] + 1/2 src[v] + 1/4 src[n2] for v < counters->num_vertices.
// reset_cell_keys != nullptr: also empty the hash cell of every vertex (vertex_cell[v]).
hipError_t blur_axis(int vd, const Counters *counters, int max_vertices, const float *src, float *dst,
                     const int2 *neighbours_of_axis, uint64_t *reset_cell_keys,
                     const int *vertex_cell, int launch_vertices, hipStream_t s);

// Two axes in one launch: the result of blur_axis with nbr_first followed by blur_axis with
// nbr_second, bit for bit.
hipError_t blur_two_axes(int vd, const Counters *counters, int max_vertices, const float *src,
                         float *dst, const int2 *nbr_first, const int2 *nbr_second,
                         uint64_t *reset_cell_keys, const int *vertex_cell, int launch_vertices,
                         hipStream_t s);

// Three axes in one launch (vd 2..4 only: blur_can_take_three_axes), bit for bit three blur_axis.
bool blur_can_take_three_axes(int vd);
hipError_t blur_three_axes(int vd, const Counters *counters, int max_vertices, const float *src,
                           float *dst, const int2 *nbr_first, const int2 *nbr_second,
                           const int2 *nbr_third, uint64_t *reset_cell_keys, const int *vertex_cell,
                           int launch_vertices, hipStream_t s);
hipError_t blur_three_axes_f64(int vd, const Counters *counters, int max_vertices, const double *src,
                               double *dst, const int2 *nbr_first, const int2 *nbr_second,
                               const int2 *nbr_third, uint64_t *reset_cell_keys,
                               const int *vertex_cell, int launch_vertices, hipStream_t s);

// Stage 5.  normalize: divide by the homogeneous channel and write vd-1 channels; else write vd.
// cell_vertex != nullptr: the replay rows still hold hash cells (vd <= 8 only).
hipError_t slice(int pd, int vd, const PointMap &map, const ReplayEntry *replay,
                 const int *cell_vertex, const float *values,
                 float *output, int normalize, hipStream_t s);

hipError_t debug_simplex(int pd, const float *positions, int N, const ScaleFactor &scale,
                         short *rem0, short *rank, short *keys, float *barycentric, hipStream_t s);

// How the debug exports count the vertices: densely, segment after segment.  before[k]: vertices
// in the segments below k; total: all of them.
struct VertexNumbers {
    int n_segments;      // 0: the numbers are dense already
    unsigned stride;
    unsigned before[kMaxSegments + 1];
    unsigned total;
    __host__ __device__ unsigned dense_of(unsigned v) const {
        if (n_segments == 0) return v;
        const unsigned k = v / stride;
        return before[k] + (v - k * stride);
    }
    __host__ __device__ unsigned vertex_of(unsigned dense) const {
        if (n_segments == 0) return dense;
        unsigned k = 0;
        while (k + 1 < (unsigned)n_segments && dense >= before[k + 1]) ++k;
        return k * stride + (dense - before[k]);
    }
};
hipError_t export_keys(int pd, const uint64_t *vertex_keys, const VertexNumbers &numbers, short *keys,
                       bool wide_keys, hipStream_t s);
// out[d * words ..] := the row of the d-th vertex (rows of `words` floats)
hipError_t export_values(const float *values, int words, const VertexNumbers &numbers, float *out,
                         hipStream_t s);

// replay arrays in point order: vertex[r*N+n], weight[r*N+n]; cell_vertex != nullptr when
// the replay rows still hold hash cells
hipError_t export_replay(int pd, const PointMap &map, const ReplayEntry *replay,
                         const int *cell_vertex, const VertexNumbers &numbers, int *vertex,
                         float *weight, hipStream_t s);

// The value passes for double values (pl_kernels_f64.hip): as splat, blur_axis, slice,
// debug_simplex and compute_positions above, with `weights` (thread order, like the replay rows)
// carrying the barycentric weights the double build wrote.
hipError_t splat_f64(int pd, int vd, const PointMap &map, const double *input, int in_channels,
                     ReplayEntry *replay, const double *weights, const int *cell_vertex,
                     double *values, int xcd_aware, hipStream_t s);
hipError_t blur_axis_f64(int vd, const Counters *counters, int max_vertices, const double *src,
                         double *dst, const int2 *neighbours_of_axis, uint64_t *reset_cell_keys,
                         const int *vertex_cell, int launch_vertices, hipStream_t s);
// (in pl_kernels.hip: the float kernels over the value type)
hipError_t blur_two_axes_f64(int vd, const Counters *counters, int max_vertices, const double *src,
                             double *dst, const int2 *nbr_first, const int2 *nbr_second,
                             uint64_t *reset_cell_keys, const int *vertex_cell,
                             int launch_vertices, hipStream_t s);
// (vd 2..4: in pl_kernels.hip, rows of doubles gathered whole)
hipError_t slice_rows_f64(int pd, int vd, const PointMap &map, const ReplayEntry *replay,
                          const double *weights, const int *cell_vertex, const double *values,
                          double *output, int normalize, hipStream_t s);
hipError_t slice_f64(int pd, int vd, const PointMap &map, const ReplayEntry *replay,
                     const double *weights, const int *cell_vertex, const double *values,
                     double *output, int normalize, hipStream_t s);
hipError_t debug_simplex_f64(int pd, const double *positions, int N, const ScaleFactor64 &scale,
                             short *rem0, short *rank, short *keys, double *barycentric,
                             hipStream_t s);
hipError_t compute_positions_f64(const double *reference, double *positions, int N,
                                 int n_ref_channels, int n_spatial_dims, const SpatialDims &dims,
                                 double spatial_std, double feature_std, hipStream_t s);

// First index at which feature 0 (period[0]) and feature 1 (period[1]) of consecutive points
// differ, and whether all their changes lie exactly at the multiples of those indices.
// *guess must be {N, N}, 0 before the call.
struct GridGuess {
    int period[2];
    int mismatch;
};
hipError_t guess_grid(const float *positions, int N, int pd, GridGuess *guess, hipStream_t s);

// A plain list of points, put in an order in which neighbours in space are neighbours in the
// list, so that 256 consecutive points share lattice vertices as the pixels of an image tile do
// and the merging build works for them as well.  The points are binned by their first two
// features, and by the third when its extent compares with theirs (the points of a volume):
// square or cubic bins, sized to hold about 60 points if these lay evenly in their bounding box,
// numbered so that 2x2 bins are consecutive, each next to the one before it, and feature 0 grows
// with the number.  When the points lie evenly enough (an image or a regular grid given as a
// list), every bin starts a wavefront of its own: a bin is then a wavefront's 64 points as 8x8
// pixels are, at the price of the places left empty; that is done when it takes at most
// max_tiles workgroups (a quarter more than the points fill).  Otherwise the bins follow each
// other without gaps and a wavefront takes parts of two.  Four launches: the bins (from the
// bounding box of a sample of the points), count (every point draws its rank in its bin), scan of
// the counts, scatter.
// The order inside a bin is whatever the atomics gave; it only orders the work.
// bin_count must be zero before the first call; every call leaves it so.
constexpr size_t kLocalityBinsBytes = 64;
struct LocalityScratch {
    void *bins;            // [kLocalityBinsBytes] the bins of this call, from its first kernel to the others
    float *range0;         // [2] smallest and largest feature 0 (of the sampled points)
    unsigned *bin_count;   // [max_bins], 16-byte aligned
    unsigned *bin_first;   // [max_bins], 16-byte aligned
    uint2 *bin_rank;       // [N] bin of the point, its rank there
    unsigned max_bins;     // a multiple of four
    unsigned *n_tiles;     // out: workgroups of 256 places that hold points
    unsigned max_tiles;    // order has 256 * max_tiles entries
    // for the scan of many bins by many workgroups, each a chunk of 4096 bins:
    unsigned *chunk_sums;  // [2 * locality_scan_chunks(max_bins)]
    unsigned *chunk_first; // [locality_scan_chunks(max_bins) + 1]
};
inline unsigned locality_scan_chunks(unsigned max_bins) { return (max_bins / 4u + 1023u) / 1024u; }
inline unsigned locality_tiles_for(int N) {
    const unsigned waves = ((unsigned)N + 63u) / 64u;
    return (waves + waves / 4u + 3u) / 4u + 1u;
}
inline unsigned locality_bins_for(int N) { return ((unsigned)N / 32u + 1024u) & ~3u; }
// positions or positions64 (the other null); order: 256 * scratch.max_tiles entries
hipError_t order_by_locality(const float *positions, const double *positions64, int N, int pd,
                             const LocalityScratch &scratch, int *order, hipStream_t s);

hipError_t compute_positions(const float *reference, float *positions, int N, int n_ref_channels,
                             int n_spatial_dims, const SpatialDims &dims, float spatial_std,
                             float feature_std, hipStream_t s);

}  // namespace plk
