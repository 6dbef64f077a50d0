// Host side of the C ABI declared in include/permutohedral_lattice.h: the lattice object, its
// scratch memory, the build/apply orchestration and the LatticeFilter op loop.
//
// A filter call enqueues its kernels back to back: the vertex count of the lattice stays on the
// device (every later kernel reads it there and is launched for an estimate of it), so the host
// waits once, for an event behind the build's kernels, to learn whether the hash table was large
// enough, and is back at the caller while the blur and the slice still run.
#include "permutohedral_lattice.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "pl_kernels.h"

namespace {

thread_local int g_last_hip_error = 0;

inline int hip_failed(hipError_t e) {
    if (e == hipSuccess) return 0;
    g_last_hip_error = (int)e;
    return 1;
}
#define PL_HIP(call)                          \
    do {                                      \
        if (hip_failed((call))) return PL_EHIP; \
    } while (0)

void *default_alloc(void *, size_t bytes) {
    void *p = nullptr;
    if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) return nullptr;
    return p;
}
void default_free(void *, void *p) {
    if (p) (void)hipFree(p);
}

uint32_t pow2_at_least(uint64_t x) {
    uint64_t p = 1;
    while (p < x) p <<= 1;
    return (uint32_t)p;
}

// scale factors of the elevation, with the rounding of the reference CPU path
// (src/PermutohedralLatticeCPU.h:209-214: double intermediates, float results)
void compute_scale_factor(int pd, plk::ScaleFactor &sf) {
    const float inv_std_dev = (float)((double)(pd + 1) * std::sqrt(2.0 / 3.0));
    for (int i = 0; i < plk::kMaxPd; ++i) sf.v[i] = 0.0f;
    for (int i = 0; i < pd; ++i)
        sf.v[i] = (float)(1.0 / std::sqrt((double)((i + 1) * (i + 2))) * (double)inv_std_dev);
}

// T = double: all of it in double (src/PermutohedralLatticeCPU.h:209-214 with T = double)
void compute_scale_factor(int pd, plk::ScaleFactor64 &sf) {
    const double inv_std_dev = (double)(pd + 1) * std::sqrt(2.0 / 3.0);
    for (int i = 0; i < plk::kMaxPd; ++i) sf.v[i] = 0.0;
    for (int i = 0; i < pd; ++i) sf.v[i] = 1.0 / std::sqrt((double)((i + 1) * (i + 2))) * inv_std_dev;
}

enum { EV_T0, EV_CLEAR, EV_BUILD, EV_IDS, EV_NBR, EV_A0, EV_FILL, EV_SPLAT, EV_BLUR, EV_SLICE, EV_COUNT };

}  // namespace

struct pl_lattice {
    int pd = 0, vd = 0, N = 0;
    int device = 0;
    hipStream_t stream = nullptr;
    pl_alloc alloc{};
    plk::ScaleFactor scale{};
    // T = double (pl_create_f64): values, weights, inputs and outputs are doubles; the value
    // arrays below are then arrays of double behind their float pointers
    bool f64 = false;
    plk::ScaleFactor64 scale64{};
    double *weights64 = nullptr;       // barycentric weights, layout of the replay rows

    // hash table and the per-vertex arrays; a table of n_cells holds at most 3/4 n_cells vertices
    uint64_t *cell_keys = nullptr;     // [n_cells_alloc]
    int *cell_vertex = nullptr;        // [n_cells_alloc]
    uint64_t *vertex_keys = nullptr;   // [3/4 n_cells_alloc]
    int *vertex_cell = nullptr;        // [3/4 n_cells_alloc]
    float *values[2] = {nullptr, nullptr};  // [3/4 n_cells_alloc * vd]
    int2 *neighbours = nullptr;        // [(pd+1) * 3/4 n_cells_alloc]
    float *cell_values = nullptr;      // [n_cells_alloc * vd] values, rows by hash cell (fused build+splat)
    bool cell_values_clean = false;    // all zero
    uint32_t n_cells_alloc = 0;
    uint32_t n_cells = 0;              // in use by the last build
    uint32_t max_cells = 0;            // enough for N*(pd+1) vertices
    long forced_cells = 0;
    bool table_clean = false;          // every cell of [0, n_cells) is empty
    // Keys of two words (plk::Key128), for coordinates that do not fit the packed key (pd >= 5):
    // a build that meets such a coordinate is repeated with them, and so are the next
    // wide_backoff builds of this lattice (doubled every time it happens again, up to 1024)
    // before the packed key is tried again.  The key arrays are then twice as large.
    bool wide_keys = false;            // the last build (and the arrays) use them
    bool wide_alloc = false;           // cell_keys, vertex_keys and the lists have room for them
    int wide_for = 0, wide_backoff = 32;
    bool may_widen = true;             // (not in the static scratch of pl_filter_static: no room)

    // per-point arrays, (pd+1) rows of map.n_blocks*256 entries in thread order
    plk::PointMap map{};
    plk::ReplayEntry *replay = nullptr;
    // what each workgroup of the build created (see plk::CreatedLists); the chunk counts exist
    // twice and alternate between builds like the counters
    uint4 *created_entries = nullptr;      // [n_blocks * list_stride()]
    int *block_count = nullptr;            // [n_blocks]
    int *chunk_count = nullptr;            // [2][n_chunks]
    size_t n_chunks = 0;
    size_t replay_capacity = 0;
    bool lists_wide = false;               // created_entries has room for two entries per vertex

    // A lattice that is built to be applied (pl_build) also gets, per vertex, the list of the
    // (point, weight) that touch it; pl_apply then splats by gathering (plk::VertexLists)
    bool vertex_lists = true;              // option
    plk::VertexLists lists_of_vertices{};
    size_t lists_for_vertices = 0;         // max_vertices the arrays were allocated for
    bool lists_valid = false;              // they describe the last build
    unsigned list_chunks = 0, long_lists = 0;   // of the last build: chunks in all, lists of several

    plk::Counters *d_counters = nullptr;   // two sets, used by alternate builds
    int counter_set = 0;                   // the set of the last build
    plk::HostStatus *h_status = nullptr;   // pinned, written by the device
    unsigned status_sequence = 0;          // the number of the last build enqueued: what its report carries
    // a lattice in the library's static scratch (pl_filter_static) owns no pinned memory and no
    // event: h_status is device memory there, copied to the host when the build is verified
    bool status_on_device = false;

    int M = 0;
    int last_M = -1;
    // how the last build numbered its vertices (plk::Counters): segments, and the fullest one
    int n_segments = 0, max_segment = 0;
    int last_n_segments = 0, last_max_segment = -1;
    // A build at the largest table whose vertices crowd one eighth of the image overflows that
    // eighth's run of numbers: the call is repeated with the numbers in one run, and so are the
    // next one_segment_backoff builds of this lattice (doubled every time it happens again, up to
    // 1024) before eight runs are tried again.
    int one_segment_for = 0, one_segment_backoff = 32;
    int forced_segments = 0;           // option: 0 = by the size of the build, else 1, 8 or 64
    // A merging build numbers its vertices itself unless that costs more than it saves: when it
    // has many thousands of workgroups (they draw their numbers one after the other), or when
    // the last such build of these points held so many rows of sums for vertices of other
    // workgroups that adding them afterwards, an atomic each, outweighs the numbering pass.
    bool numbering_pass_pays = false;
    long foreign_rows = -1;            // of the last build (an estimate from a sample); -1: it listed none
    bool built = false;                // a build has been enqueued and, if verified, fitted
    bool verified = false;             // its status has been read on the host
    bool replay_holds_cells = false;
    bool values_zeroed = false;        // values[0] rows of all vertices are zero
    bool values_splatted = false;      // values[0] already holds the splat of the pending apply
    bool normalize = true;
    int stop_after = 0;                // PL_OPT_STOP_AFTER: 1 = an apply ends behind the splat, 2 = behind the blur
    int current_values = 0;            // which of values[] the last apply left the vertex values in
    bool profile = false;
    bool xcd_aware = true;
    bool merge_tiles = true;      // option: workgroups merge their keys in LDS when the points are a grid
    // A build that found a tile with too many distinct keys for its LDS table switches merging off
    // for the next tiles_backoff builds of this lattice (doubled every time it happens again, up
    // to 1024): inputs change, and one noisy image must not slow a long-lived lattice for good.
    int tiles_off_for = 0;
    int tiles_backoff = 32;
    bool last_build_merged = false;
    bool pair_blur = true;
    // the grid the points form: given by the caller (pl_set_point_grid), or guessed once from the
    // first positions the handle sees
    bool grid_given = false;
    bool guess_grid = true;
    bool grid_guessed = false;             // a guess has been made (whatever came out)
    plk::GridGuess *d_guess = nullptr;
    // A plain list of points (no grid given or found) is worked on in an order in which
    // neighbours in space are neighbours in the list (plk::order_by_locality), made anew by every
    // build, so that the merging build serves it too
    bool order_points = true;              // option
    int *point_order = nullptr;            // [256 * locality_tiles_for(N)]
    unsigned *locality_words = nullptr;    // the bins, range of feature 0, counts and firsts of the bins
    uint2 *bin_rank = nullptr;             // [N]
    int order_capacity = 0;
    hipEvent_t ev[EV_COUNT] = {};
    bool ev_recorded[EV_COUNT] = {};
    // which of the eight stages pl_stage_ms reports launched a kernel in the last build / apply
    // (an interval between two events with nothing in between still reads a few microseconds)
    bool stage_ran[8] = {};

    // a filter call that has been enqueued but not yet checked on the host (pl_filter_*_begin)
    struct Pending {
        bool active = false;
        bool build_only = false;       // pl_build_*_begin: no apply behind the build
        bool lists = false;            // ... and the per-vertex lists behind it
        plk::PointFeatures features{};
        const double *positions64 = nullptr;
        void *output = nullptr;
        const void *input = nullptr;
        int reverse = 0;
    } pending;

    void *dmalloc(size_t bytes) { return alloc.alloc(alloc.ctx, bytes); }
    template <typename T>
    void dfree(T *&p) {
        if (p) alloc.free(alloc.ctx, (void *)p);
        p = nullptr;
    }
    void mark(int which) {
        if (profile && ev[which]) ev_recorded[which] = hipEventRecord(ev[which], stream) == hipSuccess;
    }
    plk::Counters *counters() { return d_counters + counter_set; }
    // workgroups of the build that hold points (of an ordered list: about; the rest end at once)
    unsigned working_blocks() const {
        return map.mode == 1 ? (unsigned)(((size_t)N + 255) / 256) : map.n_blocks;
    }
    size_t value_size() const { return f64 ? sizeof(double) : sizeof(float); }
    int max_vertices() const { return (int)plk::max_vertices_for(n_cells); }
    // what the grids of the kernels over the vertices are sized for: the count when the host
    // knows it, else the previous build's with a margin (the kernels cover any count)
    // (every XCD walks the segments of its eighth of the image, or its eighth of the numbers:
    // segments as full as the fullest, each with a block that is partly used, cover them all)
    int launch_vertices() const {
        const int mv = max_vertices();
        auto walked = [](long long m, int segments, long long fullest) {
            return (segments > 1 ? segments * fullest : m) + 256ll * (segments > 8 ? segments : 8);
        };
        if (built && verified) {
            const long long m = walked(M, n_segments, max_segment);
            return m < mv ? (int)m : mv;
        }
        if (last_M <= 0) return mv;
        const long long last = walked(last_M, last_n_segments, last_max_segment);
        const long long guess = last + last / 8 + 1024;
        return guess < mv ? (int)guess : mv;
    }
    int list_stride() const { return plk::created_list_stride(pd, f64) * (lists_wide ? 2 : 1); }
    plk::CreatedLists lists(int set) const {
        return plk::CreatedLists{created_entries, block_count, chunk_count + (size_t)set * n_chunks,
                                 list_stride()};
    }
};

namespace {

int ensure_table(pl_lattice *h, uint32_t cells, bool wide) {
    if (cells <= h->n_cells_alloc && (!wide || h->wide_alloc)) return PL_OK;
    if (cells < h->n_cells_alloc) cells = h->n_cells_alloc;
    // the old arrays may still be read by work in flight
    PL_HIP(hipStreamSynchronize(h->stream));
    h->dfree(h->cell_keys);
    h->dfree(h->cell_vertex);
    h->dfree(h->vertex_keys);
    h->dfree(h->vertex_cell);
    h->dfree(h->values[0]);
    h->dfree(h->values[1]);
    h->dfree(h->neighbours);
    h->dfree(h->cell_values);
    h->n_cells_alloc = 0;
    h->table_clean = false;
    h->cell_values_clean = false;
    const size_t mv = plk::max_vertices_for(cells);
    const size_t key_words = wide || h->wide_alloc ? 2 : 1;
    h->cell_keys = (uint64_t *)h->dmalloc(sizeof(uint64_t) * key_words * (size_t)cells);
    h->cell_vertex = (int *)h->dmalloc(sizeof(int) * (size_t)cells);
    h->vertex_keys = (uint64_t *)h->dmalloc(sizeof(uint64_t) * key_words * mv);
    h->vertex_cell = (int *)h->dmalloc(sizeof(int) * mv);
    h->values[0] = (float *)h->dmalloc(h->value_size() * mv * (size_t)h->vd);
    h->values[1] = (float *)h->dmalloc(h->value_size() * mv * (size_t)h->vd);
    h->neighbours = (int2 *)h->dmalloc(sizeof(int2) * mv * (size_t)(h->pd + 1));
    const bool fused_splat = plk::build_can_splat(h->vd);
    if (fused_splat)
        h->cell_values = (float *)h->dmalloc(h->value_size() * (size_t)cells * (size_t)h->vd);
    if (!h->cell_keys || !h->cell_vertex || !h->vertex_keys || !h->vertex_cell || !h->values[0] ||
        !h->values[1] || !h->neighbours || (fused_splat && !h->cell_values))
        return PL_ENOMEM;
    h->n_cells_alloc = cells;
    h->wide_alloc = key_words == 2;
    return PL_OK;
}

int ensure_replay(pl_lattice *h, bool wide) {
    const size_t want = (size_t)h->map.n_blocks * 256 * (size_t)(h->pd + 1);
    if (want <= h->replay_capacity && h->replay && (!wide || h->lists_wide)) return PL_OK;
    h->lists_wide = h->lists_wide || wide;
    PL_HIP(hipStreamSynchronize(h->stream));
    h->dfree(h->replay);
    h->dfree(h->weights64);
    h->dfree(h->created_entries);
    h->dfree(h->block_count);
    h->dfree(h->chunk_count);
    h->replay_capacity = 0;
    h->n_chunks = (h->map.n_blocks + plk::kBlocksPerChunk - 1) / plk::kBlocksPerChunk + 1;
    h->replay = (plk::ReplayEntry *)h->dmalloc(sizeof(plk::ReplayEntry) * (want ? want : 1));
    const size_t entries = (size_t)h->map.n_blocks * (size_t)h->list_stride();
    h->created_entries = (uint4 *)h->dmalloc(sizeof(uint4) * (entries ? entries : 1));
    h->block_count = (int *)h->dmalloc(sizeof(int) * (h->map.n_blocks ? h->map.n_blocks : 1));
    h->chunk_count = (int *)h->dmalloc(sizeof(int) * 2 * h->n_chunks);
    if (h->f64) h->weights64 = (double *)h->dmalloc(sizeof(double) * (want ? want : 1));
    if (!h->replay || !h->created_entries || !h->block_count || !h->chunk_count ||
        (h->f64 && !h->weights64))
        return PL_ENOMEM;
    PL_HIP(plk::fill_zero(reinterpret_cast<float *>(h->chunk_count), 2 * h->n_chunks, h->stream));
    h->replay_capacity = want;
    return PL_OK;
}

int ensure_vertex_lists(pl_lattice *h) {
    const size_t mv = plk::max_vertices_for(h->n_cells_alloc);
    plk::VertexLists &l = h->lists_of_vertices;
    if (l.start && h->lists_for_vertices >= mv && l.capacity >= h->replay_capacity) return PL_OK;
    PL_HIP(hipStreamSynchronize(h->stream));
    h->dfree(l.start);
    h->dfree(l.entries);
    h->dfree(l.count);
    h->dfree(l.places);
    h->dfree(l.block_sums);
    h->dfree(l.chunks.chunk_start);
    h->dfree(l.chunks.chunk);
    h->dfree(l.chunks.long_lists);
    h->dfree(l.chunks.partial_rows);
    h->lists_for_vertices = 0;
    l.capacity = 0;
    const size_t rows = h->replay_capacity ? h->replay_capacity : 1;
    const size_t max_chunks = plk::vertex_list_max_chunks((int)mv, rows);
    const size_t max_long = plk::vertex_list_max_long(rows);
    l.start = (unsigned *)h->dmalloc(sizeof(unsigned) * (mv + 1));
    l.entries = (plk::ListEntry *)h->dmalloc(sizeof(plk::ListEntry) * rows);
    l.count = (unsigned *)h->dmalloc(sizeof(unsigned) * (mv + 2));
    l.places = (unsigned *)h->dmalloc(sizeof(unsigned) * rows);
    l.block_sums = (unsigned *)h->dmalloc(sizeof(unsigned) * 2 * (plk::vertex_list_scan_blocks((int)mv) + 1));
    l.chunks.chunk_start = (unsigned *)h->dmalloc(sizeof(unsigned) * (mv + 1));
    l.chunks.chunk = (plk::ListChunk *)h->dmalloc(sizeof(plk::ListChunk) * max_chunks);
    l.chunks.long_lists = (plk::LongList *)h->dmalloc(sizeof(plk::LongList) * max_long);
    l.chunks.partial_rows = (float *)h->dmalloc(sizeof(float) * max_chunks * (size_t)h->vd);
    if (!l.start || !l.entries || !l.count || !l.places || !l.block_sums || !l.chunks.chunk_start ||
        !l.chunks.chunk || !l.chunks.long_lists || !l.chunks.partial_rows)
        return PL_ENOMEM;
    // (the counts start at zero and every build leaves them so)
    PL_HIP(plk::fill_zero(reinterpret_cast<float *>(l.count), mv + 2, h->stream));
    l.chunks.info = l.count + mv;
    l.chunks.max_chunks = (unsigned)max_chunks;
    l.chunks.max_long = (unsigned)max_long;
    l.chunks.rows = plk::list_chunk_rows(h->vd);
    h->lists_for_vertices = mv;
    l.capacity = h->replay_capacity;
    return PL_OK;
}

// The arrays of the ordering pass for a plain list of N points
plk::LocalityScratch locality_scratch(const pl_lattice *h) {
    const unsigned max_bins = plk::locality_bins_for(h->N);
    plk::LocalityScratch scratch{};
    // (32 words ahead of the arrays: the record of the bins, the range, the number of tiles)
    constexpr size_t head_words = 32;
    static_assert(plk::kLocalityBinsBytes <= 16 * sizeof(unsigned), "the record fits its place");
    scratch.bins = h->locality_words;
    scratch.range0 = reinterpret_cast<float *>(h->locality_words + 16);
    scratch.n_tiles = h->locality_words + 20;
    scratch.bin_count = h->locality_words + head_words;
    scratch.bin_first = h->locality_words + head_words + max_bins;
    scratch.bin_rank = h->bin_rank;
    scratch.max_bins = max_bins;
    scratch.max_tiles = plk::locality_tiles_for(h->N);
    scratch.chunk_sums = h->locality_words + head_words + 2 * (size_t)max_bins;
    scratch.chunk_first = scratch.chunk_sums + 2 * (size_t)plk::locality_scan_chunks(max_bins);
    return scratch;
}

int ensure_order(pl_lattice *h) {
    if (h->point_order && h->order_capacity >= h->N) return PL_OK;
    PL_HIP(hipStreamSynchronize(h->stream));
    h->dfree(h->point_order);
    h->dfree(h->locality_words);
    h->dfree(h->bin_rank);
    h->dfree(h->lists_of_vertices.start);
    h->dfree(h->lists_of_vertices.entries);
    h->dfree(h->lists_of_vertices.count);
    h->dfree(h->lists_of_vertices.places);
    h->dfree(h->lists_of_vertices.block_sums);
    h->dfree(h->lists_of_vertices.chunks.chunk_start);
    h->dfree(h->lists_of_vertices.chunks.chunk);
    h->dfree(h->lists_of_vertices.chunks.long_lists);
    h->dfree(h->lists_of_vertices.chunks.partial_rows);
    h->order_capacity = 0;
    const unsigned max_bins = plk::locality_bins_for(h->N);
    const size_t words = 32 + 2 * (size_t)max_bins + 3 * (size_t)plk::locality_scan_chunks(max_bins) + 1;
    h->point_order = (int *)h->dmalloc(sizeof(int) * 256 * (size_t)plk::locality_tiles_for(h->N));
    h->locality_words = (unsigned *)h->dmalloc(sizeof(unsigned) * words);
    h->bin_rank = (uint2 *)h->dmalloc(sizeof(uint2) * (size_t)h->N);
    if (!h->point_order || !h->locality_words || !h->bin_rank) return PL_ENOMEM;
    // (the pass leaves its counts zero for the next call)
    PL_HIP(plk::fill_zero(reinterpret_cast<float *>(h->locality_words), words, h->stream));
    h->order_capacity = h->N;
    return PL_OK;
}

uint32_t initial_cells(const pl_lattice *h) {
    uint64_t want;
    if (h->forced_cells > 0) {
        want = (uint64_t)h->forced_cells;
    } else if (h->last_M > 0) {
        // Load factor 0.1..0.2 if the next input resembles the last.  A wavefront of the build
        // waits for the longest probe sequence among its ~40 keys, two dependent memory round
        // trips per step (1024x1024 image: 3.6 steps at load 0.34, 2.4 at 0.17), and no kernel
        // walks the cells, so a sparser table costs memory only.
        want = (uint64_t)h->last_M * 5;
    } else {
        want = (uint64_t)h->N * (uint64_t)(h->pd + 1) / 8;
    }
    if (want < 4096) want = 4096;
    uint32_t cells = pow2_at_least(want);
    if (cells > h->max_cells) cells = h->max_cells;
    return cells;
}

// Enqueue one build with a table of `cells` cells.  Nothing here waits for the device.
// splat_input != nullptr: the build kernel also splats these values (when it can for this vd),
// and the value table holds them when the build is done.
// A lattice for double values takes its positions from positions64 and never splats in the build.
int enqueue_build(pl_lattice *h, const plk::PointFeatures &features, const double *positions64,
                  uint32_t cells, const void *splat_input) {
    // keys of two words while a build that needed them is recent (the plain build only)
    const bool wide = h->wide_for > 0;
    if (h->wide_for > 0) h->wide_for -= 1;
    if (wide != h->wide_keys) h->table_clean = false;   // (cells of another width)
    h->wide_keys = wide;
    int rc = ensure_table(h, cells, wide);
    if (rc != PL_OK) return rc;
    // tiles of an image share most of their vertices among their four wavefronts
    const bool merge_allowed = h->merge_tiles && h->tiles_off_for == 0 && !wide;
    if (h->tiles_off_for > 0 && !wide) h->tiles_off_for -= 1;
    // a plain list is put in an order that gives its workgroups such tiles
    if (h->map.mode <= 1) {
        const bool ordered = merge_allowed && h->order_points && h->N >= 4096 &&
                             (positions64 || features.positions);
        if (ordered) {
            rc = ensure_order(h);
            if (rc != PL_OK) return rc;
        }
        h->map.mode = ordered ? 1 : 0;
        h->map.order = ordered ? h->point_order : nullptr;
        h->map.n_tiles = ordered ? locality_scratch(h).n_tiles : nullptr;
        // (an ordered list may leave places empty: room for a quarter more than the points fill)
        h->map.n_blocks = ordered ? plk::locality_tiles_for(h->N)
                                  : (unsigned)(((size_t)h->N + 255) / 256);
    }
    const bool merge = merge_allowed && h->map.mode != 0;
    h->last_build_merged = merge;
    // the per-point arrays follow the point map; an allocation that failed when the map was set
    // is made up for here
    rc = ensure_replay(h, wide);
    if (rc != PL_OK) return rc;
    // (a lattice of doubles splats in its build only in the merging kernel)
    const bool fused = splat_input && plk::build_can_splat(h->vd) && (!h->f64 || merge);
    // (a build for one filter: a lattice built to be applied many times is numbered by the
    // numbering pass, in the order of the image tiles, which the passes over the vertices walk
    // a few per cent faster than the order in which the workgroups happened to finish)
    const bool numbers_in_build = merge && fused && !h->numbering_pass_pays && h->forced_segments >= 0;
    const size_t floats_per_value = h->f64 ? 2 : 1;
    if (fused && !numbers_in_build && !h->cell_values_clean) {
        PL_HIP(plk::fill_zero(h->cell_values, (size_t)h->n_cells_alloc * h->vd * floats_per_value,
                              h->stream));
        h->cell_values_clean = true;
    }
    // (what this build's report will carry; never 0, which is what a fresh status holds)
    h->status_sequence = h->status_sequence + 1u ? h->status_sequence + 1u : 1u;
    const plk::HostReport report_to{h->h_status, h->status_sequence};
    h->mark(EV_T0);
    h->stage_ran[0] = h->map.mode == 1 || !h->table_clean || cells != h->n_cells;
    h->stage_ran[1] = true;
    h->stage_ran[2] = !numbers_in_build;
    h->stage_ran[3] = true;
    if (h->map.mode == 1)
        PL_HIP(plk::order_by_locality(h->f64 ? nullptr : features.positions,
                                      h->f64 ? positions64 : nullptr, h->N, h->pd,
                                      locality_scratch(h), h->point_order, h->stream));
    if (!h->table_clean || cells != h->n_cells) {
        PL_HIP(plk::clear_table(h->cell_keys, wide ? 2 * cells : cells, h->stream));
    }
    h->table_clean = false;
    h->n_cells = cells;
    h->mark(EV_CLEAR);
    // the previous vertex-numbering kernel (or pl_create) left the other counter set zeroed
    const int previous_set = h->counter_set;
    h->counter_set = 1 - previous_set;
    const plk::VertexTables vertices{h->cell_vertex, h->vertex_keys, h->vertex_cell, h->neighbours,
                                     h->max_vertices()};
    const plk::CreatedLists lists = h->lists(h->counter_set);
    // the merging build numbers its vertices itself and reports to the host
    const plk::InBuildNumbering numbering{
        h->cell_vertex, h->vertex_keys, h->vertex_cell, h->neighbours, h->max_vertices(),
        h->values[0], h->f64 ? 2 * h->vd : h->vd,
        !numbers_in_build ? 0 : (h->one_segment_for > 0 ? 1 : plk::segments_for((uint32_t)h->max_vertices(),
                                                                              h->forced_segments == 64 ? 1u << 20 : h->forced_segments == 8 ? 1u : h->working_blocks()))};
    if (numbers_in_build && h->one_segment_for > 0) h->one_segment_for -= 1;
    // keys go to the part of the table that belongs to their band of rows when the points are
    // known to be a grid (and feature 0 then runs with its slowest extent)
    plk::RegionSource regions{};
    regions.enabled = h->xcd_aware && h->map.mode != 0;
    regions.N = h->N;
    regions.pd = h->pd;
    regions.scale0 = h->f64 ? (float)h->scale64.v[0] : h->scale.v[0];
    regions.positions = h->f64 ? nullptr : features.positions;
    regions.positions64 = h->f64 ? positions64 : nullptr;
    // (in the order of a list feature 0 grows with the workgroups as it does down an image)
    regions.range0 = h->map.mode == 1 ? locality_scratch(h).range0 : nullptr;
    if (!h->f64 && !features.positions) {
        if (features.n_spatial_dims > 0) {
            regions.first = 0.0f;
            regions.last = (float)(features.dims.v[0] - 1) / features.spatial_std;
        } else {
            regions.enabled = 0;
        }
    }
    if (h->f64) {
        const plk::Points64 points{positions64, h->weights64, h->scale64};
        PL_HIP(plk::build_f64(h->pd, points, h->map, h->cell_keys, cells, h->counters(), h->replay,
                              h->xcd_aware ? 1 : 0, lists, regions, merge ? &numbering : nullptr,
                              fused ? h->vd : 0,
                              static_cast<const double *>(splat_input),
                              h->normalize ? h->vd - 1 : h->vd,
                              reinterpret_cast<double *>(h->cell_values), wide, h->stream));
    } else {
        PL_HIP(plk::build(h->pd, features, h->map, h->scale, h->cell_keys, cells, h->counters(),
                          h->replay, h->xcd_aware ? 1 : 0, fused ? h->vd : 0,
                          static_cast<const float *>(splat_input),
                          h->normalize ? h->vd - 1 : h->vd, h->cell_values, lists,
                          regions, merge ? &numbering : nullptr, wide, h->stream));
    }
    h->mark(EV_BUILD);
    if (!numbers_in_build) {
        // the numbering pass zeroes the vertices' value rows: a row of vd doubles is 2*vd zero floats
        PL_HIP(plk::number_vertices(h->pd, h->map, lists,
                                    h->chunk_count + (size_t)previous_set * h->n_chunks,
                                    (unsigned)h->n_chunks, vertices,
                                    h->values[0], h->f64 ? 2 * h->vd : h->vd,
                                    fused ? h->cell_values : nullptr, h->counters(),
                                    h->d_counters + previous_set, report_to, wide, h->stream));
    }
    h->mark(EV_IDS);
    // (the rows a build that numbered its vertices listed for vertices of other workgroups join
    // the value table here, and its counts reach the host from here)
    PL_HIP(plk::neighbours(h->pd, vertices, h->counters(), h->cell_keys, cells,
                           h->launch_vertices(), numbers_in_build && fused ? &lists : nullptr,
                           h->map.n_blocks, h->values[0], h->vd, h->f64,
                           numbers_in_build ? h->counters() : nullptr,
                           h->d_counters + previous_set, report_to, wide, h->stream));
    h->mark(EV_NBR);
    h->replay_holds_cells = true;
    h->values_zeroed = !fused;
    h->values_splatted = fused;
    h->built = true;
    h->verified = false;
    h->lists_valid = false;
    return PL_OK;
}

// The value passes for a lattice of doubles: plain splat, one blur launch per axis, slice.
int enqueue_apply_f64(pl_lattice *h, double *output, const double *input, int reverse) {
    const int pd = h->pd, vd = h->vd;
    const int in_channels = h->normalize ? vd - 1 : vd;
    const int mv = h->max_vertices();
    double *values[2] = {reinterpret_cast<double *>(h->values[0]),
                         reinterpret_cast<double *>(h->values[1])};
    h->mark(EV_A0);
    h->stage_ran[4] = !h->values_splatted && !h->values_zeroed;
    h->stage_ran[5] = !h->values_splatted;
    h->stage_ran[6] = h->stop_after != 1;
    h->stage_ran[7] = h->stop_after == 0;
    if (!h->values_splatted) {
        if (!h->values_zeroed)
            PL_HIP(plk::fill_zero(h->values[0], (size_t)mv * vd * 2, h->stream));
        h->mark(EV_FILL);
        PL_HIP(plk::splat_f64(pd, vd, h->map, input, in_channels, h->replay, h->weights64,
                              h->replay_holds_cells ? h->cell_vertex : nullptr, values[0],
                              h->xcd_aware ? 1 : 0, h->stream));
        h->replay_holds_cells = false;
    } else {
        h->mark(EV_FILL);
    }
    h->values_zeroed = false;
    h->values_splatted = false;
    h->mark(EV_SPLAT);
    int cur = 0;
    h->current_values = 0;
    if (h->stop_after == 1) return PL_OK;
    for (int step = 0; step <= pd;) {
        const int axis = reverse ? pd - step : step;
        uint64_t *reset = (!h->table_clean && step == 0 && !h->wide_keys) ? h->cell_keys : nullptr;
        const int left = pd + 1 - step;
        // (three axes in one launch pay only when they are all there is: pd = 2; otherwise 27 row
        // gathers per vertex cost more than the launch they save)
        if (h->pair_blur && plk::blur_can_take_three_axes(vd) && left == 3 && step == 0) {
            const int d = reverse ? -1 : 1;
            PL_HIP(plk::blur_three_axes_f64(vd, h->counters(), mv, values[cur], values[1 - cur],
                                            h->neighbours + (size_t)axis * mv,
                                            h->neighbours + (size_t)(axis + d) * mv,
                                            h->neighbours + (size_t)(axis + 2 * d) * mv, reset,
                                            h->vertex_cell, h->launch_vertices(), h->stream));
            step += 3;
        } else if (h->pair_blur && step + 1 <= pd) {
            const int next_axis = reverse ? axis - 1 : axis + 1;
            PL_HIP(plk::blur_two_axes_f64(vd, h->counters(), mv, values[cur], values[1 - cur],
                                          h->neighbours + (size_t)axis * mv,
                                          h->neighbours + (size_t)next_axis * mv, reset,
                                          h->vertex_cell, h->launch_vertices(), h->stream));
            step += 2;
        } else {
            PL_HIP(plk::blur_axis_f64(vd, h->counters(), mv, values[cur], values[1 - cur],
                                      h->neighbours + (size_t)axis * mv, reset, h->vertex_cell,
                                      h->launch_vertices(), h->stream));
            step += 1;
        }
        if (reset) h->table_clean = true;
        cur = 1 - cur;
    }
    h->mark(EV_BLUR);
    h->current_values = cur;
    if (h->stop_after == 2) return PL_OK;
    PL_HIP(plk::slice_f64(pd, vd, h->map, h->replay, h->weights64,
                          h->replay_holds_cells ? h->cell_vertex : nullptr, values[cur], output,
                          h->normalize ? 1 : 0, h->stream));
    h->mark(EV_SLICE);
    return PL_OK;
}

// output and input are arrays of the lattice's value type
int enqueue_apply(pl_lattice *h, void *output_any, const void *input_any, int reverse) {
    if (h->f64)
        return enqueue_apply_f64(h, static_cast<double *>(output_any),
                                 static_cast<const double *>(input_any), reverse);
    float *output = static_cast<float *>(output_any);
    const float *input = static_cast<const float *>(input_any);
    const int pd = h->pd, vd = h->vd;
    const int in_channels = h->normalize ? vd - 1 : vd;
    const int mv = h->max_vertices();
    h->mark(EV_A0);
    const bool gather = !h->values_splatted && h->lists_valid;
    h->stage_ran[4] = !h->values_splatted && !h->values_zeroed && !gather;
    h->stage_ran[5] = !h->values_splatted;
    h->stage_ran[6] = h->stop_after != 1;
    h->stage_ran[7] = h->stop_after == 0;
    if (gather) {
        // (every vertex's row is written whole: nothing to clear)
        h->mark(EV_FILL);
        PL_HIP(plk::splat_gather(vd, h->lists_of_vertices, h->list_chunks, h->long_lists, input,
                                 in_channels, h->values[0], h->stream));
    } else if (!h->values_splatted) {
        if (!h->values_zeroed) PL_HIP(plk::fill_zero(h->values[0], (size_t)mv * vd, h->stream));
        h->mark(EV_FILL);
        PL_HIP(plk::splat(pd, vd, h->map, input, in_channels, h->replay,
                          h->replay_holds_cells ? h->cell_vertex : nullptr, h->values[0],
                          h->xcd_aware ? 1 : 0, h->stream));
        h->replay_holds_cells = false;
    } else {
        h->mark(EV_FILL);
    }
    h->values_zeroed = false;
    h->values_splatted = false;
    h->mark(EV_SPLAT);
    int cur = 0;
    h->current_values = 0;
    if (h->stop_after == 1) return PL_OK;
    for (int step = 0; step <= pd;) {
        // axes 0..pd, or pd..0 for the reverse pass; two per launch while two are left
        const int axis = reverse ? pd - step : step;
        // the first blur after a build also empties the vertices' hash cells
        uint64_t *reset = (!h->table_clean && step == 0 && !h->wide_keys) ? h->cell_keys : nullptr;
        const int left = pd + 1 - step;
        // (three axes in one launch pay only when they are all there is: pd = 2; otherwise 27 row
        // gathers per vertex cost more than the launch they save)
        if (h->pair_blur && plk::blur_can_take_three_axes(vd) && left == 3 && step == 0) {
            const int d = reverse ? -1 : 1;
            PL_HIP(plk::blur_three_axes(vd, h->counters(), mv, h->values[cur], h->values[1 - cur],
                                        h->neighbours + (size_t)axis * mv,
                                        h->neighbours + (size_t)(axis + d) * mv,
                                        h->neighbours + (size_t)(axis + 2 * d) * mv, reset,
                                        h->vertex_cell, h->launch_vertices(), h->stream));
            step += 3;
        } else if (h->pair_blur && step + 1 <= pd) {
            const int next_axis = reverse ? axis - 1 : axis + 1;
            PL_HIP(plk::blur_two_axes(vd, h->counters(), mv, h->values[cur], h->values[1 - cur],
                                      h->neighbours + (size_t)axis * mv,
                                      h->neighbours + (size_t)next_axis * mv, reset, h->vertex_cell,
                                      h->launch_vertices(), h->stream));
            step += 2;
        } else {
            PL_HIP(plk::blur_axis(vd, h->counters(), mv, h->values[cur], h->values[1 - cur],
                                  h->neighbours + (size_t)axis * mv, reset, h->vertex_cell,
                                  h->launch_vertices(), h->stream));
            step += 1;
        }
        if (reset) h->table_clean = true;
        cur = 1 - cur;
    }
    h->mark(EV_BLUR);
    h->current_values = cur;
    if (h->stop_after == 2) return PL_OK;
    PL_HIP(plk::slice(pd, vd, h->map, h->replay,
                      h->replay_holds_cells ? h->cell_vertex : nullptr, h->values[cur], output,
                      h->normalize ? 1 : 0, h->stream));
    h->mark(EV_SLICE);
    return PL_OK;
}

// Wait until the last build has reported (not for what was enqueued behind it: the host learns
// whether the table was large enough while the blur and the slice still run, and the caller's next
// call is enqueued behind them without a gap).  PL_OK: it fitted, h->M is valid.
// Otherwise *retry_cells is the table size to try next (0: give up with the returned status).
// The kernels that report to the host write the number of the build they belong to last, behind a
// system-wide fence, into pinned memory, and the host polls that word.  (An event recorded between
// the reporting kernel and the next kept the next from starting for 6 us, and the host learned
// of the report only when the reporting kernel had ended; now it knows when that kernel starts.)
// Should the word never come -- a launch that failed -- the wait for the stream says why.
int wait_for_report(pl_lattice *h, const volatile unsigned *word) {
    const auto started = std::chrono::steady_clock::now();
    for (unsigned spins = 1; *word != h->status_sequence; ++spins) {
        if ((spins & 0xfffu) == 0 &&
            std::chrono::steady_clock::now() - started > std::chrono::seconds(2)) {
            PL_HIP(hipStreamSynchronize(h->stream));
            if (*word != h->status_sequence) return PL_EHIP;
            break;
        }
    }
    std::atomic_thread_fence(std::memory_order_acquire);
    return PL_OK;
}

int verify_build(pl_lattice *h, uint32_t *retry_cells) {
    *retry_cells = 0;
    plk::HostStatus status;
    if (h->status_on_device) {
        PL_HIP(hipMemcpyAsync(&status, h->h_status, sizeof(status), hipMemcpyDeviceToHost, h->stream));
        PL_HIP(hipStreamSynchronize(h->stream));
    } else {
        const int rc = wait_for_report(h, &h->h_status->sequence);
        if (rc != PL_OK) return rc;
        status = *h->h_status;
    }
    const int flags = status.flags;
    const int m = status.num_vertices;
    h->last_n_segments = status.n_segments;
    h->last_max_segment = status.max_segment;
    if (flags & plk::kFlagKeyRange) {
        // (the build may also have overflowed the table, and then rows of sums of the vertices
        // beyond its capacity are still where the fused splat put them)
        h->built = false;
        h->table_clean = false;
        h->cell_values_clean = false;
        // A coordinate that does not fit the packed key: once more with keys of two words, which
        // hold every short (and so do the next builds of this lattice, for a while).  With those
        // the coordinate is beyond the reference's own keys.
        if (!h->wide_keys && h->may_widen && plk::key_field_bits(h->pd) < 16) {
            h->wide_for = h->wide_backoff;
            h->wide_backoff = h->wide_backoff >= 512 ? 1024 : h->wide_backoff * 2;
            *retry_cells = h->n_cells;
        }
        return PL_EOVERFLOW;
    }
    if (flags & plk::kFlagTileFull) {
        // a tile with more distinct keys than the merging build's LDS table holds: this call is
        // repeated, and the next builds of this lattice run, without merging
        h->built = false;
        h->table_clean = false;
        h->cell_values_clean = false;
        h->tiles_off_for = h->tiles_backoff;
        h->tiles_backoff = h->tiles_backoff >= 512 ? 1024 : h->tiles_backoff * 2;
        *retry_cells = h->n_cells;
        return PL_EOVERFLOW;
    }
    if ((flags & plk::kFlagTableFull) || (uint32_t)m > plk::max_vertices_for(h->n_cells)) {
        h->built = false;
        h->table_clean = false;  // keys beyond the numbered vertices may remain
        h->cell_values_clean = false;
        if (h->n_cells >= h->max_cells) {
            // the largest table holds every vertex, but a segment of it may not hold all that
            // one part of the image creates: once more with the numbers in one run
            if (status.n_segments <= 1 || (uint32_t)m > plk::max_vertices_for(h->n_cells))
                return PL_EOVERFLOW;   // (cannot happen)
            h->one_segment_for = h->one_segment_backoff;
            h->one_segment_backoff = h->one_segment_backoff >= 512 ? 1024 : h->one_segment_backoff * 2;
            *retry_cells = h->n_cells;
            return PL_EOVERFLOW;
        }
        *retry_cells = (h->n_cells > h->max_cells / 4) ? h->max_cells : h->n_cells * 4;
        return PL_EOVERFLOW;
    }
    h->M = m;
    h->last_M = m;
    h->n_segments = status.n_segments;
    h->max_segment = status.max_segment;
    // (in ns, as measured on 1024x1024 and 512x512 images and a 128x256x256 volume: a row added
    // afterwards takes 0.037 of the atomic unit's time (1.85 M rows of the volume: 69 us); the
    // numbering pass 1.25 per workgroup of the build and 0.02 per vertex (the volume's 32 768
    // workgroups: 41 us), and the build 1500 longer with all its rows going out as atomics)
    h->foreign_rows = status.n_segments != 0 ? (long)status.foreign_rows : -1;
    if (status.n_segments != 0 &&
        0.037 * status.foreign_rows > 1.25 * h->working_blocks() + 0.02 * m + 1500.0)
        h->numbering_pass_pays = true;
    h->verified = true;
    if (h->last_build_merged) h->tiles_backoff = 32;
    return PL_OK;
}

}  // namespace

extern "C" {

int pl_supported(int pd, int vd) { return pd >= 1 && pd <= plk::kMaxPd && vd >= 2 ? 1 : 0; }

const char *pl_strerror(int status) {
    switch (status) {
        case PL_OK: return "ok";
        case PL_EINVAL: return "invalid argument";
        case PL_EUNSUPPORTED: return "unsupported (pd, vd)";
        case PL_ENOMEM: return "out of device memory";
        case PL_EOVERFLOW: return "size or lattice coordinate out of range";
        case PL_EHIP: return "HIP runtime error";
        case PL_ESTATE: return "call out of order";
        case PL_ETOOLARGE:
            return "too large for the static scratch of pl_filter_static (N*(pd+1) <= 131072, vd <= 8)";
        default: return "unknown status";
    }
}

int pl_last_hip_error(void) { return g_last_hip_error; }

#ifndef PL_SOURCE_HASH
#define PL_SOURCE_HASH 0
#endif
int pl_library_info(int what, long long *value) {
    if (!value) return PL_EINVAL;
    switch (what) {
        case PL_LIB_LAYOUT_VERSION: *value = PL_LAYOUT_VERSION; return PL_OK;
        case PL_LIB_REPLAY_ROW_BYTES: *value = (long long)sizeof(plk::ReplayEntry); return PL_OK;
        case PL_LIB_SOURCE_HASH: *value = (long long)(PL_SOURCE_HASH); return PL_OK;
        default: return PL_EINVAL;
    }
}

static int create_lattice(int pd, int vd, int N, bool f64, pl_stream stream, const pl_alloc *alloc,
                          pl_handle *out) {
    if (!out) return PL_EINVAL;
    *out = nullptr;
    if (N < 0 || pd < 1 || vd < 2) return PL_EINVAL;
    if (!pl_supported(pd, vd)) return PL_EUNSUPPORTED;
    if (alloc && (!alloc->alloc || !alloc->free)) return PL_EINVAL;
    // N*(pd+1) replay rows and N*vd values must be addressable with the table sizes used here
    const uint64_t rows = (uint64_t)N * (uint64_t)(pd + 1);
    if (rows > (1ull << 30) || (uint64_t)N * (uint64_t)vd > (1ull << 31) - 1) return PL_EOVERFLOW;

    pl_lattice *h = new (std::nothrow) pl_lattice();
    if (!h) return PL_ENOMEM;
    h->pd = pd;
    h->vd = vd;
    h->N = N;
    h->f64 = f64;
    h->stream = (hipStream_t)stream;
    if (alloc) {
        h->alloc = *alloc;
    } else {
        h->alloc.alloc = default_alloc;
        h->alloc.free = default_free;
        h->alloc.ctx = nullptr;
    }
    compute_scale_factor(pd, h->scale);
    compute_scale_factor(pd, h->scale64);
    // holds N*(pd+1) vertices, up to the size the kernels address cells in (32-bit byte offsets
    // of 8-byte cells, cell_at in pl_kernels.hip); a lattice with more vertices than 3/4 of that
    // is refused with PL_EOVERFLOW when a build finds them
    h->max_cells = pow2_at_least(rows * 2 < 4096 ? 4096 : rows * 2);
    if (h->max_cells > plk::kMaxCells) h->max_cells = plk::kMaxCells;
    h->map = plk::make_point_map(N, 0, nullptr);

    int rc = PL_OK;
    if (hip_failed(hipGetDevice(&h->device))) rc = PL_EHIP;
    if (rc == PL_OK) rc = ensure_replay(h, false);
    if (rc == PL_OK) {
        h->d_counters = (plk::Counters *)h->dmalloc(2 * sizeof(plk::Counters));
        if (!h->d_counters) rc = PL_ENOMEM;
    }
    if (rc == PL_OK && hip_failed(plk::fill_zero(reinterpret_cast<float *>(h->d_counters),
                                                 2 * sizeof(plk::Counters) / sizeof(float), h->stream)))
        rc = PL_EHIP;
    if (rc == PL_OK &&
        hip_failed(hipHostMalloc((void **)&h->h_status, sizeof(plk::HostStatus) + 3 * sizeof(unsigned),
                                 hipHostMallocCoherent)))
        rc = PL_EHIP;
    if (rc != PL_OK) {
        pl_destroy(h);
        return rc;
    }
    h->h_status->num_vertices = 0;
    h->h_status->flags = 0;
    h->h_status->sequence = 0;
    reinterpret_cast<unsigned *>(h->h_status + 1)[2] = 0;   // (the lists' report, behind the status)
    *out = h;
    return PL_OK;
}

int pl_create(int pd, int vd, int N, pl_stream stream, const pl_alloc *alloc, pl_handle *out) {
    return create_lattice(pd, vd, N, false, stream, alloc, out);
}

int pl_create_f64(int pd, int vd, int N, pl_stream stream, const pl_alloc *alloc, pl_handle *out) {
    return create_lattice(pd, vd, N, true, stream, alloc, out);
}

int pl_destroy(pl_handle h) {
    if (!h) return PL_OK;
    (void)hipStreamSynchronize(h->stream);
    h->dfree(h->cell_keys);
    h->dfree(h->cell_vertex);
    h->dfree(h->vertex_keys);
    h->dfree(h->vertex_cell);
    h->dfree(h->values[0]);
    h->dfree(h->values[1]);
    h->dfree(h->neighbours);
    h->dfree(h->cell_values);
    h->dfree(h->replay);
    h->dfree(h->weights64);
    h->dfree(h->created_entries);
    h->dfree(h->block_count);
    h->dfree(h->chunk_count);
    h->dfree(h->d_counters);
    h->dfree(h->d_guess);
    h->dfree(h->point_order);
    h->dfree(h->locality_words);
    h->dfree(h->bin_rank);
    if (h->h_status) (void)hipHostFree(h->h_status);
    for (int i = 0; i < EV_COUNT; ++i)
        if (h->ev[i]) (void)hipEventDestroy(h->ev[i]);
    delete h;
    return PL_OK;
}

int pl_set_option(pl_handle h, int option, long value) {
    if (!h) return PL_EINVAL;
    switch (option) {
        case PL_OPT_NORMALIZE:
            h->normalize = value != 0;
            return PL_OK;
        case PL_OPT_PROFILE:
            h->profile = value != 0;
            if (h->profile)
                for (int i = 0; i < EV_COUNT; ++i)
                    if (!h->ev[i]) PL_HIP(hipEventCreate(&h->ev[i]));
            return PL_OK;
        case PL_OPT_XCD_AWARE:
            h->xcd_aware = value != 0;
            return PL_OK;
        case PL_OPT_PAIR_BLUR:
            h->pair_blur = value != 0;
            return PL_OK;
        case PL_OPT_GUESS_GRID:
            h->guess_grid = value != 0;
            return PL_OK;
        case PL_OPT_MERGE_TILES:
            h->merge_tiles = value != 0;
            return PL_OK;
        case PL_OPT_ORDER_POINTS:
            h->order_points = value != 0;
            return PL_OK;
        case PL_OPT_NUMBER_SEGMENTS:
            if (value != 0 && value != 8 && value != 64 && value != -1) return PL_EINVAL;
            h->forced_segments = (int)value;
            return PL_OK;
        case PL_OPT_VERTEX_LISTS:
            h->vertex_lists = value != 0;
            if (!h->vertex_lists) h->lists_valid = false;
            return PL_OK;
        case PL_OPT_STOP_AFTER:
            if (value < 0 || value > 2) return PL_EINVAL;
            h->stop_after = (int)value;
            return PL_OK;
        case PL_OPT_TABLE_CELLS:
            if (value < 0 || (value & (value - 1)) != 0) return PL_EINVAL;
            h->forced_cells = value;
            h->last_M = -1;
            return PL_OK;
        default:
            return PL_EINVAL;
    }
}

int pl_set_point_grid(pl_handle h, int n_dims, const int *dims) {
    if (!h || n_dims < 0 || (n_dims > 0 && !dims)) return PL_EINVAL;
    if (h->pending.active) return PL_ESTATE;
    if (n_dims > 0) {
        long long prod = 1;
        for (int i = 0; i < n_dims; ++i) {
            if (dims[i] < 1) return PL_EINVAL;
            prod *= dims[i];
            if (prod > 2147483647LL) return PL_EINVAL;
        }
        if (prod != (long long)h->N) return PL_EINVAL;
    }
    h->built = false;
    h->grid_given = n_dims > 0;
    h->map = plk::make_point_map(h->N, n_dims, dims);
    h->numbering_pass_pays = false;
    h->one_segment_for = 0;
    h->one_segment_backoff = 32;
    return ensure_replay(h, false);
}

int pl_get_point_grid(pl_handle h, int *n_dims, int dims[3]) {
    if (!h || !n_dims || !dims) return PL_EINVAL;
    *n_dims = h->map.mode <= 1 ? 0 : h->map.mode;
    for (int i = 0; i < 3; ++i) dims[i] = 0;
    if (h->map.mode == 2) {
        dims[0] = h->map.dims[1];
        dims[1] = h->map.dims[2];
    } else if (h->map.mode == 3) {
        for (int i = 0; i < 3; ++i) dims[i] = h->map.dims[i];
    }
    return PL_OK;
}

namespace {

plk::PointFeatures features_from_positions(const float *positions) {
    plk::PointFeatures f{};
    f.positions = positions;
    return f;
}

// A caller of filter(output, input, positions, reverse) has no way to say that its points are the
// pixels of an image, but positions made by the reference's feature builder show it: the first
// time a handle without a grid hint sees positions, two small kernels look for the row length
// (and the slice size of a volume) and, if the points turn out to be a row-major grid, the
// workgroups take tiles of it as with pl_set_point_grid.  One stream synchronisation, once per
// handle; what is found only orders the work.
int guess_point_grid(pl_lattice *h, const float *positions) {
    if (h->grid_given || !h->guess_grid || h->grid_guessed || h->N < 4096) return PL_OK;
    h->grid_guessed = true;
    if (!h->d_guess) {
        h->d_guess = (plk::GridGuess *)h->dmalloc(sizeof(plk::GridGuess));
        if (!h->d_guess) return PL_ENOMEM;
    }
    plk::GridGuess guess{{h->N, h->N}, 0};
    PL_HIP(hipMemcpyAsync(h->d_guess, &guess, sizeof(guess), hipMemcpyHostToDevice, h->stream));
    PL_HIP(plk::guess_grid(positions, h->N, h->pd, h->d_guess, h->stream));
    PL_HIP(hipMemcpyAsync(&guess, h->d_guess, sizeof(guess), hipMemcpyDeviceToHost, h->stream));
    PL_HIP(hipStreamSynchronize(h->stream));
    const int p0 = guess.period[0], p1 = h->pd >= 2 ? guess.period[1] : 1;
    if (guess.mismatch || p0 < 8 || p0 >= h->N || h->N % p0 != 0) return PL_OK;
    int dims[3], n_dims;
    if (p1 == 1) {                      // feature 1 changes with every point: an image
        n_dims = 2;
        dims[0] = h->N / p0;
        dims[1] = p0;
    } else {                            // feature 1 changes every p1 points: a volume
        if (p1 < 4 || p0 % p1 != 0 || p0 / p1 < 2) return PL_OK;
        n_dims = 3;
        dims[0] = h->N / p0;
        dims[1] = p0 / p1;
        dims[2] = p1;
    }
    if (dims[0] < 2) return PL_OK;
    h->map = plk::make_point_map(h->N, n_dims, dims);
    h->numbering_pass_pays = false;
    h->one_segment_for = 0;
    h->one_segment_backoff = 32;
    return ensure_replay(h, false);
}

// Checks the arguments of the *_image entry points, sets the grid hint and describes the features.
int features_from_image(pl_lattice *h, const float *reference, int n_reference_channels,
                        int n_spatial_dims, const int *spatial_dims, float spatial_std,
                        float feature_std, plk::PointFeatures *out) {
    if (n_reference_channels < 0 || n_spatial_dims < 0) return PL_EINVAL;
    if (n_spatial_dims > plk::kMaxSpatialDims) return PL_EUNSUPPORTED;
    if (n_spatial_dims + n_reference_channels != h->pd) return PL_EINVAL;
    if (n_spatial_dims > 0 && !spatial_dims) return PL_EINVAL;
    if (n_reference_channels > 0 && !reference && h->N > 0) return PL_EINVAL;
    plk::PointFeatures f{};
    f.reference = reference;
    f.n_spatial_dims = n_spatial_dims;
    f.n_reference_channels = n_reference_channels;
    f.spatial_std = spatial_std;
    f.feature_std = feature_std;
    for (int i = 0; i < plk::kMaxSpatialDims; ++i) f.dims.v[i] = 1;
    for (int i = 0; i < n_spatial_dims; ++i) f.dims.v[i] = spatial_dims[i];
    if (n_spatial_dims > 0) {
        // also checks that the extents are positive and that their product is N
        const int rc = pl_set_point_grid(h, n_spatial_dims, spatial_dims);
        if (rc != PL_OK) return rc;
    }
    *out = f;
    return PL_OK;
}

// pl_build in two halves, as pl_filter below: begin enqueues the build, and behind it the lists
// of a lattice that keeps them, and returns; end waits for the build's report, repeats the build
// with a larger table where it did not fit, and reads how many chunks the lists have.
int enqueue_build_only(pl_lattice *h, const plk::PointFeatures &features, const double *positions64,
                       uint32_t cells, bool lists) {
    int rc = enqueue_build(h, features, positions64, cells, nullptr);
    if (rc != PL_OK) return rc;
    if (lists) {
        // The lattice is there to be applied: per vertex the list of the rows that name it, so
        // that every apply splats by gathering (float values; a build without a splat numbers its
        // vertices densely).  Enqueued before the host waits for the build's report.
        rc = ensure_vertex_lists(h);
        if (rc != PL_OK) return rc;
        PL_HIP(plk::build_vertex_lists(h->pd, h->map, h->replay,
                                       h->replay_holds_cells ? h->cell_vertex : nullptr,
                                       h->max_vertices(), h->lists_of_vertices,
                                       reinterpret_cast<unsigned *>(h->h_status + 1),
                                       h->status_sequence, h->stream));
        h->replay_holds_cells = false;
    }
    return PL_OK;
}

int build_begin(pl_lattice *h, const plk::PointFeatures &features,
                const double *positions64 = nullptr) {
    if (h->pending.active) return PL_ESTATE;
    h->built = false;
    h->M = 0;
    for (int i = 0; i <= EV_NBR; ++i) h->ev_recorded[i] = false;
    if (h->N == 0) {
        h->built = h->verified = true;
        return PL_OK;
    }
    const bool lists = h->vertex_lists && !h->f64 && !h->status_on_device;
    const int rc = enqueue_build_only(h, features, positions64, initial_cells(h), lists);
    if (rc != PL_OK) return rc;
    h->pending.active = true;
    h->pending.build_only = true;
    h->pending.lists = lists;
    h->pending.features = features;
    h->pending.positions64 = positions64;
    return PL_OK;
}

int build_end(pl_lattice *h) {
    if (!h->pending.active) return PL_OK;   // nothing in flight (or an empty lattice)
    if (!h->pending.build_only) return PL_ESTATE;
    const bool lists = h->pending.lists;
    for (;;) {
        uint32_t cells = 0;
        int rc = verify_build(h, &cells);
        if (rc == PL_OK) break;
        if (cells) rc = enqueue_build_only(h, h->pending.features, h->pending.positions64, cells, lists);
        if (!cells || rc != PL_OK) {
            h->pending.active = false;
            return rc;
        }
    }
    h->pending.active = false;
    if (lists && h->n_segments == 0) {
        // (how many chunks there are, and whether any list has several, sizes every apply's
        // launches: the last kernel of the lists wrote them behind the build's status, in pinned
        // memory; read once here, where the caller is building and expects to wait)
        const volatile unsigned *info = reinterpret_cast<const volatile unsigned *>(h->h_status + 1);
        const int rc = wait_for_report(h, info + 2);
        if (rc != PL_OK) return rc;
        const plk::ListChunks &c = h->lists_of_vertices.chunks;
        h->long_lists = info[0] < c.max_long ? info[0] : c.max_long;
        h->list_chunks = info[1] < c.max_chunks ? info[1] : c.max_chunks;
        h->lists_valid = true;
    }
    return PL_OK;
}

int build_lattice(pl_lattice *h, const plk::PointFeatures &features,
                  const double *positions64 = nullptr) {
    const int rc = build_begin(h, features, positions64);
    return rc == PL_OK ? build_end(h) : rc;
}

// pl_filter in two halves.  begin: build and apply are enqueued together and the call returns.
// end: waits for the lattice's stream; if the table turned out too small the whole call is
// repeated with a larger one (the output is simply written again).
int filter_begin(pl_lattice *h, void *output, const void *input,
                 const plk::PointFeatures &features, int reverse,
                 const double *positions64 = nullptr) {
    if (h->pending.active) return PL_ESTATE;
    h->built = false;
    h->M = 0;
    for (int i = 0; i < EV_COUNT; ++i) h->ev_recorded[i] = false;
    if (h->N == 0) {
        h->built = h->verified = true;
        return PL_OK;
    }
    const uint32_t cells = initial_cells(h);
    // (only a lattice of floats splats in its build, and its input is then floats)
    int rc = enqueue_build(h, features, positions64, cells, input);
    if (rc != PL_OK) return rc;
    rc = enqueue_apply(h, output, input, reverse);
    if (rc != PL_OK) return rc;
    h->pending.active = true;
    h->pending.build_only = false;
    h->pending.features = features;
    h->pending.positions64 = positions64;
    h->pending.output = output;
    h->pending.input = input;
    h->pending.reverse = reverse;
    return PL_OK;
}

int filter_end(pl_lattice *h) {
    if (!h->pending.active) return PL_OK;   // nothing in flight (or an empty lattice)
    if (h->pending.build_only) return PL_ESTATE;
    for (;;) {
        uint32_t cells = 0;
        int rc = verify_build(h, &cells);
        if (rc == PL_OK || !cells) {
            h->pending.active = false;
            return rc;
        }
        rc = enqueue_build(h, h->pending.features, h->pending.positions64, cells,
                           h->pending.input);
        if (rc == PL_OK) rc = enqueue_apply(h, h->pending.output, h->pending.input, h->pending.reverse);
        if (rc != PL_OK) {
            h->pending.active = false;
            return rc;
        }
    }
}

int filter_lattice(pl_lattice *h, void *output, const void *input,
                   const plk::PointFeatures &features, int reverse,
                   const double *positions64 = nullptr) {
    const int rc = filter_begin(h, output, input, features, reverse, positions64);
    return rc == PL_OK ? filter_end(h) : rc;
}

}  // namespace

int pl_build(pl_handle h, const float *positions) {
    if (!h || (!positions && h->N > 0)) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->pending.active) return PL_ESTATE;
    const int rc = guess_point_grid(h, positions);
    if (rc != PL_OK) return rc;
    return build_lattice(h, features_from_positions(positions));
}

int pl_build_image(pl_handle h, const float *reference, int n_reference_channels,
                   int n_spatial_dims, const int *spatial_dims, float spatial_std,
                   float feature_std) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->pending.active) return PL_ESTATE;
    plk::PointFeatures features;
    const int rc = features_from_image(h, reference, n_reference_channels, n_spatial_dims,
                                       spatial_dims, spatial_std, feature_std, &features);
    return rc == PL_OK ? build_lattice(h, features) : rc;
}

int pl_build_begin(pl_handle h, const float *positions) {
    if (!h || (!positions && h->N > 0)) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->pending.active) return PL_ESTATE;
    const int rc = guess_point_grid(h, positions);
    if (rc != PL_OK) return rc;
    return build_begin(h, features_from_positions(positions));
}

int pl_build_image_begin(pl_handle h, const float *reference, int n_reference_channels,
                         int n_spatial_dims, const int *spatial_dims, float spatial_std,
                         float feature_std) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->pending.active) return PL_ESTATE;
    plk::PointFeatures features;
    const int rc = features_from_image(h, reference, n_reference_channels, n_spatial_dims,
                                       spatial_dims, spatial_std, feature_std, &features);
    return rc == PL_OK ? build_begin(h, features) : rc;
}

int pl_build_end(pl_handle h) {
    if (!h) return PL_EINVAL;
    return build_end(h);
}

int pl_apply(pl_handle h, float *output, const float *input, int reverse) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (!h->built || !h->verified || h->pending.active) return PL_ESTATE;
    if (h->N == 0) return PL_OK;
    if (!output || !input) return PL_EINVAL;
    return enqueue_apply(h, output, input, reverse);
}

int pl_filter(pl_handle h, float *output, const float *input, const float *positions, int reverse) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->N > 0 && (!output || !input || !positions)) return PL_EINVAL;
    if (h->pending.active) return PL_ESTATE;
    const int rc = guess_point_grid(h, positions);
    if (rc != PL_OK) return rc;
    return filter_lattice(h, output, input, features_from_positions(positions), reverse);
}

int pl_filter_image(pl_handle h, float *output, const float *input, const float *reference,
                    int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                    float spatial_std, float feature_std, int reverse) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->pending.active) return PL_ESTATE;
    if (h->N > 0 && (!output || !input)) return PL_EINVAL;
    plk::PointFeatures features;
    const int rc = features_from_image(h, reference, n_reference_channels, n_spatial_dims,
                                       spatial_dims, spatial_std, feature_std, &features);
    return rc == PL_OK ? filter_lattice(h, output, input, features, reverse) : rc;
}

int pl_filter_begin(pl_handle h, float *output, const float *input, const float *positions,
                    int reverse) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->N > 0 && (!output || !input || !positions)) return PL_EINVAL;
    if (h->pending.active) return PL_ESTATE;
    const int rc = guess_point_grid(h, positions);
    if (rc != PL_OK) return rc;
    return filter_begin(h, output, input, features_from_positions(positions), reverse);
}

int pl_filter_image_begin(pl_handle h, float *output, const float *input, const float *reference,
                          int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                          float spatial_std, float feature_std, int reverse) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (h->pending.active) return PL_ESTATE;
    if (h->N > 0 && (!output || !input)) return PL_EINVAL;
    plk::PointFeatures features;
    const int rc = features_from_image(h, reference, n_reference_channels, n_spatial_dims,
                                       spatial_dims, spatial_std, feature_std, &features);
    return rc == PL_OK ? filter_begin(h, output, input, features, reverse) : rc;
}

// T = double: the same calls on a lattice made by pl_create_f64
int pl_build_f64(pl_handle h, const double *positions) {
    if (!h || !h->f64 || (!positions && h->N > 0)) return PL_EINVAL;
    if (h->pending.active) return PL_ESTATE;
    return build_lattice(h, plk::PointFeatures{}, positions);
}

int pl_apply_f64(pl_handle h, double *output, const double *input, int reverse) {
    if (!h || !h->f64) return PL_EINVAL;
    if (!h->built || !h->verified || h->pending.active) return PL_ESTATE;
    if (h->N == 0) return PL_OK;
    if (!output || !input) return PL_EINVAL;
    return enqueue_apply(h, output, input, reverse);
}

int pl_filter_f64(pl_handle h, double *output, const double *input, const double *positions,
                  int reverse) {
    if (!h || !h->f64) return PL_EINVAL;
    if (h->N > 0 && (!output || !input || !positions)) return PL_EINVAL;
    if (h->pending.active) return PL_ESTATE;
    return filter_lattice(h, output, input, plk::PointFeatures{}, reverse, positions);
}

int pl_debug_simplex_f64(pl_handle h, const double *positions, short *rem0, short *rank,
                         short *keys, double *barycentric) {
    if (!h || !h->f64 || (!positions && h->N > 0)) return PL_EINVAL;
    PL_HIP(plk::debug_simplex_f64(h->pd, positions, h->N, h->scale64, rem0, rank, keys,
                                  barycentric, h->stream));
    return PL_OK;
}

int pl_filter_end(pl_handle h) {
    if (!h) return PL_EINVAL;
    return filter_end(h);
}

int pl_num_vertices(pl_handle h, int *num_vertices) {
    if (!h || !num_vertices) return PL_EINVAL;
    if (!h->built || !h->verified) return PL_ESTATE;
    *num_vertices = h->M;
    return PL_OK;
}

int pl_get_info(pl_handle h, int what, long *value) {
    if (!h || !value) return PL_EINVAL;
    switch (what) {
        case PL_INFO_BUILD_MERGED: *value = h->last_build_merged ? 1 : 0; return PL_OK;
        case PL_INFO_TABLE_CELLS: *value = (long)h->n_cells; return PL_OK;
        case PL_INFO_FOREIGN_ROWS: *value = h->foreign_rows; return PL_OK;
        case PL_INFO_SCRATCH_BYTES: {
            const size_t mv = plk::max_vertices_for(h->n_cells_alloc);
            size_t b = (size_t)h->n_cells_alloc * (sizeof(uint64_t) + sizeof(int)) +
                       mv * (sizeof(uint64_t) + sizeof(int) + 2 * h->value_size() * h->vd +
                             sizeof(int2) * (size_t)(h->pd + 1));
            if (h->cell_values) b += h->value_size() * (size_t)h->n_cells_alloc * h->vd;
            b += h->replay_capacity * (sizeof(plk::ReplayEntry) + sizeof(uint4) +
                                       (h->f64 ? sizeof(double) : 0));
            if (h->lists_of_vertices.start)
                b += sizeof(unsigned) * (3 * h->lists_for_vertices + 5 +
                                         2 * (plk::vertex_list_scan_blocks((int)h->lists_for_vertices) + 1)) +
                     sizeof(plk::LongList) * h->lists_of_vertices.chunks.max_long +
                     (size_t)h->lists_of_vertices.chunks.max_chunks * (sizeof(plk::ListChunk) + sizeof(float) * h->vd) +
                     h->lists_of_vertices.capacity * (sizeof(plk::ListEntry) + sizeof(unsigned));
            if (h->point_order) {
                const unsigned max_bins = plk::locality_bins_for(h->order_capacity);
                b += sizeof(int) * 256 * (size_t)plk::locality_tiles_for(h->order_capacity) +
                     sizeof(uint2) * (size_t)h->order_capacity +
                     sizeof(unsigned) * (33 + 2 * (size_t)max_bins +
                                         3 * (size_t)plk::locality_scan_chunks(max_bins));
            }
            *value = (long)b;
            return PL_OK;
        }
        default: return PL_EINVAL;
    }
}

int pl_stage_ms(pl_handle h, float ms[8]) {
    if (!h || !ms) return PL_EINVAL;
    if (!h->profile) return PL_ESTATE;
    PL_HIP(hipStreamSynchronize(h->stream));
    const int pairs[8][2] = {{EV_T0, EV_CLEAR},   {EV_CLEAR, EV_BUILD}, {EV_BUILD, EV_IDS},
                             {EV_IDS, EV_NBR},    {EV_A0, EV_FILL},     {EV_FILL, EV_SPLAT},
                             {EV_SPLAT, EV_BLUR}, {EV_BLUR, EV_SLICE}};
    for (int i = 0; i < 8; ++i) {
        ms[i] = 0.0f;
        if (h->stage_ran[i] && h->ev_recorded[pairs[i][0]] && h->ev_recorded[pairs[i][1]])
            PL_HIP(hipEventElapsedTime(&ms[i], h->ev[pairs[i][0]], h->ev[pairs[i][1]]));
    }
    return PL_OK;
}

int pl_debug_simplex(pl_handle h, const float *positions, short *rem0, short *rank, short *keys,
                     float *barycentric) {
    if (!h || (!positions && h->N > 0)) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    PL_HIP(plk::debug_simplex(h->pd, positions, h->N, h->scale, rem0, rank, keys, barycentric,
                              h->stream));
    return PL_OK;
}

// The debug exports count the vertices densely, whatever numbers the build gave them: read how
// many each segment holds (these calls are for tests; they wait for the stream).
static int vertex_numbers(pl_lattice *h, plk::VertexNumbers *numbers) {
    plk::Counters counters;
    PL_HIP(hipMemcpyAsync(&counters, h->counters(), sizeof(counters), hipMemcpyDeviceToHost,
                          h->stream));
    PL_HIP(hipStreamSynchronize(h->stream));
    numbers->n_segments = counters.n_segments;
    numbers->stride = plk::segment_stride((uint32_t)h->max_vertices(), counters.n_segments);
    numbers->before[0] = 0;
    for (int k = 0; k < plk::kMaxSegments; ++k)
        numbers->before[k + 1] =
            numbers->before[k] + (k < counters.n_segments ? counters.segment_count[k].n : 0u);
    numbers->total = counters.n_segments ? numbers->before[plk::kMaxSegments] : (unsigned)h->M;
    return numbers->total == (unsigned)h->M ? PL_OK : PL_ESTATE;
}

int pl_debug_keys(pl_handle h, short *keys) {
    if (!h || !keys) return PL_EINVAL;
    if (!h->built || !h->verified) return PL_ESTATE;
    plk::VertexNumbers numbers;
    const int rc = vertex_numbers(h, &numbers);
    if (rc != PL_OK) return rc;
    PL_HIP(plk::export_keys(h->pd, h->vertex_keys, numbers, keys, h->wide_keys, h->stream));
    return PL_OK;
}

int pl_debug_values(pl_handle h, void *values) {
    if (!h || !values) return PL_EINVAL;
    if (!h->built || !h->verified) return PL_ESTATE;
    if (h->M == 0) return PL_OK;
    plk::VertexNumbers numbers;
    const int rc = vertex_numbers(h, &numbers);
    if (rc != PL_OK) return rc;
    PL_HIP(plk::export_values(h->values[h->current_values], h->f64 ? 2 * h->vd : h->vd, numbers,
                              static_cast<float *>(values), h->stream));
    return PL_OK;
}

int pl_debug_replay(pl_handle h, int *vertex, float *weight) {
    if (!h) return PL_EINVAL;
    if (h->f64) return PL_EINVAL;   // a lattice of doubles: use the *_f64 entry points
    if (!h->built || !h->verified) return PL_ESTATE;
    plk::VertexNumbers numbers;
    const int rc = vertex_numbers(h, &numbers);
    if (rc != PL_OK) return rc;
    PL_HIP(plk::export_replay(h->pd, h->map, h->replay,
                              h->replay_holds_cells ? h->cell_vertex : nullptr, numbers, vertex,
                              weight, h->stream));
    return PL_OK;
}

int pl_compute_positions(const float *reference, float *positions, int num_super_pixels,
                         int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                         float spatial_std, float feature_std, pl_stream stream) {
    if (num_super_pixels < 0 || n_reference_channels < 0 || n_spatial_dims < 0) return PL_EINVAL;
    if (n_spatial_dims > plk::kMaxSpatialDims) return PL_EUNSUPPORTED;
    if (n_spatial_dims + n_reference_channels < 1) return PL_EINVAL;
    if (num_super_pixels == 0) return PL_OK;
    if (!positions || (n_spatial_dims > 0 && !spatial_dims)) return PL_EINVAL;
    if (n_reference_channels > 0 && !reference) return PL_EINVAL;
    plk::SpatialDims dims{};
    for (int i = 0; i < plk::kMaxSpatialDims; ++i) dims.v[i] = 1;
    for (int i = 0; i < n_spatial_dims; ++i) {
        if (spatial_dims[i] < 1) return PL_EINVAL;
        dims.v[i] = spatial_dims[i];
    }
    PL_HIP(plk::compute_positions(reference, positions, num_super_pixels, n_reference_channels,
                                  n_spatial_dims, dims, spatial_std, feature_std,
                                  (hipStream_t)stream));
    return PL_OK;
}

int pl_compute_positions_f64(const double *reference, double *positions, int num_super_pixels,
                             int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                             double spatial_std, double feature_std, pl_stream stream) {
    if (num_super_pixels < 0 || n_reference_channels < 0 || n_spatial_dims < 0) return PL_EINVAL;
    if (n_spatial_dims > plk::kMaxSpatialDims) return PL_EUNSUPPORTED;
    if (n_spatial_dims + n_reference_channels < 1) return PL_EINVAL;
    if (num_super_pixels == 0) return PL_OK;
    if (!positions || (n_spatial_dims > 0 && !spatial_dims)) return PL_EINVAL;
    if (n_reference_channels > 0 && !reference) return PL_EINVAL;
    plk::SpatialDims dims{};
    for (int i = 0; i < plk::kMaxSpatialDims; ++i) dims.v[i] = 1;
    for (int i = 0; i < n_spatial_dims; ++i) {
        if (spatial_dims[i] < 1) return PL_EINVAL;
        dims.v[i] = spatial_dims[i];
    }
    PL_HIP(plk::compute_positions_f64(reference, positions, num_super_pixels, n_reference_channels,
                                      n_spatial_dims, dims, spatial_std, feature_std,
                                      (hipStream_t)stream));
    return PL_OK;
}

}  // extern "C"

// ------------------------------------------------------------------------------------------------
// Op level: shape arithmetic and per-item loop of LatticeFilterOp::Compute
// (src/LatticeFilterKernel.cpp:111-179 of the reference tree)
// ------------------------------------------------------------------------------------------------
namespace {

// With the default allocator the op keeps its lattices between calls (per device, shape and
// stream), because hipMalloc/hipFree per call would serialise the device.  A batch is spread
// over up to g_op_lanes lattices, the first on the caller's stream, the others on streams of
// their own: the items are independent lattices (LatticeFilterKernel.cpp:152-179), and the
// kernels over the few hundred thousand vertices of one item leave most of the GPU idle.
// With a caller-supplied allocator everything is taken from it and returned before the call
// ends, as the reference does with TensorFlow temporaries (src/DeviceMemoryAllocator.h:52-71),
// and the items run one after the other.
struct OpLane {
    pl_handle lattice = nullptr;
    hipStream_t stream = nullptr;   // owned unless it is the caller's (lane 0)
    bool owns_stream = false;
    hipEvent_t done = nullptr;
};
struct OpCacheEntry {
    int device, pd, vd, N;
    hipStream_t stream;
    bool f64;                       // lattices of doubles
    std::vector<OpLane> lanes;
    hipEvent_t fork = nullptr;
    double *positions64 = nullptr;  // [N*pd], the positions of the item being filtered (doubles only)
};
std::mutex g_op_cache_mutex;
std::vector<OpCacheEntry> g_op_cache;
constexpr size_t kOpCacheMax = 8;
constexpr int kOpLanesMax = 8;
int g_op_lanes = 4;

void destroy_entry(OpCacheEntry &e) {
    for (auto &lane : e.lanes) {
        pl_destroy(lane.lattice);   // waits for the lane's stream
        if (lane.done) (void)hipEventDestroy(lane.done);
        if (lane.owns_stream && lane.stream) (void)hipStreamDestroy(lane.stream);
    }
    if (e.fork) (void)hipEventDestroy(e.fork);
    if (e.positions64) (void)hipFree(e.positions64);
    e.positions64 = nullptr;
    e.lanes.clear();
}

// The cached lattices for this device, shape, stream and value type (g_op_cache_mutex held).
OpCacheEntry *op_cache_entry(int device, int pd, int vd, int N, hipStream_t stream, bool f64) {
    for (auto &e : g_op_cache)
        if (e.device == device && e.pd == pd && e.vd == vd && e.N == N && e.stream == stream &&
            e.f64 == f64)
            return &e;
    if (g_op_cache.size() >= kOpCacheMax) {
        destroy_entry(g_op_cache.front());
        g_op_cache.erase(g_op_cache.begin());
    }
    g_op_cache.push_back(OpCacheEntry{device, pd, vd, N, stream, f64, {}, nullptr, nullptr});
    return &g_op_cache.back();
}

// Lattices and streams for `want` concurrent items.
int ensure_lanes(OpCacheEntry &e, int want) {
    while ((int)e.lanes.size() < want) {
        OpLane lane;
        if (e.lanes.empty()) {
            lane.stream = e.stream;
        } else {
            PL_HIP(hipStreamCreateWithFlags(&lane.stream, hipStreamNonBlocking));
            lane.owns_stream = true;
        }
        int rc = e.f64 ? pl_create_f64(e.pd, e.vd, e.N, (pl_stream)lane.stream, nullptr, &lane.lattice)
                       : pl_create(e.pd, e.vd, e.N, (pl_stream)lane.stream, nullptr, &lane.lattice);
        if (rc == PL_OK && hipEventCreateWithFlags(&lane.done, hipEventDisableTiming) != hipSuccess)
            rc = PL_EHIP;
        if (rc != PL_OK) {
            pl_destroy(lane.lattice);
            if (lane.owns_stream) (void)hipStreamDestroy(lane.stream);
            return rc;
        }
        e.lanes.push_back(lane);
    }
    if (want > 1 && !e.fork) PL_HIP(hipEventCreateWithFlags(&e.fork, hipEventDisableTiming));
    return PL_OK;
}

}  // namespace

extern "C" int pl_lattice_filter_op(const float *input, const float *reference, float *output,
                                    int batch, int n_spatial_dims, const int *spatial_dims,
                                    int n_input_channels, int n_reference_channels, int bilateral,
                                    float theta_alpha, float theta_beta, float theta_gamma,
                                    int reverse, pl_stream stream, const pl_alloc *alloc) {
    if (batch < 0 || n_spatial_dims < 1 || n_input_channels < 1 || !spatial_dims) return PL_EINVAL;
    if (n_spatial_dims > plk::kMaxSpatialDims) return PL_EUNSUPPORTED;
    long long n = 1;
    for (int i = 0; i < n_spatial_dims; ++i) {
        if (spatial_dims[i] < 1) return PL_EINVAL;
        n *= spatial_dims[i];
        if (n > 2147483647LL) return PL_EOVERFLOW;
    }
    // the reference refuses tensors with more than INT32_MAX elements (LatticeFilterKernel.cpp:108)
    if (n * (long long)batch * n_input_channels > 2147483647LL) return PL_EOVERFLOW;
    const int N = (int)n;
    const int vd = n_input_channels + 1;
    const int ref_ch = bilateral ? n_reference_channels : 0;
    if (bilateral && (n_reference_channels < 1 || (!reference && batch > 0))) return PL_EINVAL;
    const int pd = n_spatial_dims + ref_ch;
    // bilateral: theta_alpha / theta_beta; spatial only: theta_gamma (LatticeFilterKernel.cpp:131-142)
    const float spatial_std = bilateral ? theta_alpha : theta_gamma;
    const float feature_std = bilateral ? theta_beta : -1.0f;
    if (!pl_supported(pd, vd)) return PL_EUNSUPPORTED;
    if (batch == 0) return PL_OK;
    if (!input || !output) return PL_EINVAL;

    int device = 0;
    PL_HIP(hipGetDevice(&device));

    if (alloc) {
        // caller's scratch: one lattice, items one after the other, everything returned at the end
        pl_handle lattice = nullptr;
        int rc = pl_create(pd, vd, N, stream, alloc, &lattice);
        for (int b = 0; b < batch && rc == PL_OK; ++b) {
            const float *ref_b = ref_ch ? reference + (size_t)b * N * ref_ch : nullptr;
            rc = pl_filter_image(lattice, output + (size_t)b * N * n_input_channels,
                                 input + (size_t)b * N * n_input_channels, ref_b, ref_ch,
                                 n_spatial_dims, spatial_dims, spatial_std, feature_std, reverse);
        }
        pl_destroy(lattice);  // synchronises the stream first
        return rc;
    }

    // held for the whole call: cached lattices are not re-entrant
    std::lock_guard<std::mutex> lock(g_op_cache_mutex);
    OpCacheEntry *entry = op_cache_entry(device, pd, vd, N, (hipStream_t)stream, false);
    // Items in flight: small items leave most of the GPU idle and gain from four at a time
    // (512x512: 1.44 -> 0.87 ms for eight items forward + reverse); the kernels of an item of a
    // million points fill it, and more than two such items only crowd each other (1.37 / 1.21 /
    // 1.32 ms for one / two / four at a time).
    int n_lanes = batch < g_op_lanes ? batch : g_op_lanes;
    if (N > (1 << 19) && n_lanes > 2) n_lanes = 2;
    int rc = ensure_lanes(*entry, n_lanes);
    if (rc != PL_OK) return rc;

    // the other lanes start after whatever the caller's stream holds so far
    if (n_lanes > 1) {
        PL_HIP(hipEventRecord(entry->fork, (hipStream_t)stream));
        for (int l = 1; l < n_lanes; ++l)
            PL_HIP(hipStreamWaitEvent(entry->lanes[l].stream, entry->fork, 0));
    }
    // One lattice per batch item (LatticeFilterKernel.cpp:152-179).  The feature vectors are built
    // inside the lattice's first kernel, from the item's reference image and the grid coordinates.
    for (int b = 0; b < batch && rc == PL_OK; ++b) {
        pl_handle lattice = entry->lanes[b % n_lanes].lattice;
        rc = pl_filter_end(lattice);   // the item this lane took before
        if (rc != PL_OK) break;
        const float *ref_b = ref_ch ? reference + (size_t)b * N * ref_ch : nullptr;
        rc = pl_filter_image_begin(lattice, output + (size_t)b * N * n_input_channels,
                                   input + (size_t)b * N * n_input_channels, ref_b, ref_ch,
                                   n_spatial_dims, spatial_dims, spatial_std, feature_std, reverse);
    }
    // every lane is drained, also after an error; the caller's stream continues after all of them
    for (int l = 0; l < n_lanes; ++l) {
        const int rc_end = pl_filter_end(entry->lanes[l].lattice);
        if (rc == PL_OK) rc = rc_end;
    }
    for (int l = 1; l < n_lanes; ++l) {
        if (hipEventRecord(entry->lanes[l].done, entry->lanes[l].stream) != hipSuccess ||
            hipStreamWaitEvent((hipStream_t)stream, entry->lanes[l].done, 0) != hipSuccess) {
            if (rc == PL_OK) rc = PL_EHIP;
        }
    }
    return rc;
}

extern "C" int pl_set_op_concurrency(int lanes) {
    if (lanes < 1 || lanes > kOpLanesMax) return PL_EINVAL;
    std::lock_guard<std::mutex> lock(g_op_cache_mutex);
    g_op_lanes = lanes;
    return PL_OK;
}

// The op for T = double (registered by the reference next to float,
// src/LatticeFilterKernel.cpp:196-208): positions are built per item, as the reference does
// (:153-160), and the items are filtered one after the other on one lattice.  With a caller's
// allocator its scratch and the positions array come from there and are returned before the call
// ends; without one the lattice and the positions array are kept between calls like the float
// op's.
extern "C" int pl_lattice_filter_op_f64(const double *input, const double *reference, double *output,
                                        int batch, int n_spatial_dims, const int *spatial_dims,
                                        int n_input_channels, int n_reference_channels,
                                        int bilateral, float theta_alpha, float theta_beta,
                                        float theta_gamma, int reverse, pl_stream stream,
                                        const pl_alloc *alloc) {
    if (batch < 0 || n_spatial_dims < 1 || n_input_channels < 1 || !spatial_dims) return PL_EINVAL;
    if (n_spatial_dims > plk::kMaxSpatialDims) return PL_EUNSUPPORTED;
    if (alloc && (!alloc->alloc || !alloc->free)) return PL_EINVAL;
    long long n = 1;
    for (int i = 0; i < n_spatial_dims; ++i) {
        if (spatial_dims[i] < 1) return PL_EINVAL;
        n *= spatial_dims[i];
        if (n > 2147483647LL) return PL_EOVERFLOW;
    }
    if (n * (long long)batch * n_input_channels > 2147483647LL) return PL_EOVERFLOW;
    const int N = (int)n;
    const int vd = n_input_channels + 1;
    const int ref_ch = bilateral ? n_reference_channels : 0;
    if (bilateral && (n_reference_channels < 1 || (!reference && batch > 0))) return PL_EINVAL;
    const int pd = n_spatial_dims + ref_ch;
    // the attributes are floats for every T (LatticeFilterKernel.cpp:36-38)
    const double spatial_std = bilateral ? theta_alpha : theta_gamma;
    const double feature_std = bilateral ? theta_beta : -1.0f;
    if (!pl_supported(pd, vd)) return PL_EUNSUPPORTED;
    if (batch == 0) return PL_OK;
    if (!input || !output) return PL_EINVAL;

    // pl_filter_f64 returns after the build has been waited for, and the build's kernel is the
    // only reader of the positions, so the next item may overwrite them
    auto filter_items = [&](pl_handle lattice, double *positions) {
        int rc = pl_set_point_grid(lattice, n_spatial_dims, spatial_dims);
        for (int b = 0; b < batch && rc == PL_OK; ++b) {
            const double *ref_b = ref_ch ? reference + (size_t)b * N * ref_ch : nullptr;
            rc = pl_compute_positions_f64(ref_b, positions, N, ref_ch, n_spatial_dims,
                                          spatial_dims, spatial_std, feature_std, stream);
            if (rc == PL_OK)
                rc = pl_filter_f64(lattice, output + (size_t)b * N * n_input_channels,
                                   input + (size_t)b * N * n_input_channels, positions, reverse);
        }
        return rc;
    };
    const size_t position_bytes = sizeof(double) * (size_t)N * (size_t)pd;

    if (alloc) {
        pl_handle lattice = nullptr;
        int rc = pl_create_f64(pd, vd, N, stream, alloc, &lattice);
        double *positions = nullptr;
        if (rc == PL_OK) {
            positions = (double *)alloc->alloc(alloc->ctx, position_bytes);
            if (!positions) rc = PL_ENOMEM;
        }
        if (rc == PL_OK) rc = filter_items(lattice, positions);
        pl_destroy(lattice);   // synchronises the stream first
        if (positions) alloc->free(alloc->ctx, positions);
        return rc;
    }

    int device = 0;
    PL_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(g_op_cache_mutex);
    OpCacheEntry *entry = op_cache_entry(device, pd, vd, N, (hipStream_t)stream, true);
    int rc = ensure_lanes(*entry, 1);
    if (rc != PL_OK) return rc;
    if (!entry->positions64 &&
        hip_failed(hipMalloc((void **)&entry->positions64, position_bytes))) {
        entry->positions64 = nullptr;
        return PL_ENOMEM;
    }
    return filter_items(entry->lanes[0].lattice, entry->positions64);
}

// ------------------------------------------------------------------------------------------------
// pl_filter_static: pl_filter on a lattice whose every array lies in a static device array, for
// callers that cannot allocate.  No hipMalloc, hipFree, hipHostMalloc or event creation anywhere
// on this path; the lattice object itself is static host memory.
// ------------------------------------------------------------------------------------------------
namespace {

constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
constexpr long long kStaticMaxRows = 1 << 17;   // N * (pd + 1)
constexpr int kStaticMaxVd = 8;
constexpr int kStaticMaxDevices = 32;

// Every GPU the library runs on holds its own copy of this array, at its own address, until the
// process ends.  In host code the name is a stand-in for the symbol, never an address to pass on:
// the address on the current device comes from hipGetSymbolAddress (static_scratch_of).
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct StaticLattice {
    unsigned char *base = nullptr;   // address of `scratch` on this device
    size_t used = 0;
    pl_lattice lattice;
};
StaticLattice g_static[kStaticMaxDevices];
std::mutex g_static_mutex;

void *static_alloc(void *ctx, size_t bytes) {
    StaticLattice *st = static_cast<StaticLattice *>(ctx);
    const size_t start = (st->used + 255) & ~(size_t)255;
    if (start + bytes > kStaticScratchBytes) return nullptr;
    st->used = start + bytes;
    return st->base + start;
}
void static_free(void *, void *) {}

// The address of `scratch` on the current device, asked for once per device.
int static_scratch_of(int device, StaticLattice **out) {
    if (device < 0 || device >= kStaticMaxDevices) return PL_EUNSUPPORTED;
    StaticLattice *st = &g_static[device];
    if (!st->base) {
        void *ptr = nullptr;
        PL_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return PL_EHIP;
        st->base = static_cast<unsigned char *>(ptr);
    }
    *out = st;
    return PL_OK;
}

}  // namespace

extern "C" int pl_filter_static(int pd, int vd, int N, float *output, const float *input,
                                const float *positions, int reverse, pl_stream stream) {
    if (N < 0 || pd < 1 || vd < 2) return PL_EINVAL;
    if (!pl_supported(pd, vd)) return PL_EUNSUPPORTED;
    if ((long long)N * (pd + 1) > kStaticMaxRows || vd > kStaticMaxVd) return PL_ETOOLARGE;
    if (N == 0) return PL_OK;
    if (!output || !input || !positions) return PL_EINVAL;

    // one call at a time per process: the calls share the lattice object below, and on a GPU the
    // array itself (the call returns when its work on the stream is done, see verify_build)
    std::lock_guard<std::mutex> lock(g_static_mutex);
    int device = 0;
    PL_HIP(hipGetDevice(&device));
    // the array's address is that of the current device: a stream of another GPU would run the
    // kernels there with this one's address (NULL, the default stream, follows the current device)
    if (stream) {
        int stream_device = -1;
        PL_HIP(hipStreamGetDevice((hipStream_t)stream, &stream_device));
        if (stream_device != device) return PL_EINVAL;
    }
    StaticLattice *st = nullptr;
    int rc = static_scratch_of(device, &st);
    if (rc != PL_OK) return rc;

    // A fresh lattice over the array: whatever the last call left there is cleared by the build
    // as for memory that has just been allocated (hash cells, rows of sums, counters, chunk sums).
    st->used = 0;
    st->lattice = pl_lattice();
    pl_lattice *h = &st->lattice;
    h->pd = pd;
    h->vd = vd;
    h->N = N;
    h->device = device;
    h->stream = (hipStream_t)stream;
    h->alloc.alloc = static_alloc;
    h->alloc.free = static_free;
    h->alloc.ctx = st;
    compute_scale_factor(pd, h->scale);
    compute_scale_factor(pd, h->scale64);
    // a table that holds N*(pd+1) vertices, the most there can be: no build is ever repeated
    const uint64_t rows = (uint64_t)N * (uint64_t)(pd + 1);
    h->max_cells = pow2_at_least(rows * 2 < 4096 ? 4096 : rows * 2);
    h->forced_cells = (long)h->max_cells;
    h->guess_grid = false;   // (looking for a grid in the positions would allocate and wait)
    h->may_widen = false;    // (keys of two words would need the arrays allocated again)
    h->order_points = false; // (no room for the arrays of the ordering pass)
    h->map = plk::make_point_map(N, 0, nullptr);
    h->status_on_device = true;
    rc = ensure_replay(h, false);
    if (rc != PL_OK) return rc;
    h->d_counters = (plk::Counters *)h->dmalloc(2 * sizeof(plk::Counters));
    h->h_status = (plk::HostStatus *)h->dmalloc(sizeof(plk::HostStatus));
    if (!h->d_counters || !h->h_status) return PL_ENOMEM;
    PL_HIP(plk::fill_zero(reinterpret_cast<float *>(h->d_counters),
                          2 * sizeof(plk::Counters) / sizeof(float), h->stream));
    rc = filter_lattice(h, output, input, features_from_positions(positions), reverse);
    // verify_build has waited for the stream; after an error make sure nothing is left running
    // on an array the next call will overwrite
    if (rc != PL_OK) (void)hipStreamSynchronize(h->stream);
    return rc;
}
