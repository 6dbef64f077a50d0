/*
 * C ABI of the gfx950 (MI355X) permutohedral-lattice filter.
 *
 * Plain pointers and sizes only.  Every pointer named "device" must be device memory of the
 * GPU that is current when the call is made; all work is enqueued on the lattice's stream.
 * Each entry point cites the reference interface it stands in for (paths are relative to the
 * reference tree, MiguelMonteiro/permutohedral_lattice).
 *
 * Status codes: every function returns PL_OK (0) or a negative pl_status; nothing here calls
 * exit() or throws (the reference GPU path exits the process on errors:
 * src/PermutohedralLatticeGPU.cuh:49-55, src/DeviceMemoryAllocator.h:29-37).
 */
#ifndef PERMUTOHEDRAL_LATTICE_H
#define PERMUTOHEDRAL_LATTICE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum pl_status {
    PL_OK = 0,
    PL_EINVAL = -1,       /* null pointer, negative size, bad option */
    PL_EUNSUPPORTED = -2, /* (pd, vd) outside what the kernels are built for */
    PL_ENOMEM = -3,       /* allocator returned NULL */
    PL_EOVERFLOW = -4,    /* sizes do not fit int32, or lattice coordinates do not fit a short (the range of
                             the reference's keys; pl_filter_static: do not fit the packed 64-bit key) */
    PL_EHIP = -5,         /* a HIP runtime call failed; pl_last_hip_error() has the code */
    PL_ESTATE = -6,       /* pl_apply before pl_build, and the like */
    PL_ETOOLARGE = -7     /* pl_filter_static: the lattice does not fit the library's static scratch */
} pl_status;

/* Opaque lattice object. */
typedef struct pl_lattice *pl_handle;

/* A hipStream_t passed as an untyped pointer (NULL = the default stream). */
typedef void *pl_stream;

/*
 * Scratch-memory callbacks.  Stands in for DeviceMemoryAllocator (src/DeviceMemoryAllocator.h:47-120),
 * which backs the lattice's scratch either with TensorFlow temporaries or with cudaMalloc.
 * NULL in pl_create means hipMalloc/hipFree.
 */
typedef struct pl_alloc {
    void *(*alloc)(void *ctx, size_t bytes); /* device memory, 256-byte aligned, or NULL */
    void (*free)(void *ctx, void *ptr);
    void *ctx;
} pl_alloc;

/* pl_set_option keys */
typedef enum pl_option {
    PL_OPT_NORMALIZE = 1,  /* 1 (default): slice divides by the homogeneous channel as the reference
                              does (src/PermutohedralLatticeCPU.h:347-350).  0: input and output carry all
                              vd channels and nothing is divided -- the bare linear operator, for tests. */
    PL_OPT_PROFILE = 2,    /* 1: record per-stage HIP events, read with pl_stage_ms */
    PL_OPT_TABLE_CELLS = 3, /* force the initial number of hash cells (power of two), 0 = automatic */
    PL_OPT_XCD_AWARE = 4,   /* 1 (default): kernels with atomic updates give each XCD a contiguous range
                               of points; 0: plain workgroup order (for measuring the difference) */
    PL_OPT_PAIR_BLUR = 5,   /* 1 (default): two blur axes per kernel launch (all three when pd = 2 and
                               vd <= 4); 0: one launch per axis (same results bit for bit; for measuring
                               the difference) */
    PL_OPT_GUESS_GRID = 6,  /* 1 (default): a handle without pl_set_point_grid looks, the first time it
                               sees positions, whether they describe a row-major image or volume (feature
                               0 changing exactly every row length points ...) and if so orders its
                               work as with the hint; 0: never (points are a plain list) */
    PL_OPT_MERGE_TILES = 7, /* 1 (default): when the points are a grid, a workgroup of the build merges
                               the keys and sums of its tile in LDS before they go to the hash table;
                               0: every wavefront goes to the table itself (same results; for
                               measuring the difference) */
    PL_OPT_STOP_AFTER = 8,  /* 0 (default): a filter or apply runs to the end.  1: it ends behind the
                               splat, 2: behind the blur; the output is then not written and
                               pl_debug_values gives the vertex values of that stage (for checking the
                               stages one by one against src/PermutohedralLatticeCPU.h:306-317, 362-415) */
    PL_OPT_VERTEX_LISTS = 10, /* 1 (default): pl_build also writes, per vertex, the list of the (point,
                               weight) rows that name it, and every pl_apply on that lattice splats
                               by gathering along those lists (no atomics, the same order of
                               additions on every call); 0: pl_apply splats as pl_filter does, point
                               by point with sums per wavefront (same results up to the order of
                               float additions; for measuring the difference).  Float lattices. */
    PL_OPT_NUMBER_SEGMENTS = 11, /* 0 (default): a build that numbers its vertices itself draws the numbers
                               from 8 counters (one per eighth of the image), or from 64 when it has more
                               than 8192 workgroups; 8 or 64: always that many, table size permitting;
                               -1: no build numbers its vertices itself, the numbering pass runs
                               (same results; for tests and measurements) */
    PL_OPT_ORDER_POINTS = 9 /* 1 (default): points that are a plain list (no grid given or found, at
                               least 4096 of them) are worked on in an order in which neighbours in
                               space are neighbours in the list, found anew by every build from the
                               first two or three features, so that the workgroups of the build can merge their
                               keys as for an image (PL_OPT_MERGE_TILES); 0: in the order of the list
                               (same results up to the order of float additions) */
} pl_option;

/* 1 when a lattice can be built for these dimensions, else 0.
 * Replaces the compile-time (pd, vd) pairs of src/LatticeFilterKernel.cu:87-100 by run-time dispatch. */
int pl_supported(int pd, int vd);

const char *pl_strerror(int status);

/* hipError_t of the last failed HIP call on this thread (0 if none). */
int pl_last_hip_error(void);

/*
 * What this build of the library is, for bindings and harnesses that must not drive a library
 * whose device-side array layouts differ from the ones they were written for (no handle, no GPU
 * needed).  The reference has no counterpart: its host and device code are one translation unit.
 */
typedef enum pl_library_property {
    PL_LIB_LAYOUT_VERSION = 1,   /* bumped whenever the layout of an array that one kernel writes and
                                    another reads changes (replay rows, hash cells, per-vertex tables) */
    PL_LIB_REPLAY_ROW_BYTES = 2, /* size of one replay row (vertex or cell, barycentric weight) */
    PL_LIB_SOURCE_HASH = 3       /* first 48 bits of the SHA-256 over the library's source files as its
                                    build script hashed them (0 when built without the script) */
} pl_library_property;
#define PL_LAYOUT_VERSION 3
int pl_library_info(int what, long long *value);

/*
 * Lattice for (pd, vd, N): pd feature dimensions, vd = value channels + 1 homogeneous, N points.
 * Stands in for PermutohedralLatticeCPU<T>(pd, vd, N) (src/PermutohedralLatticeCPU.h:419) and
 * PermutohedralLatticeGPU<T,pd,vd>(n, allocator, stream) (src/PermutohedralLatticeGPU.cuh:434).
 * Unlike the reference objects, which are single-shot, a handle may be used for any number of
 * filter calls; each behaves as if on a fresh lattice.
 */
int pl_create(int pd, int vd, int N, pl_stream stream, const pl_alloc *alloc, pl_handle *out);
int pl_destroy(pl_handle h);

/*
 * output[N*(vd-1)] = filter(input[N*(vd-1)]) under positions[N*pd]; all three are device pointers,
 * row-major, one row per point.  reverse != 0 visits the blur axes pd..0 (the gradient pass).
 * Stands in for filter(output, input, positions, reverse)
 * (src/PermutohedralLatticeCPU.h:442-446, src/PermutohedralLatticeGPU.cuh:453-479).
 * Equivalent to pl_build followed by pl_apply.  Everything is enqueued at once; the call returns
 * when the build has reported whether its hash table was large enough (the calling thread
 * polls a word in pinned memory that the kernel behind the build writes; if the table was too
 * small, the call is repeated with a larger one), while the rest of the call may still be running.  The output is complete in the order of the
 * lattice's stream, as with the reference's GPU path.
 */
int pl_filter(pl_handle h, float *output, const float *input, const float *positions, int reverse);

/*
 * pl_filter for callers that cannot allocate (code under HIP graph capture elsewhere in the
 * process, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference, whose lattice objects allocate in their constructors
 * (src/PermutohedralLatticeGPU.cuh:434-451).  No handle: the lattice lives for the length of the call
 * in a static device array of 64 MiB inside the library, and the call makes no hipMalloc, hipFree,
 * hipHostMalloc or event.  The array is part of the library's code object: every process that
 * loads the library holds 64 MiB of device memory on each GPU it runs kernels of the library on,
 * until the process ends, whether it ever calls this entry point or not.  `stream` must belong to
 * the GPU that is current when the call is made (NULL: its default stream), else PL_EINVAL.
 * Limits: N*(pd+1) <= 131072 (e.g. 21845 points at pd = 5) and vd <= 8, float values; beyond them
 * PL_ETOOLARGE.  The hash table is sized for N*(pd+1) vertices, so no input makes it overflow.
 * The points are taken as a plain list (no grid is looked for).  Same results as pl_filter; the
 * call returns when its work on `stream` is complete.  All calls on a GPU share that GPU's array
 * and what the last call left in it (each call clears what it needs to be zero), so calls that
 * overlapped on one GPU would race: the library takes a lock for the length of each call.
 */
int pl_filter_static(int pd, int vd, int N, float *output, const float *input,
                     const float *positions, int reverse, pl_stream stream);

/*
 * Build the lattice for positions[N*pd] (embed, enclosing simplex, hash insertion, neighbour
 * table) once; pl_apply then runs splat, blur, slice for any number of inputs, forward or reverse,
 * under those positions.  The reference rebuilds for every call
 * (src/LatticeFilterKernel.cpp:79, src/LatticeFilterKernel.cu:88); results are the same.
 * pl_apply only launches kernels on the lattice's stream (no allocation, no wait, no memset):
 * after the first pl_apply that follows a build, further ones may be captured in a HIP graph.
 */
int pl_build(pl_handle h, const float *positions);
int pl_apply(pl_handle h, float *output, const float *input, int reverse);

/*
 * Optional hint: the N points are a row-major grid of these extents (their product must be N),
 * as the op's tensors are (src/LatticeFilterKernel.cpp:117-124: spatial_dims).  Workgroups then
 * take compact tiles of the grid instead of runs of consecutive points, so more of the points
 * that share lattice vertices meet inside one wavefront.  Results do not depend on the hint.
 * n_dims = 0 removes it.  pl_lattice_filter_op sets it by itself.
 */
int pl_set_point_grid(pl_handle h, int n_dims, const int *dims);

/* The grid the handle currently orders its work by: *n_dims = 0 (none), 2 or 3, extents in dims
 * (leading extents of a longer hint folded into the first).  Given by pl_set_point_grid, by the
 * *_image entry points, or found in the positions (PL_OPT_GUESS_GRID). */
int pl_get_point_grid(pl_handle h, int *n_dims, int dims[3]);

/* Number of lattice vertices of the last build (HashTableCPU::size(), src/PermutohedralLatticeCPU.h:151). */
int pl_num_vertices(pl_handle h, int *num_vertices);

int pl_set_option(pl_handle h, int option, long value);

/* What the handle's last build did (for benchmarks and tests): */
typedef enum pl_info {
    PL_INFO_BUILD_MERGED = 1,  /* 1 when the last build merged its tiles' keys in LDS (PL_OPT_MERGE_TILES), 0
                                  when every wavefront went to the table itself (no grid, or a tile with
                                  too many distinct keys switched merging off for a while) */
    PL_INFO_TABLE_CELLS = 2,   /* hash cells the last build used */
    PL_INFO_SCRATCH_BYTES = 3, /* device memory the handle holds for its tables and per-point rows */
    PL_INFO_FOREIGN_ROWS = 4   /* when the last build numbered its vertices itself: how many rows of sums
                                  its workgroups held for vertices that other workgroups created (an
                                  estimate from every eighth workgroup); else -1 */
} pl_info;
int pl_get_info(pl_handle h, int what, long *value);

/* Milliseconds of the kernels of the last pl_build and pl_apply (or pl_filter) with
 * PL_OPT_PROFILE on, from HIP events on the lattice's stream: ms[0] table clear, ms[1] build
 * (embed + simplex + hash insertion), ms[2] vertex numbering, ms[3] neighbour table, ms[4] value
 * clear, ms[5] splat, ms[6] blur (all pd+1 launches together), ms[7] slice.  Synchronises the stream. */
int pl_stage_ms(pl_handle h, float ms[8]);

/*
 * Debug export of the per-point integer results of the last build, for parity checks; device
 * pointers, any may be NULL: rem0[N*(pd+1)], rank[N*(pd+1)], keys[N*(pd+1)*pd] (vertex-major
 * inside a point), barycentric[N*(pd+1)].  Same quantities as
 * find_enclosing_simplex / compute_barycentric_coordinates / the key loop of splat_point
 * (src/PermutohedralLatticeCPU.h:233-304).
 */
int pl_debug_simplex(pl_handle h, const float *positions, short *rem0, short *rank, short *keys,
                     float *barycentric);

/* Keys of the vertices of the last build, M*pd shorts to device memory, in vertex-index order
 * (HashTableCPU::getKeys(), src/PermutohedralLatticeCPU.h:154; the order is not the reference's). */
int pl_debug_keys(pl_handle h, short *keys);

/* Values of the vertices as the last pl_filter / pl_apply left them, M*vd floats (doubles for a
 * lattice of doubles) to device memory, rows in the vertex order of pl_debug_keys: after the blur,
 * or after the stage PL_OPT_STOP_AFTER names (HashTableCPU::getValues(),
 * src/PermutohedralLatticeCPU.h:157, read after splat :322-326 or blur :362-415). */
int pl_debug_values(pl_handle h, void *values);

/* Vertex index (0..M-1) and weight of each point's simplex vertices of the last build: vertex[(pd+1)*N], weight[(pd+1)*N], laid out [r][n]; device pointers.  The replay
 * matrix of src/PermutohedralLatticeCPU.h:187-191, 314-317. */
int pl_debug_replay(pl_handle h, int *vertex, float *weight);

/*
 * Feature vectors of one batch item: positions[n][0..k) = coordinate / spatial_std (tensor order,
 * last dimension fastest), positions[n][k..k+rc) = reference[n][c] / feature_std.
 * reference and positions are device pointers; spatial_dims is a HOST array of n_spatial_dims ints.
 * Stands in for compute_kernel_cpu / compute_kernel
 * (src/PermutohedralLatticeCPU.h:452-474, src/PermutohedralLatticeGPU.cuh:482-506) and the
 * ComputeKernel functor (src/LatticeFilterKernel.h:42-54).
 */
int pl_compute_positions(const float *reference, float *positions, int num_super_pixels,
                         int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                         float spatial_std, float feature_std, pl_stream stream);

/*
 * pl_filter / pl_build with the feature vectors built on the fly: the result of
 * pl_compute_positions(reference, positions, N, ...) followed by pl_filter(h, output, input,
 * positions, reverse) (or pl_build(h, positions)), without a positions array ever being written
 * or read.  The lattice must have pd = n_spatial_dims + n_reference_channels and N = the product
 * of spatial_dims (a HOST array); the grid hint of pl_set_point_grid is set from them.
 * n_reference_channels = 0: spatial features only, reference may be NULL.
 * Stands in for the pair of functor calls of the op's per-item loop
 * (src/LatticeFilterKernel.cpp:160-178: ComputeKernel, then LatticeFilter), i.e. compute_kernel
 * (src/PermutohedralLatticeGPU.cuh:482-506) fused into the splat stage of filter (:454-479).
 */
int pl_filter_image(pl_handle h, float *output, const float *input, const float *reference,
                    int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                    float spatial_std, float feature_std, int reverse);
int pl_build_image(pl_handle h, const float *reference, int n_reference_channels,
                   int n_spatial_dims, const int *spatial_dims, float spatial_std,
                   float feature_std);

/*
 * pl_filter / pl_filter_image in two halves, for callers that keep several lattices (each on a
 * stream of its own) in flight: *_begin enqueues the whole call on the lattice's stream and
 * returns at once; pl_filter_end waits for the build's report and, should the hash table have
 * turned out too small, repeats the call with a larger one before it returns.  The arguments of *_begin
 * must stay valid until pl_filter_end; between the two only pl_filter_end and pl_destroy may be
 * called on the handle (anything else returns PL_ESTATE).  pl_filter_end with nothing in flight
 * returns PL_OK.  The reference's filter (src/PermutohedralLatticeGPU.cuh:454-479) enqueues on
 * its stream without waiting as well; what the second half adds is the check of the table size.
 */
int pl_filter_begin(pl_handle h, float *output, const float *input, const float *positions,
                    int reverse);
int pl_filter_image_begin(pl_handle h, float *output, const float *input, const float *reference,
                          int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                          float spatial_std, float feature_std, int reverse);
int pl_filter_end(pl_handle h);

/*
 * pl_build / pl_build_image in two halves, for callers that build several lattices at a time
 * (each on a stream of its own): *_begin enqueues the build and returns at once; pl_build_end
 * waits for the build's report, repeats the build with a larger hash table should it have turned
 * out too small, and returns when the lattice is ready for pl_apply.  The arguments of *_begin
 * must stay valid until pl_build_end; between the two only pl_build_end and pl_destroy may be
 * called on the handle (anything else returns PL_ESTATE, also pl_filter_end).  pl_build_end with
 * nothing in flight returns PL_OK.  No counterpart in the reference, which builds inside every
 * filter call (src/LatticeFilterKernel.cpp:79).
 */
int pl_build_begin(pl_handle h, const float *positions);
int pl_build_image_begin(pl_handle h, const float *reference, int n_reference_channels,
                         int n_spatial_dims, const int *spatial_dims, float spatial_std,
                         float feature_std);
int pl_build_end(pl_handle h);

/*
 * The LatticeFilter op on channels-last device tensors input[B, s_1..s_k, C_in],
 * reference[B, s_1..s_k, C_ref] -> output (shape of input).  bilateral: features are
 * (coords/theta_alpha, reference/theta_beta); otherwise coords/theta_gamma and the reference is
 * ignored (may be NULL).  One lattice per batch item.  Stands in for LatticeFilterOp::Compute
 * (src/LatticeFilterKernel.cpp:98-181); its gradient is the same call on the upstream gradient
 * with reverse = 1 (lattice_filter_op_loader.py:32-54).  Scratch comes from alloc; with NULL the
 * library keeps lattices of its own between calls and runs several batch items at a time (see
 * pl_set_op_concurrency).  Returns when every item's build has been checked; the output is
 * complete in the order of `stream`.
 */
int pl_lattice_filter_op(const float *input, const float *reference, float *output, int batch,
                         int n_spatial_dims, const int *spatial_dims, int n_input_channels,
                         int n_reference_channels, int bilateral, float theta_alpha,
                         float theta_beta, float theta_gamma, int reverse, pl_stream stream,
                         const pl_alloc *alloc);

/*
 * How many batch items pl_lattice_filter_op (with alloc = NULL) keeps in flight at once, each on a
 * lattice and a stream of its own (1..8, default 4; 1 = one after the other as the reference's
 * loop, src/LatticeFilterKernel.cpp:152-179).  Items of more than 2^19 points run at most two at
 * a time whatever is set: their kernels fill the GPU.  Process-wide.
 */
int pl_set_op_concurrency(int lanes);

/* ------------------------------------------------------------------------------------------
 * T = double.  The reference is a template over the value type and its op is registered for
 * float and double (src/PermutohedralLatticeCPU.h:173, src/LatticeFilterKernel.cpp:196-208).
 * A lattice made by pl_create_f64 takes positions, inputs and outputs as doubles through the
 * calls below, which mean what their float namesakes mean; pl_destroy, pl_set_point_grid,
 * pl_get_point_grid, pl_set_option, pl_num_vertices, pl_stage_ms and pl_debug_keys serve both
 * kinds, every other float entry point returns PL_EINVAL for a lattice of doubles (and these for
 * a lattice of floats).  The lattice (keys, vertex count) equals the CPU path's for T = double
 * exactly; values agree to rounding of the sums (about 1e-15 relative), because the splat adds
 * in another order than a sequential loop.  The float path is the one tuned for speed (this one
 * runs at roughly half of it), and the points of a lattice of doubles are not looked at for a
 * grid (give one with pl_set_point_grid; the op does).
 * ---------------------------------------------------------------------------------------- */
int pl_create_f64(int pd, int vd, int N, pl_stream stream, const pl_alloc *alloc, pl_handle *out);
int pl_filter_f64(pl_handle h, double *output, const double *input, const double *positions,
                  int reverse);
int pl_build_f64(pl_handle h, const double *positions);
int pl_apply_f64(pl_handle h, double *output, const double *input, int reverse);
int pl_debug_simplex_f64(pl_handle h, const double *positions, short *rem0, short *rank,
                         short *keys, double *barycentric);
/* compute_kernel<double> (src/PermutohedralLatticeCPU.h:452-474, src/LatticeFilterKernel.h:42-54) */
int pl_compute_positions_f64(const double *reference, double *positions, int num_super_pixels,
                             int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                             double spatial_std, double feature_std, pl_stream stream);
/* LatticeFilterOp<Device, double>::Compute (src/LatticeFilterKernel.cpp:98-181); the attributes
 * are floats for every T (:36-38).  One lattice, the items one after the other.  With alloc its
 * scratch and the positions of an item come from there and go back before the call ends; with
 * NULL the library keeps them between calls, as pl_lattice_filter_op does. */
int pl_lattice_filter_op_f64(const double *input, const double *reference, double *output,
                             int batch, int n_spatial_dims, const int *spatial_dims,
                             int n_input_channels, int n_reference_channels, int bilateral,
                             float theta_alpha, float theta_beta, float theta_gamma, int reverse,
                             pl_stream stream, const pl_alloc *alloc);

#ifdef __cplusplus
}
#endif
#endif /* PERMUTOHEDRAL_LATTICE_H */
