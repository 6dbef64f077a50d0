// C entry points around the reference's own CPU header, for validating the oracle and as the
// "reference" CPU baseline.  TEST INFRASTRUCTURE ONLY.
//
// This file contains no reference code: it includes src/PermutohedralLatticeCPU.h from the
// reference tree at build time (see oracle/Makefile; -I points there, -fno-access-control
// exposes the private per-point functions so their intermediate results can be dumped).
// The resulting library lives in oracle/_ref/ and is never committed.
#include <cmath>
#include <cstdio>   // the reference header uses printf/sqrt/ceil/floor without including these
#include <cstdlib>
#include <ctime>

// the header reports every growth of its hash table on stdout; keep stdout clean for callers
// that print machine-readable results
#define printf(...) ((void)0)
#include "PermutohedralLatticeCPU.h"
#undef printf

namespace {
double now_seconds() {
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return double(ts.tv_sec) + 1e-9 * double(ts.tv_nsec);
}

template <typename T>
void scale_factor(int pd, T *scale) {
    PermutohedralLatticeCPU<T> lattice(pd, 2, 1);
    for (int i = 0; i < pd; ++i) scale[i] = lattice.scaleFactor[i];
}

template <typename T>
void dump_simplex(int pd, int N, const T *positions, short *rem0, short *rank, short *keys,
                  T *barycentric, T *elevated) {
    PermutohedralLatticeCPU<T> lattice(pd, 2, 1);
    const int d1 = pd + 1;
    for (int n = 0; n < N; ++n) {
        lattice.embed_position_vector(positions + size_t(n) * pd);
        lattice.find_enclosing_simplex();
        lattice.compute_barycentric_coordinates();
        for (int i = 0; i < d1; ++i) {
            if (elevated) elevated[size_t(n) * d1 + i] = lattice.elevated[i];
            if (rem0) rem0[size_t(n) * d1 + i] = short(lattice.rem0[i]);
            if (rank) rank[size_t(n) * d1 + i] = lattice.rank[i];
            if (barycentric) barycentric[size_t(n) * d1 + i] = lattice.barycentric[i];
            if (keys) {
                // same expression the reference's splat uses to address vertex i
                for (int k = 0; k < pd; ++k) {
                    short c = static_cast<short>(lattice.rem0[k] + i);
                    if (lattice.rank[k] > pd - i) c -= (pd + 1);
                    keys[(size_t(n) * d1 + i) * pd + k] = c;
                }
            }
        }
    }
}

template <typename T>
void compute_positions(const T *reference, T *positions, int num_super_pixels,
                             int reference_channels, int n_sdims, const int *sdims,
                             T spatial_std, T feature_std) {
    compute_kernel_cpu<T>(reference, positions, num_super_pixels, reference_channels, n_sdims,
                              sdims, spatial_std, feature_std);
}

// One filter call on a fresh lattice.  Optional outputs: vertex count, keys (first-touch
// order, caller provides N*(pd+1)*pd shorts at most), seconds for the whole call.
template <typename T>
void filter(int pd, int vd, int N, T *output, const T *input,
                  const T *positions, int reverse, int *num_vertices, short *keys_out,
                  double *seconds) {
    const double t0 = now_seconds();
    {
        PermutohedralLatticeCPU<T> lattice(pd, vd, N);
        lattice.filter(output, input, positions, reverse != 0);
        if (seconds) *seconds = now_seconds() - t0;
        if (num_vertices) *num_vertices = lattice.hashTable.size();
        if (keys_out) {
            const short *k = lattice.hashTable.getKeys();
            for (size_t i = 0; i < size_t(lattice.hashTable.size()) * pd; ++i) keys_out[i] = k[i];
        }
    }
}

// Stage-by-stage run exposing the vertex values after splat and after blur
// (each M*vd floats, caller sizes them for N*(pd+1) vertices), and per-stage seconds.
template <typename T>
void filter_stages(int pd, int vd, int N, T *output, const T *input,
                         const T *positions, int reverse, int *num_vertices,
                         T *values_after_splat, T *values_after_blur,
                         double *stage_seconds /* splat, blur, slice */) {
    PermutohedralLatticeCPU<T> lattice(pd, vd, N);
    double t0 = now_seconds();
    lattice.splat(positions, input);
    double t1 = now_seconds();
    const int M = lattice.hashTable.size();
    if (num_vertices) *num_vertices = M;
    if (values_after_splat)
        for (size_t i = 0; i < size_t(M) * vd; ++i) values_after_splat[i] = lattice.hashTable.getValues()[i];
    double t2 = now_seconds();
    lattice.blur(reverse != 0);
    double t3 = now_seconds();
    if (values_after_blur)
        for (size_t i = 0; i < size_t(M) * vd; ++i) values_after_blur[i] = lattice.hashTable.getValues()[i];
    double t4 = now_seconds();
    lattice.slice(output);
    double t5 = now_seconds();
    if (stage_seconds) {
        stage_seconds[0] = t1 - t0;
        stage_seconds[1] = t3 - t2;
        stage_seconds[2] = t5 - t4;
    }
}

// One filter call that also hands out what the slice replays: per point and simplex corner the
// index of the vertex the splat's lookup returned and its weight (matrix[n*(pd+1)+r], the
// reference's {offset = vertex*vd, weight}), and the vertex keys in first-touch order.  Where the
// reference's index doubled and entered a key twice, the list holds that key twice and the rows
// say which of the two each point was given.
template <typename T>
void filter_replay(int pd, int vd, int N, T *output, const T *input, const T *positions,
                   int reverse, int *num_vertices, short *keys_out, int *replay_vertex,
                   T *replay_weight) {
    PermutohedralLatticeCPU<T> lattice(pd, vd, N);
    lattice.filter(output, input, positions, reverse != 0);
    const int M = lattice.hashTable.size();
    if (num_vertices) *num_vertices = M;
    if (keys_out) {
        const short *k = lattice.hashTable.getKeys();
        for (size_t i = 0; i < size_t(M) * pd; ++i) keys_out[i] = k[i];
    }
    for (size_t i = 0; i < size_t(N) * (pd + 1); ++i) {
        if (replay_vertex) replay_vertex[i] = lattice.matrix[i].offset / vd;
        if (replay_weight) replay_weight[i] = lattice.matrix[i].weight;
    }
}

// The op's per-batch-item loop (src/LatticeFilterKernel.cpp:111-179) driven through the
// reference's own CPU functor bodies (compute_kernel_cpu + PermutohedralLatticeCPU::filter).
template <typename T>
int lattice_filter_op(const T *input, const T *reference, T *output, int batch,
                            int n_spatial_dims, const int *spatial_dims, int n_input_channels,
                            int n_reference_channels, int bilateral, float theta_alpha,
                            float theta_beta, float theta_gamma, int reverse) {
    int N = 1;
    for (int i = 0; i < n_spatial_dims; ++i) N *= spatial_dims[i];
    const int vd = n_input_channels + 1;
    const int ref_ch = bilateral ? n_reference_channels : 0;
    const int pd = n_spatial_dims + ref_ch;
    const T spatial_std = bilateral ? theta_alpha : theta_gamma;   // float attributes for every T
    const T feature_std = bilateral ? theta_beta : -1.0f;
    T *positions = new T[size_t(N) * pd];
    for (int b = 0; b < batch; ++b) {
        compute_kernel_cpu<T>(reference + size_t(b) * N * ref_ch, positions, N, ref_ch,
                                  n_spatial_dims, spatial_dims, spatial_std, feature_std);
        PermutohedralLatticeCPU<T> lattice(pd, vd, N);
        lattice.filter(output + size_t(b) * N * n_input_channels,
                       input + size_t(b) * N * n_input_channels, positions, reverse != 0);
    }
    delete[] positions;
    return 0;
}


}  // namespace

// T = float: plref_<name>; T = double: plref_<name>_f64
#define PLREF_EXPORTS(T, SUFFIX)                                                                   \
    void plref_scale_factor##SUFFIX(int pd, T *scale) { scale_factor<T>(pd, scale); }              \
    void plref_dump_simplex##SUFFIX(int pd, int N, const T *positions, short *rem0, short *rank,   \
                                    short *keys, T *barycentric, T *elevated) {                    \
        dump_simplex<T>(pd, N, positions, rem0, rank, keys, barycentric, elevated);                \
    }                                                                                              \
    void plref_compute_positions##SUFFIX(const T *reference, T *positions, int num_super_pixels,   \
                                         int reference_channels, int n_sdims, const int *sdims,    \
                                         T spatial_std, T feature_std) {                           \
        compute_positions<T>(reference, positions, num_super_pixels, reference_channels, n_sdims,  \
                             sdims, spatial_std, feature_std);                                     \
    }                                                                                              \
    void plref_filter##SUFFIX(int pd, int vd, int N, T *output, const T *input,                    \
                              const T *positions, int reverse, int *num_vertices,                  \
                              short *keys_out, double *seconds) {                                  \
        filter<T>(pd, vd, N, output, input, positions, reverse, num_vertices, keys_out, seconds);  \
    }                                                                                              \
    void plref_filter_stages##SUFFIX(int pd, int vd, int N, T *output, const T *input,             \
                                     const T *positions, int reverse, int *num_vertices,           \
                                     T *values_after_splat, T *values_after_blur,                  \
                                     double *stage_seconds) {                                      \
        filter_stages<T>(pd, vd, N, output, input, positions, reverse, num_vertices,               \
                         values_after_splat, values_after_blur, stage_seconds);                    \
    }                                                                                              \
    void plref_filter_replay##SUFFIX(int pd, int vd, int N, T *output, const T *input,             \
                                     const T *positions, int reverse, int *num_vertices,           \
                                     short *keys_out, int *replay_vertex, T *replay_weight) {      \
        filter_replay<T>(pd, vd, N, output, input, positions, reverse, num_vertices, keys_out,     \
                         replay_vertex, replay_weight);                                            \
    }                                                                                              \
    int plref_lattice_filter_op##SUFFIX(const T *input, const T *reference, T *output, int batch,  \
                                        int n_spatial_dims, const int *spatial_dims,               \
                                        int n_input_channels, int n_reference_channels,            \
                                        int bilateral, float theta_alpha, float theta_beta,        \
                                        float theta_gamma, int reverse) {                          \
        return lattice_filter_op<T>(input, reference, output, batch, n_spatial_dims, spatial_dims, \
                                    n_input_channels, n_reference_channels, bilateral,             \
                                    theta_alpha, theta_beta, theta_gamma, reverse);                \
    }

extern "C" {
PLREF_EXPORTS(float, )
PLREF_EXPORTS(double, _f64)
}  // extern "C"
