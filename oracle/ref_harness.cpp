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
}  // namespace

extern "C" {

void plref_scale_factor(int pd, float *scale) {
    PermutohedralLatticeCPU<float> lattice(pd, 2, 1);
    for (int i = 0; i < pd; ++i) scale[i] = lattice.scaleFactor[i];
}

void plref_dump_simplex(int pd, int N, const float *positions, short *rem0, short *rank,
                        short *keys, float *barycentric, float *elevated) {
    PermutohedralLatticeCPU<float> lattice(pd, 2, 1);
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

void plref_compute_positions(const float *reference, float *positions, int num_super_pixels,
                             int reference_channels, int n_sdims, const int *sdims,
                             float spatial_std, float feature_std) {
    compute_kernel_cpu<float>(reference, positions, num_super_pixels, reference_channels, n_sdims,
                              sdims, spatial_std, feature_std);
}

// One filter call on a fresh lattice.  Optional outputs: vertex count, keys (first-touch
// order, caller provides N*(pd+1)*pd shorts at most), seconds for the whole call.
void plref_filter(int pd, int vd, int N, float *output, const float *input,
                  const float *positions, int reverse, int *num_vertices, short *keys_out,
                  double *seconds) {
    const double t0 = now_seconds();
    {
        PermutohedralLatticeCPU<float> lattice(pd, vd, N);
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
void plref_filter_stages(int pd, int vd, int N, float *output, const float *input,
                         const float *positions, int reverse, int *num_vertices,
                         float *values_after_splat, float *values_after_blur,
                         double *stage_seconds /* splat, blur, slice */) {
    PermutohedralLatticeCPU<float> lattice(pd, vd, N);
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

// The op's per-batch-item loop (src/LatticeFilterKernel.cpp:111-179) driven through the
// reference's own CPU functor bodies (compute_kernel_cpu + PermutohedralLatticeCPU::filter).
int plref_lattice_filter_op(const float *input, const float *reference, float *output, int batch,
                            int n_spatial_dims, const int *spatial_dims, int n_input_channels,
                            int n_reference_channels, int bilateral, float theta_alpha,
                            float theta_beta, float theta_gamma, int reverse) {
    int N = 1;
    for (int i = 0; i < n_spatial_dims; ++i) N *= spatial_dims[i];
    const int vd = n_input_channels + 1;
    const int ref_ch = bilateral ? n_reference_channels : 0;
    const int pd = n_spatial_dims + ref_ch;
    const float spatial_std = bilateral ? theta_alpha : theta_gamma;
    const float feature_std = bilateral ? theta_beta : -1.0f;
    float *positions = new float[size_t(N) * pd];
    for (int b = 0; b < batch; ++b) {
        compute_kernel_cpu<float>(reference + size_t(b) * N * ref_ch, positions, N, ref_ch,
                                  n_spatial_dims, spatial_dims, spatial_std, feature_std);
        PermutohedralLatticeCPU<float> lattice(pd, vd, N);
        lattice.filter(output + size_t(b) * N * n_input_channels,
                       input + size_t(b) * N * n_input_channels, positions, reverse != 0);
    }
    delete[] positions;
    return 0;
}

}  // extern "C"
