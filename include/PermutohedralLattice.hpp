// C++ face of the C ABI in permutohedral_lattice.h, shaped like the reference's own classes so that
// code written against them reads the same:
//
//   * PermutohedralLatticeHIP<T>(pd, vd, N[, stream]) with filter(output, input, positions, reverse)
//     -- PermutohedralLatticeCPU<T>(pd, vd, N) (src/PermutohedralLatticeCPU.h:419-446) and
//        PermutohedralLatticeGPU<T,pd,vd>(n, allocator, stream) (src/PermutohedralLatticeGPU.cuh:434-479),
//        with run-time (pd, vd) and device pointers;
//   * functors LatticeFilter<HipDevice,T> and ComputeKernel<HipDevice,T>
//     -- the device functors of src/LatticeFilterKernel.h:28-54 (same argument lists; the
//        OpKernelContext* becomes an optional allocator);
//   * lattice_filter(...) -- LatticeFilterOp::Compute (src/LatticeFilterKernel.cpp:98-181).
//
// Errors are thrown as PermutohedralError (the reference GPU path calls exit()).  T = float and
// T = double, the two types the reference registers (src/LatticeFilterKernel.cpp:196-208); the
// fused feature builder (filter_image, build_image) exists for float only.
#ifndef PERMUTOHEDRAL_LATTICE_HPP
#define PERMUTOHEDRAL_LATTICE_HPP

#include <stdexcept>
#include <string>

#include "permutohedral_lattice.h"

namespace permutohedral {

class PermutohedralError : public std::runtime_error {
public:
    PermutohedralError(int status, const char *where)
        : std::runtime_error(std::string(where) + ": " + pl_strerror(status)), status_(status) {}
    int status() const { return status_; }

private:
    int status_;
};

inline void check(int status, const char *where) {
    if (status != PL_OK) throw PermutohedralError(status, where);
}

// Stand-in for Eigen::GpuDevice in the functor signatures: the stream work is enqueued on.
struct HipDevice {
    pl_stream stream_ = nullptr;
    pl_stream stream() const { return stream_; }
};

template <typename T>
class PermutohedralLatticeHIP;

template <>
class PermutohedralLatticeHIP<float> {
public:
    PermutohedralLatticeHIP(int pd, int vd, int N, pl_stream stream = nullptr,
                            const pl_alloc *allocator = nullptr) {
        check(pl_create(pd, vd, N, stream, allocator, &handle_), "pl_create");
    }
    ~PermutohedralLatticeHIP() { pl_destroy(handle_); }
    PermutohedralLatticeHIP(const PermutohedralLatticeHIP &) = delete;
    PermutohedralLatticeHIP &operator=(const PermutohedralLatticeHIP &) = delete;

    // values and positions must already be device pointers
    void filter(float *output, const float *input, const float *positions, bool reverse) {
        check(pl_filter(handle_, output, input, positions, reverse ? 1 : 0), "pl_filter");
    }

    // build once, apply many (forward, reverse, further inputs under the same positions)
    void build(const float *positions) { check(pl_build(handle_, positions), "pl_build"); }
    void apply(float *output, const float *input, bool reverse) {
        check(pl_apply(handle_, output, input, reverse ? 1 : 0), "pl_apply");
    }

    // filter / build under the features ComputeKernel would write for this reference image
    // (grid coordinates / spatial_std, reference channels / feature_std), built on the fly
    void filter_image(float *output, const float *input, const float *reference,
                      int n_reference_channels, int n_spatial_dims, const int *spatial_dims,
                      float spatial_std, float feature_std, bool reverse) {
        check(pl_filter_image(handle_, output, input, reference, n_reference_channels,
                              n_spatial_dims, spatial_dims, spatial_std, feature_std,
                              reverse ? 1 : 0),
              "pl_filter_image");
    }
    void build_image(const float *reference, int n_reference_channels, int n_spatial_dims,
                     const int *spatial_dims, float spatial_std, float feature_std) {
        check(pl_build_image(handle_, reference, n_reference_channels, n_spatial_dims,
                             spatial_dims, spatial_std, feature_std),
              "pl_build_image");
    }

    // the N points form a row-major grid of these extents (performance hint only)
    void set_point_grid(int n_dims, const int *dims) {
        check(pl_set_point_grid(handle_, n_dims, dims), "pl_set_point_grid");
    }

    int size() const {
        int m = 0;
        check(pl_num_vertices(handle_, &m), "pl_num_vertices");
        return m;
    }
    pl_handle handle() const { return handle_; }

private:
    pl_handle handle_ = nullptr;
};

template <>
class PermutohedralLatticeHIP<double> {
public:
    PermutohedralLatticeHIP(int pd, int vd, int N, pl_stream stream = nullptr,
                            const pl_alloc *allocator = nullptr) {
        check(pl_create_f64(pd, vd, N, stream, allocator, &handle_), "pl_create_f64");
    }
    ~PermutohedralLatticeHIP() { pl_destroy(handle_); }
    PermutohedralLatticeHIP(const PermutohedralLatticeHIP &) = delete;
    PermutohedralLatticeHIP &operator=(const PermutohedralLatticeHIP &) = delete;

    void filter(double *output, const double *input, const double *positions, bool reverse) {
        check(pl_filter_f64(handle_, output, input, positions, reverse ? 1 : 0), "pl_filter_f64");
    }
    void build(const double *positions) { check(pl_build_f64(handle_, positions), "pl_build_f64"); }
    void apply(double *output, const double *input, bool reverse) {
        check(pl_apply_f64(handle_, output, input, reverse ? 1 : 0), "pl_apply_f64");
    }
    void set_point_grid(int n_dims, const int *dims) {
        check(pl_set_point_grid(handle_, n_dims, dims), "pl_set_point_grid");
    }
    int size() const {
        int m = 0;
        check(pl_num_vertices(handle_, &m), "pl_num_vertices");
        return m;
    }
    pl_handle handle() const { return handle_; }

private:
    pl_handle handle_ = nullptr;
};

template <typename Device, typename T>
struct LatticeFilter;
template <typename Device, typename T>
struct ComputeKernel;

template <>
struct LatticeFilter<HipDevice, float> {
    void operator()(const HipDevice &d, const pl_alloc *allocator, float *output, const float *input,
                    const float *positions, int num_super_pixels, int pd, int vd, bool reverse) {
        PermutohedralLatticeHIP<float> lattice(pd, vd, num_super_pixels, d.stream(), allocator);
        lattice.filter(output, input, positions, reverse);
    }
};

template <>
struct ComputeKernel<HipDevice, float> {
    // spatial_dims is a host array, as in the reference (the CUDA functor copies it itself)
    void operator()(const HipDevice &d, const pl_alloc * /*allocator*/, const float *reference_image,
                    float *positions, int num_super_pixels, int n_spatial_dims, int *spatial_dims,
                    int n_reference_channels, float spatial_std, float features_std) {
        check(pl_compute_positions(reference_image, positions, num_super_pixels, n_reference_channels,
                                   n_spatial_dims, spatial_dims, spatial_std, features_std, d.stream()),
              "pl_compute_positions");
    }
};

template <>
struct LatticeFilter<HipDevice, double> {
    void operator()(const HipDevice &d, const pl_alloc *allocator, double *output,
                    const double *input, const double *positions, int num_super_pixels, int pd,
                    int vd, bool reverse) {
        PermutohedralLatticeHIP<double> lattice(pd, vd, num_super_pixels, d.stream(), allocator);
        lattice.filter(output, input, positions, reverse);
    }
};

template <>
struct ComputeKernel<HipDevice, double> {
    void operator()(const HipDevice &d, const pl_alloc * /*allocator*/,
                    const double *reference_image, double *positions, int num_super_pixels,
                    int n_spatial_dims, int *spatial_dims, int n_reference_channels,
                    double spatial_std, double features_std) {
        check(pl_compute_positions_f64(reference_image, positions, num_super_pixels,
                                       n_reference_channels, n_spatial_dims, spatial_dims,
                                       spatial_std, features_std, d.stream()),
              "pl_compute_positions_f64");
    }
};

// The op on channels-last device tensors [batch, s_1..s_k, C]; attrs as in REGISTER_OP("LatticeFilter").
inline void lattice_filter(const HipDevice &d, const float *input_image, const float *reference_image,
                           float *output, int batch, int n_spatial_dims, const int *spatial_dims,
                           int n_input_channels, int n_reference_channels, bool bilateral = true,
                           float theta_alpha = 1.0f, float theta_beta = 1.0f, float theta_gamma = 1.0f,
                           bool reverse = false, const pl_alloc *allocator = nullptr) {
    check(pl_lattice_filter_op(input_image, reference_image, output, batch, n_spatial_dims,
                               spatial_dims, n_input_channels, n_reference_channels, bilateral ? 1 : 0,
                               theta_alpha, theta_beta, theta_gamma, reverse ? 1 : 0, d.stream(),
                               allocator),
          "pl_lattice_filter_op");
}

inline void lattice_filter(const HipDevice &d, const double *input_image,
                           const double *reference_image, double *output, int batch,
                           int n_spatial_dims, const int *spatial_dims, int n_input_channels,
                           int n_reference_channels, bool bilateral = true, float theta_alpha = 1.0f,
                           float theta_beta = 1.0f, float theta_gamma = 1.0f, bool reverse = false,
                           const pl_alloc *allocator = nullptr) {
    check(pl_lattice_filter_op_f64(input_image, reference_image, output, batch, n_spatial_dims,
                                   spatial_dims, n_input_channels, n_reference_channels,
                                   bilateral ? 1 : 0, theta_alpha, theta_beta, theta_gamma,
                                   reverse ? 1 : 0, d.stream(), allocator),
          "pl_lattice_filter_op_f64");
}

}  // namespace permutohedral

#endif  // PERMUTOHEDRAL_LATTICE_HPP
