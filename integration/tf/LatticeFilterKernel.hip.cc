// The GPU half of the reference's TensorFlow op on a ROCm build of TensorFlow: the two device
// functors of src/LatticeFilterKernel.h:28-54, which the reference specialises for
// Eigen::GpuDevice in src/LatticeFilterKernel.cu:44-101, specialised here on top of the C ABI of
// libpermutohedral_hip.so.  This file takes the place of LatticeFilterKernel.cu in the op's
// build (compile as device-independent C++ and link with -lpermutohedral_hip); the op itself,
// LatticeFilterOp::Compute (src/LatticeFilterKernel.cpp:98-181), its registration
// (src/LatticeFilterKernel.cpp:30-43, 194-209) and the Python loader with the gradient rule
// (lattice_filter_op_loader.py:32-54) stay as they are.  (pd, vd) are run-time arguments: the
// -DSPATIAL_DIMS/-DINPUT_CHANNELS/-DREFERENCE_CHANNELS defines of LatticeFilterKernel.cu:30-38,
// 87-100 are not needed.
//
// It needs TensorFlow's headers, which are not part of this repository; the same functor shapes
// without TensorFlow are in include/PermutohedralLattice.hpp and are compiled and tested here
// (tests/cpp/compare_cpu_and_gpu.cpp).
#define EIGEN_USE_GPU
#include <vector>

#include "LatticeFilterKernel.h"      // the reference's functor declarations
#include "permutohedral_lattice.h"    // this library's C ABI
#include "tensorflow/core/framework/op_kernel.h"

using namespace tensorflow;
using GPUDevice = Eigen::GpuDevice;

namespace {

// Scratch memory from TensorFlow temporaries, as the reference's DeviceMemoryAllocator takes it
// (src/DeviceMemoryAllocator.h:52-71).  The temporaries live until the functor returns.
struct TfScratch {
  OpKernelContext* ctx;
  std::vector<Tensor> held;
  static void* alloc(void* self, size_t bytes) {
    auto* s = static_cast<TfScratch*>(self);
    Tensor t;
    if (!s->ctx->allocate_temp(DT_UINT8, TensorShape({static_cast<int64>(bytes)}), &t).ok())
      return nullptr;
    s->held.push_back(t);
    return t.flat<uint8>().data();
  }
  static void free(void*, void*) {}
};

}  // namespace

template <>
void ComputeKernel<GPUDevice, float>::operator()(const GPUDevice& d, OpKernelContext* context,
                                                 const float* reference_image, float* positions,
                                                 int num_super_pixels, int n_spatial_dims,
                                                 int* spatial_dims /* host memory */,
                                                 int n_reference_channels, float spatial_std,
                                                 float features_std) {
  const int rc = pl_compute_positions(reference_image, positions, num_super_pixels,
                                      n_reference_channels, n_spatial_dims, spatial_dims,
                                      spatial_std, features_std, d.stream());
  OP_REQUIRES(context, rc == PL_OK, errors::Internal("lattice features: ", pl_strerror(rc)));
}

template <>
void ComputeKernel<GPUDevice, double>::operator()(const GPUDevice& d, OpKernelContext* context,
                                                  const double* reference_image, double* positions,
                                                  int num_super_pixels, int n_spatial_dims,
                                                  int* spatial_dims /* host memory */,
                                                  int n_reference_channels, double spatial_std,
                                                  double features_std) {
  const int rc = pl_compute_positions_f64(reference_image, positions, num_super_pixels,
                                          n_reference_channels, n_spatial_dims, spatial_dims,
                                          spatial_std, features_std, d.stream());
  OP_REQUIRES(context, rc == PL_OK, errors::Internal("lattice features: ", pl_strerror(rc)));
}

template <>
void LatticeFilter<GPUDevice, float>::operator()(const GPUDevice& d, OpKernelContext* context,
                                                 float* output, const float* input,
                                                 const float* positions, int num_super_pixels,
                                                 int pd, int vd, bool reverse) {
  TfScratch scratch{context, {}};
  pl_alloc alloc{TfScratch::alloc, TfScratch::free, &scratch};
  pl_handle lattice = nullptr;
  int rc = pl_create(pd, vd, num_super_pixels, d.stream(), &alloc, &lattice);
  if (rc == PL_OK) rc = pl_filter(lattice, output, input, positions, reverse ? 1 : 0);
  pl_destroy(lattice);   // waits for the stream; the scratch goes back when `scratch` does
  OP_REQUIRES(context, rc == PL_OK, errors::Internal("lattice filter: ", pl_strerror(rc)));
}

template <>
void LatticeFilter<GPUDevice, double>::operator()(const GPUDevice& d, OpKernelContext* context,
                                                  double* output, const double* input,
                                                  const double* positions, int num_super_pixels,
                                                  int pd, int vd, bool reverse) {
  TfScratch scratch{context, {}};
  pl_alloc alloc{TfScratch::alloc, TfScratch::free, &scratch};
  pl_handle lattice = nullptr;
  int rc = pl_create_f64(pd, vd, num_super_pixels, d.stream(), &alloc, &lattice);
  if (rc == PL_OK) rc = pl_filter_f64(lattice, output, input, positions, reverse ? 1 : 0);
  pl_destroy(lattice);
  OP_REQUIRES(context, rc == PL_OK, errors::Internal("lattice filter: ", pl_strerror(rc)));
}

template struct ComputeKernel<GPUDevice, float>;
template struct ComputeKernel<GPUDevice, double>;
template struct LatticeFilter<GPUDevice, float>;
template struct LatticeFilter<GPUDevice, double>;
