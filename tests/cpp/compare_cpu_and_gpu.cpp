// C++ driver in the manner of the reference's Tests/test_compare_cpu_and_gpu.cpp: run the bilateral
// filter of an image under itself on the CPU (here: the oracle) and on the GPU (the HIP library,
// through the C++ header and the functors shaped like src/LatticeFilterKernel.h), quantise both to
// 8 bits by truncation as Tests/utils.h:30 does, and count the values that differ.  Unlike the
// reference's driver it fails (exit code 1) when the two disagree beyond the stated bounds.
//
// Scratch comes from a counting allocator passed as pl_alloc, the stand-in for the reference's
// DeviceMemoryAllocator.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "PermutohedralLattice.hpp"
#include "pl_oracle.h"

namespace {

struct CountingAllocator {
    int live = 0, total = 0;
    static void *alloc(void *ctx, size_t bytes) {
        auto *self = static_cast<CountingAllocator *>(ctx);
        void *p = nullptr;
        if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) return nullptr;
        self->live++;
        self->total++;
        return p;
    }
    static void free(void *ctx, void *p) {
        static_cast<CountingAllocator *>(ctx)->live--;
        (void)hipFree(p);
    }
};

#define HIP_OK(call)                                                                  \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess) {                                                       \
            std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));           \
            return 2;                                                                 \
        }                                                                             \
    } while (0)

}  // namespace

int main(int argc, char **argv) {
    const int height = argc > 1 ? std::atoi(argv[1]) : 240;
    const int width = argc > 2 ? std::atoi(argv[2]) : 320;
    const float theta_alpha = 8.0f, theta_beta = 0.125f;
    const int n = height * width, channels = 3, n_sdims = 2;
    int sdims[2] = {height, width};
    const int pd = n_sdims + channels, vd = channels + 1;

    // smooth colour ramps plus a deterministic pseudo-random perturbation
    std::vector<float> image((size_t)n * channels);
    unsigned state = 12345u;
    for (int y = 0; y < height; ++y)
        for (int x = 0; x < width; ++x)
            for (int c = 0; c < channels; ++c) {
                state = state * 1664525u + 1013904223u;
                const float noise = ((state >> 8) & 0xffff) / 65535.0f * 0.1f - 0.05f;
                float v = 0.5f + 0.4f * std::sin(0.02f * (x + 1) * (c + 1)) * std::cos(0.015f * y) + noise;
                image[((size_t)y * width + x) * channels + c] = std::fmin(1.0f, std::fmax(0.0f, v));
            }

    // CPU: feature builder + lattice, as Tests/bilateral_filter_cpu.h does
    std::vector<float> positions((size_t)n * pd), cpu_out((size_t)n * channels);
    plo_compute_positions(image.data(), positions.data(), n, channels, n_sdims, sdims, theta_alpha,
                          theta_beta);
    plo_lattice *cpu = plo_create(pd, vd, n);
    plo_filter(cpu, cpu_out.data(), image.data(), positions.data(), 0);
    const int cpu_vertices = plo_num_vertices(cpu);
    plo_destroy(cpu);

    // GPU: the functors under the op, as Tests/bilateral_filter_gpu.h does with device pointers
    float *d_image = nullptr, *d_positions = nullptr, *d_out = nullptr;
    HIP_OK(hipMalloc(&d_image, sizeof(float) * image.size()));
    HIP_OK(hipMalloc(&d_positions, sizeof(float) * positions.size()));
    HIP_OK(hipMalloc(&d_out, sizeof(float) * cpu_out.size()));
    HIP_OK(hipMemcpy(d_image, image.data(), sizeof(float) * image.size(), hipMemcpyHostToDevice));

    CountingAllocator counting;
    pl_alloc allocator{CountingAllocator::alloc, CountingAllocator::free, &counting};
    std::vector<float> gpu_out(cpu_out.size()), gpu_positions(positions.size());
    int gpu_vertices = 0;
    try {
        permutohedral::HipDevice device;
        permutohedral::ComputeKernel<permutohedral::HipDevice, float>()(
            device, &allocator, d_image, d_positions, n, n_sdims, sdims, channels, theta_alpha, theta_beta);
        permutohedral::LatticeFilter<permutohedral::HipDevice, float>()(
            device, &allocator, d_out, d_image, d_positions, n, pd, vd, false);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(gpu_out.data(), d_out, sizeof(float) * gpu_out.size(), hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(gpu_positions.data(), d_positions, sizeof(float) * positions.size(),
                         hipMemcpyDeviceToHost));
        // the lattice object itself, kept alive to ask for its vertex count, and the op entry point
        permutohedral::PermutohedralLatticeHIP<float> lattice(pd, vd, n, nullptr, &allocator);
        lattice.set_point_grid(n_sdims, sdims);
        lattice.filter(d_out, d_image, d_positions, false);
        gpu_vertices = lattice.size();
        std::vector<float> again(cpu_out.size());
        HIP_OK(hipMemcpy(again.data(), d_out, sizeof(float) * again.size(), hipMemcpyDeviceToHost));
        for (size_t i = 0; i < again.size(); ++i)
            if (std::fabs(again[i] - gpu_out[i]) > 1e-5f) {
                std::fprintf(stderr, "functor and lattice object disagree at %zu\n", i);
                return 1;
            }
        permutohedral::lattice_filter(device, d_image, d_image, d_out, 1, n_sdims, sdims, channels,
                                      channels, true, theta_alpha, theta_beta, 1.0f, false, &allocator);
        HIP_OK(hipDeviceSynchronize());
    } catch (const permutohedral::PermutohedralError &e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 2;
    }

    size_t position_mismatch = 0;
    for (size_t i = 0; i < positions.size(); ++i)
        if (positions[i] != gpu_positions[i]) position_mismatch++;

    size_t differ = 0;
    double max_abs = 0.0;
    for (size_t i = 0; i < cpu_out.size(); ++i) {
        const int a = (int)(cpu_out[i] * 255.0f), b = (int)(gpu_out[i] * 255.0f);
        if (a != b) differ++;
        max_abs = std::fmax(max_abs, std::fabs((double)cpu_out[i] - (double)gpu_out[i]));
    }
    const double percent = 100.0 * (double)differ / (double)cpu_out.size();
    std::printf("%dx%d pd=%d vd=%d: vertices cpu %d gpu %d, positions differing %zu, 8-bit values "
                "differing %zu (%.4f%%), max |cpu-gpu| %.3g, allocations %d (live %d)\n",
                height, width, pd, vd, cpu_vertices, gpu_vertices, position_mismatch, differ, percent,
                max_abs, counting.total, counting.live);
    (void)hipFree(d_image);
    (void)hipFree(d_positions);
    (void)hipFree(d_out);

    // The same in double, as Tests/test_bilateral_gpu.cpp:43-49 runs float and then double: the
    // oracle for T = double against the functors for T = double.
    std::vector<double> image64(image.begin(), image.end());
    std::vector<double> positions64((size_t)n * pd), cpu_out64((size_t)n * channels);
    plo_compute_positions_f64(image64.data(), positions64.data(), n, channels, n_sdims, sdims,
                              theta_alpha, theta_beta);
    plo_lattice_f64 *cpu64 = plo_create_f64(pd, vd, n);
    plo_filter_f64(cpu64, cpu_out64.data(), image64.data(), positions64.data(), 0);
    const int cpu_vertices64 = plo_num_vertices_f64(cpu64);
    plo_destroy_f64(cpu64);
    double *d_image64 = nullptr, *d_positions64 = nullptr, *d_out64 = nullptr;
    HIP_OK(hipMalloc(&d_image64, sizeof(double) * image64.size()));
    HIP_OK(hipMalloc(&d_positions64, sizeof(double) * positions64.size()));
    HIP_OK(hipMalloc(&d_out64, sizeof(double) * cpu_out64.size()));
    HIP_OK(hipMemcpy(d_image64, image64.data(), sizeof(double) * image64.size(), hipMemcpyHostToDevice));
    std::vector<double> gpu_out64(cpu_out64.size()), gpu_positions64(positions64.size());
    int gpu_vertices64 = 0;
    try {
        permutohedral::HipDevice device;
        permutohedral::ComputeKernel<permutohedral::HipDevice, double>()(
            device, &allocator, d_image64, d_positions64, n, n_sdims, sdims, channels, theta_alpha,
            theta_beta);
        permutohedral::PermutohedralLatticeHIP<double> lattice(pd, vd, n, nullptr, &allocator);
        lattice.set_point_grid(n_sdims, sdims);
        lattice.filter(d_out64, d_image64, d_positions64, false);
        gpu_vertices64 = lattice.size();
        permutohedral::LatticeFilter<permutohedral::HipDevice, double>()(
            device, &allocator, d_out64, d_image64, d_positions64, n, pd, vd, false);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(gpu_out64.data(), d_out64, sizeof(double) * gpu_out64.size(), hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(gpu_positions64.data(), d_positions64, sizeof(double) * positions64.size(),
                         hipMemcpyDeviceToHost));
    } catch (const permutohedral::PermutohedralError &e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 2;
    }
    size_t position_mismatch64 = 0;
    for (size_t i = 0; i < positions64.size(); ++i)
        if (positions64[i] != gpu_positions64[i]) position_mismatch64++;
    double max_abs64 = 0.0;
    for (size_t i = 0; i < cpu_out64.size(); ++i)
        max_abs64 = std::fmax(max_abs64, std::fabs(cpu_out64[i] - gpu_out64[i]));
    std::printf("double: vertices cpu %d gpu %d, positions differing %zu, max |cpu-gpu| %.3g, "
                "allocations %d (live %d)\n",
                cpu_vertices64, gpu_vertices64, position_mismatch64, max_abs64, counting.total,
                counting.live);
    (void)hipFree(d_image64);
    (void)hipFree(d_positions64);
    (void)hipFree(d_out64);
    const bool ok64 = cpu_vertices64 == gpu_vertices64 && position_mismatch64 == 0 &&
                      max_abs64 <= 1e-12 && counting.live == 0;
    // the reference reports ~0.2% of 8-bit values differing between its CPU and GPU paths
    // (README.md:87); here the float outputs agree to 1e-3 and the truncated bytes almost always
    const bool ok = cpu_vertices == gpu_vertices && position_mismatch == 0 && max_abs <= 1e-3 &&
                    percent <= 0.2 && counting.live == 0 && counting.total > 0;
    return ok && ok64 ? 0 : 1;
}
