// Command-line bilateral filter of a BMP image on the GPU:
//
//     bilateral_filter_hip <image file> <output file> <spatial standard deviation>
//                          <color standard deviation> [image to filter]
//
// The counterpart of the reference's Tests/test_bilateral_gpu.cpp (README.md:51-59 there): the image
// is its own guide, pixels are scaled by 1/255 (Tests/utils.h:9-23), filtered with pd = 5, vd = 4,
// and written back as int(value * 255) clamped to 0..255 (Tests/utils.h:26-40).  With a fifth
// argument that image is filtered under the first one as guide (Tests/greyscale_test.py).
// Like the reference's program (Tests/test_bilateral_gpu.cpp:43-49) it then repeats the filter in
// double precision and reports the time; the file written holds the float result.
// Reads uncompressed 24-bit and 8-bit (palette) BMP files, writes 24-bit ones.
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <stdexcept>
#include <string>
#include <vector>

#include <hip/hip_runtime.h>

#include "PermutohedralLattice.hpp"

namespace {

struct Image {
    int width = 0, height = 0;
    std::vector<unsigned char> rgb;  // [y][x][channel], top row first
};

uint32_t le32(const unsigned char *p) { return p[0] | (p[1] << 8) | (p[2] << 16) | ((uint32_t)p[3] << 24); }
uint16_t le16(const unsigned char *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

Image read_bmp(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("cannot open " + path);
    std::vector<unsigned char> b((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (b.size() < 54 || b[0] != 'B' || b[1] != 'M') throw std::runtime_error(path + ": not a BMP file");
    const uint32_t data_offset = le32(&b[10]), header_size = le32(&b[14]);
    const int32_t w = (int32_t)le32(&b[18]), h_signed = (int32_t)le32(&b[22]);
    const int bpp = le16(&b[28]);
    const uint32_t compression = le32(&b[30]);
    if (header_size < 40 || w <= 0 || h_signed == 0) throw std::runtime_error(path + ": unsupported BMP header");
    if ((bpp != 24 && bpp != 8) || (compression != 0 && !(compression == 3 && bpp == 24)))
        throw std::runtime_error(path + ": only uncompressed 24-bit and 8-bit BMP files are read");
    const bool bottom_up = h_signed > 0;
    const int h = bottom_up ? h_signed : -h_signed;
    const size_t stride = ((size_t)w * bpp / 8 + 3) & ~(size_t)3;
    if (data_offset + stride * h > b.size()) throw std::runtime_error(path + ": truncated BMP file");
    const unsigned char *palette = &b[14 + header_size];
    uint32_t colours = le32(&b[46]);
    if (bpp == 8) {
        if (colours == 0) colours = 256;
        if (14 + header_size + 4 * (size_t)colours > b.size()) throw std::runtime_error(path + ": bad palette");
    }
    Image im;
    im.width = w;
    im.height = h;
    im.rgb.resize((size_t)w * h * 3);
    for (int y = 0; y < h; ++y) {
        const unsigned char *row = &b[data_offset + stride * (size_t)(bottom_up ? h - 1 - y : y)];
        unsigned char *out = &im.rgb[(size_t)y * w * 3];
        for (int x = 0; x < w; ++x) {
            if (bpp == 24) {  // stored blue, green, red
                out[3 * x + 0] = row[3 * x + 2];
                out[3 * x + 1] = row[3 * x + 1];
                out[3 * x + 2] = row[3 * x + 0];
            } else {
                const unsigned idx = row[x] < colours ? row[x] : 0;
                out[3 * x + 0] = palette[4 * idx + 2];
                out[3 * x + 1] = palette[4 * idx + 1];
                out[3 * x + 2] = palette[4 * idx + 0];
            }
        }
    }
    return im;
}

void put32(std::vector<unsigned char> &b, size_t at, uint32_t v) {
    for (int i = 0; i < 4; ++i) b[at + i] = (unsigned char)(v >> (8 * i));
}

void write_bmp(const std::string &path, const Image &im) {
    const size_t stride = ((size_t)im.width * 3 + 3) & ~(size_t)3;
    std::vector<unsigned char> b(54 + stride * im.height, 0);
    b[0] = 'B';
    b[1] = 'M';
    put32(b, 2, (uint32_t)b.size());
    put32(b, 10, 54);
    put32(b, 14, 40);
    put32(b, 18, (uint32_t)im.width);
    put32(b, 22, (uint32_t)im.height);  // bottom-up
    b[26] = 1;
    b[28] = 24;
    put32(b, 34, (uint32_t)(stride * im.height));
    put32(b, 38, 2835);
    put32(b, 42, 2835);
    for (int y = 0; y < im.height; ++y) {
        unsigned char *row = &b[54 + stride * (size_t)(im.height - 1 - y)];
        const unsigned char *in = &im.rgb[(size_t)y * im.width * 3];
        for (int x = 0; x < im.width; ++x) {
            row[3 * x + 0] = in[3 * x + 2];
            row[3 * x + 1] = in[3 * x + 1];
            row[3 * x + 2] = in[3 * x + 0];
        }
    }
    std::ofstream f(path, std::ios::binary);
    if (!f.write((const char *)b.data(), (std::streamsize)b.size())) throw std::runtime_error("cannot write " + path);
}

void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

template <typename T = float>
struct DeviceBuffer {
    T *p = nullptr;
    explicit DeviceBuffer(size_t n) { hip_check(hipMalloc((void **)&p, n * sizeof(T)), "hipMalloc"); }
    ~DeviceBuffer() { (void)hipFree(p); }
};

std::vector<float> to_unit_floats(const Image &im) {
    std::vector<float> flat(im.rgb.size());
    for (size_t i = 0; i < flat.size(); ++i) flat[i] = im.rgb[i] / 255.0f;
    return flat;
}

}  // namespace

int main(int argc, char **argv) {
    if (argc < 5) {
        std::printf("Usage: %s <image file> <output file> <spatial standard deviation> "
                    "<color standard deviation> [image to filter]\n", argv[0]);
        return 1;
    }
    try {
        const Image guide = read_bmp(argv[1]);
        const Image source = argc > 5 ? read_bmp(argv[5]) : guide;
        if (source.width != guide.width || source.height != guide.height)
            throw std::runtime_error("the image to filter and the guide differ in size");
        const float theta_alpha = (float)std::atof(argv[3]), theta_beta = (float)std::atof(argv[4]);
        const int n = guide.width * guide.height;
        const int sdims[2] = {guide.height, guide.width};
        const std::vector<float> guide_flat = to_unit_floats(guide), flat = to_unit_floats(source);
        std::vector<float> filtered(flat.size());

        DeviceBuffer<> d_guide(flat.size()), d_in(flat.size()), d_out(flat.size());
        hip_check(hipMemcpy(d_guide.p, guide_flat.data(), flat.size() * sizeof(float), hipMemcpyHostToDevice), "copy in");
        hip_check(hipMemcpy(d_in.p, flat.data(), flat.size() * sizeof(float), hipMemcpyHostToDevice), "copy in");

        permutohedral::PermutohedralLatticeHIP<float> lattice(5, 4, n);
        const auto begin = std::chrono::steady_clock::now();
        lattice.filter_image(d_out.p, d_in.p, d_guide.p, 3, 2, sdims, theta_alpha, theta_beta, false);
        hip_check(hipDeviceSynchronize(), "filter");
        const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - begin).count();
        std::printf("Measured from function call: %f seconds (%d x %d, %d lattice vertices)\n", seconds,
                    guide.width, guide.height, lattice.size());
        hip_check(hipMemcpy(filtered.data(), d_out.p, flat.size() * sizeof(float), hipMemcpyDeviceToHost), "copy out");

        {
            std::printf("Testing for double precision\n");
            const std::vector<double> guide64(guide_flat.begin(), guide_flat.end());
            const std::vector<double> flat64(flat.begin(), flat.end());
            std::vector<double> filtered64(flat.size());
            DeviceBuffer<double> d_guide64(flat.size()), d_in64(flat.size()), d_out64(flat.size());
            DeviceBuffer<double> d_positions64((size_t)n * 5);
            hip_check(hipMemcpy(d_guide64.p, guide64.data(), flat.size() * sizeof(double), hipMemcpyHostToDevice), "copy in");
            hip_check(hipMemcpy(d_in64.p, flat64.data(), flat.size() * sizeof(double), hipMemcpyHostToDevice), "copy in");
            permutohedral::PermutohedralLatticeHIP<double> lattice64(5, 4, n);
            lattice64.set_point_grid(2, sdims);
            int dims[2] = {sdims[0], sdims[1]};
            const auto begin64 = std::chrono::steady_clock::now();
            permutohedral::ComputeKernel<permutohedral::HipDevice, double>()(
                permutohedral::HipDevice{}, nullptr, d_guide64.p, d_positions64.p, n, 2, dims, 3,
                (double)theta_alpha, (double)theta_beta);
            lattice64.filter(d_out64.p, d_in64.p, d_positions64.p, false);
            hip_check(hipDeviceSynchronize(), "filter");
            const double seconds64 =
                std::chrono::duration<double>(std::chrono::steady_clock::now() - begin64).count();
            hip_check(hipMemcpy(filtered64.data(), d_out64.p, flat.size() * sizeof(double), hipMemcpyDeviceToHost), "copy out");
            double max_diff = 0.0;
            for (size_t i = 0; i < filtered.size(); ++i) {
                const double diff = filtered64[i] - (double)filtered[i];
                max_diff = diff > max_diff ? diff : (-diff > max_diff ? -diff : max_diff);
            }
            std::printf("Measured from function call: %f seconds (%d lattice vertices, "
                        "max |double - float| %.3g)\n", seconds64, lattice64.size(), max_diff);
        }

        Image out = source;
        for (size_t i = 0; i < filtered.size(); ++i) {
            int value = (int)(filtered[i] * 255.0f);
            out.rgb[i] = (unsigned char)(value > 255 ? 255 : (value < 0 ? 0 : value));
        }
        write_bmp(argv[2], out);
    } catch (const std::exception &e) {
        std::fprintf(stderr, "%s: %s\n", argv[0], e.what());
        return 2;
    }
    return 0;
}
