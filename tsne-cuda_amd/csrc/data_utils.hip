// Dataset readers of the command-line program (host code only).
//
// Same files and the same result as the reference's readers
// (src/util/data_utils.cu:12-159): one image per row, pixel / 255 as fp32.  Every
// file is read with one call per record block instead of one per byte, and a
// short or malformed file is an error instead of a warning.
#include "tsnecuda/data_utils.h"

#include <cstdio>
#include <fstream>
#include <memory>
#include <vector>

namespace {

uint32_t big_endian_u32(const unsigned char *b) {
    return ((uint32_t)b[0] << 24) | ((uint32_t)b[1] << 16) | ((uint32_t)b[2] << 8) | (uint32_t)b[3];
}

void to_unit_range(const unsigned char *bytes, size_t count, float *out) {
    for (size_t i = 0; i < count; ++i) out[i] = static_cast<float>(bytes[i]) / 255.0f;
}

// Records of `skip` label bytes followed by `pixels` pixel bytes; appends `count` images to out.
bool read_records(std::ifstream &file, const std::string &name, size_t count, size_t skip, size_t pixels, float *out) {
    const size_t record = skip + pixels;
    const size_t batch = 1000;  // records per read
    std::vector<unsigned char> buffer(batch * record);
    for (size_t first = 0; first < count; first += batch) {
        const size_t n = count - first < batch ? count - first : batch;
        file.read(reinterpret_cast<char *>(buffer.data()), (std::streamsize)(n * record));
        if ((size_t)file.gcount() != n * record) {
            std::fprintf(stderr, "E: %s ends after %zu of %zu images.\n", name.c_str(),
                         first + (size_t)file.gcount() / record, count);
            return false;
        }
        for (size_t r = 0; r < n; ++r) to_unit_range(buffer.data() + r * record + skip, pixels, out + (first + r) * pixels);
    }
    return true;
}

constexpr size_t kCifarPixels = 3 * 32 * 32;
constexpr size_t kCifarImages = 50000;

}  // namespace

namespace tsnecuda {
namespace util {

float *LoadMnist(std::string file_name, int32_t &num_images, int32_t &num_rows, int32_t &num_columns) {
    num_images = num_rows = num_columns = 0;
    std::ifstream file(file_name, std::ios::in | std::ios::binary);
    unsigned char header[16];
    if (!file || !file.read(reinterpret_cast<char *>(header), sizeof(header))) {
        std::fprintf(stderr, "E: cannot read the header of %s.\n", file_name.c_str());
        return nullptr;
    }
    const uint32_t magic = big_endian_u32(header);
    if (magic != 2051) {
        std::fprintf(stderr, "E: Magic number: %u (an idx3-ubyte image file starts with 2051).\n", magic);
        return nullptr;
    }
    const uint32_t images = big_endian_u32(header + 4), rows = big_endian_u32(header + 8),
                   columns = big_endian_u32(header + 12);
    const uint64_t pixels = (uint64_t)rows * columns;
    if (images == 0 || pixels == 0 || images > 0x7fffffffu || pixels > 0x7fffffffu ||
        (uint64_t)images * pixels > ((uint64_t)1 << 40)) {
        std::fprintf(stderr, "E: implausible header in %s: %u images of %u x %u.\n", file_name.c_str(), images, rows,
                     columns);
        return nullptr;
    }
    std::printf("Num Images: %u\n", images);
    std::fflush(stdout);
    std::unique_ptr<float[]> data(new float[(size_t)images * pixels]);
    if (!read_records(file, file_name, images, 0, (size_t)pixels, data.get())) return nullptr;
    std::printf("Done reading!\n");
    std::fflush(stdout);
    num_images = (int32_t)images;
    num_rows = (int32_t)rows;
    num_columns = (int32_t)columns;
    return data.release();
}

float *LoadCifar10(std::string file_path) {
    std::unique_ptr<float[]> data(new float[kCifarImages * kCifarPixels]);
    const size_t per_batch = kCifarImages / 5;
    for (int batch = 0; batch < 5; ++batch) {
        const std::string name = file_path + "/data_batch_" + std::to_string(batch + 1) + ".bin";
        std::ifstream file(name, std::ios::in | std::ios::binary);
        if (!file) {
            std::fprintf(stderr, "E: cannot open %s.\n", name.c_str());
            return nullptr;
        }
        std::printf("Reading pixels from file %d...\n", batch + 1);
        std::fflush(stdout);
        if (!read_records(file, name, per_batch, 1, kCifarPixels, data.get() + (size_t)batch * per_batch * kCifarPixels))
            return nullptr;
        std::printf("Done reading!\n");
        std::fflush(stdout);
    }
    return data.release();
}

float *LoadCifar100(std::string file_name) {
    std::ifstream file(file_name, std::ios::in | std::ios::binary);
    if (!file) {
        std::fprintf(stderr, "E: cannot open %s.\n", file_name.c_str());
        return nullptr;
    }
    std::unique_ptr<float[]> data(new float[kCifarImages * kCifarPixels]);
    if (!read_records(file, file_name, kCifarImages, 2, kCifarPixels, data.get())) return nullptr;
    std::printf("Done reading!\n");
    std::fflush(stdout);
    return data.release();
}

}  // namespace util
}  // namespace tsnecuda

extern "C" {

float *tsnecuda_load_mnist(const char *file_name, int *dims) {
    if (!file_name || !dims) return nullptr;
    int32_t images = 0, rows = 0, columns = 0;
    float *data = tsnecuda::util::LoadMnist(file_name, images, rows, columns);
    dims[0] = images;
    dims[1] = rows * columns;
    return data;
}

float *tsnecuda_load_cifar10(const char *directory, int *dims) {
    if (!directory || !dims) return nullptr;
    float *data = tsnecuda::util::LoadCifar10(directory);
    dims[0] = data ? (int)kCifarImages : 0;
    dims[1] = data ? (int)kCifarPixels : 0;
    return data;
}

float *tsnecuda_load_cifar100(const char *file_name, int *dims) {
    if (!file_name || !dims) return nullptr;
    float *data = tsnecuda::util::LoadCifar100(file_name);
    dims[0] = data ? (int)kCifarImages : 0;
    dims[1] = data ? (int)kCifarPixels : 0;
    return data;
}

void tsnecuda_free_points(float *points) { delete[] points; }

}  // extern "C"
