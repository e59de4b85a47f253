/* Dataset readers used by the command-line program: the files the reference's
 * `tsne` executable reads (src/include/util/data_utils.h:30-60, implemented in
 * src/util/data_utils.cu:12-159).  Pixels become fp32 in [0, 1] (value / 255),
 * one image per row, in file order.  The returned arrays are allocated with
 * new[] and belong to the caller (delete[]), as in the reference.
 *
 * Unlike the reference, which prints "E: ..." and carries on with whatever it
 * read, a file that cannot be opened, has the wrong magic number or ends early
 * makes these functions return nullptr (the C wrappers: NULL) after printing
 * the reason to stderr. */
#ifndef TSNECUDA_DATA_UTILS_H_
#define TSNECUDA_DATA_UTILS_H_

#ifdef __cplusplus
#include <cstdint>
#include <string>

namespace tsnecuda {
namespace util {

/* MNIST image file (idx3-ubyte: big-endian magic 2051, image count, rows,
 * columns, then one byte per pixel).  src/util/data_utils.cu:12-79. */
float *LoadMnist(std::string file_name, int32_t &num_images, int32_t &num_rows, int32_t &num_columns);

/* CIFAR-10 binary version: directory holding data_batch_1.bin ... data_batch_5.bin,
 * 10000 records of 1 label byte + 3072 pixel bytes each; returns 50000 x 3072.
 * src/util/data_utils.cu:81-126. */
float *LoadCifar10(std::string file_path);

/* CIFAR-100 binary version: one file (train.bin) of 50000 records of 2 label
 * bytes + 3072 pixel bytes; returns 50000 x 3072.  src/util/data_utils.cu:128-159. */
float *LoadCifar100(std::string file_name);

}  // namespace util
}  // namespace tsnecuda

extern "C" {
#endif

/* C wrappers of the three readers for callers without C++ (ctypes); dims
 * receives {images, values per image}.  Free the result with
 * tsnecuda_free_points. */
float *tsnecuda_load_mnist(const char *file_name, int *dims);
float *tsnecuda_load_cifar10(const char *directory, int *dims);
float *tsnecuda_load_cifar100(const char *file_name, int *dims);
void tsnecuda_free_points(float *points);

#ifdef __cplusplus
}
#endif

#endif /* TSNECUDA_DATA_UTILS_H_ */
