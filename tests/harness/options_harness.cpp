// Test harness: drives tsnecuda::RunTsne through the C++ Options struct, which
// is the only way to fix Options::random_seed (the Python surface discards its
// random_seed keyword, as the reference's does, src/python/tsnecuda/TSNE.py:58).
//
//   options_harness <num_points> <num_dims> <init: 0 uniform | 1 gaussian> <seed> <iterations> <out.bin>
//
// Runs a fit of <iterations> steps on seeded pseudo-random points and writes the
// returned embedding (2 * num_points floats, xs then ys) to <out.bin>.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "tsnecuda/fit_tsne.h"

int main(int argc, char **argv) {
    if (argc != 7) {
        std::fprintf(stderr, "usage: %s num_points num_dims init seed iterations out.bin\n", argv[0]);
        return 2;
    }
    const int n = std::atoi(argv[1]), d = std::atoi(argv[2]), init = std::atoi(argv[3]);
    const int seed = std::atoi(argv[4]), iterations = std::atoi(argv[5]);
    std::vector<float> points((size_t)n * d), result((size_t)2 * n, -1.0f);
    unsigned int state = 12345u;
    for (auto &v : points) {
        state = state * 1664525u + 1013904223u;
        v = (float)(state >> 8) * (1.0f / 16777216.0f);
    }
    tsnecuda::GpuOptions gpu_opt(0);
    tsnecuda::Options opt(result.data(), points.data(), n, d);
    opt.random_seed = seed;
    opt.initialization = init == 0 ? tsnecuda::TSNE_INIT::UNIFORM : tsnecuda::TSNE_INIT::GAUSSIAN;
    opt.iterations = iterations;
    opt.num_neighbors = n < 32 ? n : 32;
    opt.perplexity = 10.0f;
    opt.verbosity = 0;
    tsnecuda::RunTsne(opt, gpu_opt);
    if (!opt.trained) return 3;
    std::FILE *f = std::fopen(argv[6], "wb");
    if (!f) return 4;
    const size_t written = std::fwrite(result.data(), sizeof(float), result.size(), f);
    std::fclose(f);
    return written == result.size() ? 0 : 5;
}
