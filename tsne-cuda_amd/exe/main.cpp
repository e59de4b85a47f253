// Command-line front end: the options and data sets of the reference's `tsne`
// executable (src/exe/main.cu:23-40 for the options, :62-213 for the four data
// sets), on top of tsnecuda::RunTsne.  The reference parses with cxxopts; this
// file has a small parser of its own for the same spellings: -l 200,
// --learning-rate 200, --learning-rate=200, and bare -d / --dump for switches.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <random>
#include <string>
#include <vector>

#include "tsnecuda/data_utils.h"
#include "tsnecuda/fit_tsne.h"

namespace {

struct OptionSpec {
    char short_name;
    const char *long_name;
    const char *help;
    const char *default_value;  // nullptr for the help switch
    bool is_switch;
};

// src/exe/main.cu:25-40: same letters, names, help texts and defaults.
const OptionSpec kOptions[] = {
    {'l', "learning-rate", "Learning Rate", "200", false},
    {'p', "perplexity", "Perplexity", "50.0", false},
    {'e', "early-ex", "Early Exaggeration Factor", "12.0", false},
    {'s', "data", "Which program to run on <cifar10,cifar100,mnist,sim>", "sim", false},
    {'k', "num-points", "How many simulated points to use", "5000", false},
    {'u', "nearest-neighbors", "How many nearest neighbors should we use", "32", false},
    {'n', "num-steps", "How many steps to take", "1000", false},
    {'i', "viz", "Use interactive visualization", "false", true},
    {'d', "dump", "Dump the output points", "false", true},
    {'m', "magnitude-factor", "Magnitude factor for KNN", "5.0", false},
    {'t', "init", "What kind of initialization to use <unif,gauss>", "gauss", false},
    {'f', "fname", "File name for loaded data...", "../train-images.idx3-ubyte", false},
    {'c', "connection", "Address for connection to vis server", "tcp://localhost:5556", false},
    {'q', "dim", "Point Dimensions", "50", false},
    {'j', "device", "Device to run on", "0", false},
    {'h', "help", "Print help", nullptr, true},
};

const OptionSpec *find_option(const std::string &token) {
    for (const OptionSpec &o : kOptions) {
        if (token.size() == 2 && token[0] == '-' && token[1] == o.short_name) return &o;
        if (token.size() > 2 && token.compare(0, 2, "--") == 0 && token.compare(2, std::string::npos, o.long_name) == 0)
            return &o;
    }
    return nullptr;
}

void print_help() {
    std::printf("Perform T-SNE in an optimized manner.\nUsage:\n  TSNE-CUDA [OPTION...]\n\n");
    for (const OptionSpec &o : kOptions) {
        std::string left = std::string("  -") + o.short_name + ", --" + o.long_name + (o.is_switch ? "" : " arg");
        std::printf("%-30s %s", left.c_str(), o.help);
        if (o.default_value && !o.is_switch) std::printf(" (default: %s)", o.default_value);
        std::printf("\n");
    }
    std::printf("\nt-SNE for MI355X (gfx950), command line of tsne-cuda 4.0.1\n");
}

bool parse(int argc, char **argv, std::map<std::string, std::string> &values) {
    for (const OptionSpec &o : kOptions)
        if (o.default_value) values[o.long_name] = o.default_value;
    for (int a = 1; a < argc; ++a) {
        std::string token = argv[a], inline_value;
        bool has_inline = false;
        const size_t eq = token.find('=');
        if (token.compare(0, 2, "--") == 0 && eq != std::string::npos) {
            inline_value = token.substr(eq + 1);
            token = token.substr(0, eq);
            has_inline = true;
        }
        const OptionSpec *o = find_option(token);
        if (!o) {
            std::fprintf(stderr, "Option '%s' does not exist\n", argv[a]);
            return false;
        }
        if (o->is_switch) {
            values[o->long_name] = has_inline ? inline_value : "true";
        } else if (has_inline) {
            values[o->long_name] = inline_value;
        } else if (a + 1 < argc) {
            values[o->long_name] = argv[++a];
        } else {
            std::fprintf(stderr, "Option '%s' is missing an argument\n", argv[a]);
            return false;
        }
    }
    return true;
}

bool to_float(const std::string &name, const std::string &text, float &out) {
    char *end = nullptr;
    out = std::strtof(text.c_str(), &end);
    if (end == text.c_str() || *end != '\0') {
        std::fprintf(stderr, "Argument '%s' failed to parse for option '%s'\n", text.c_str(), name.c_str());
        return false;
    }
    return true;
}

bool to_int(const std::string &name, const std::string &text, int &out) {
    char *end = nullptr;
    const long v = std::strtol(text.c_str(), &end, 10);
    if (end == text.c_str() || *end != '\0') {
        std::fprintf(stderr, "Argument '%s' failed to parse for option '%s'\n", text.c_str(), name.c_str());
        return false;
    }
    out = (int)v;
    return true;
}

}  // namespace

int main(int argc, char **argv) {
    std::map<std::string, std::string> v;
    if (!parse(argc, argv, v)) return 1;
    if (v.count("help")) {
        print_help();
        return 0;
    }
    float learning_rate, perplexity, early_ex, magnitude_factor;
    int num_points, neighbors, steps, dim, device;
    if (!to_float("learning-rate", v["learning-rate"], learning_rate) ||
        !to_float("perplexity", v["perplexity"], perplexity) || !to_float("early-ex", v["early-ex"], early_ex) ||
        !to_float("magnitude-factor", v["magnitude-factor"], magnitude_factor) ||
        !to_int("num-points", v["num-points"], num_points) || !to_int("nearest-neighbors", v["nearest-neighbors"], neighbors) ||
        !to_int("num-steps", v["num-steps"], steps) || !to_int("dim", v["dim"], dim) ||
        !to_int("device", v["device"], device))
        return 1;
    const bool dump = v["dump"] == "true", viz = v["viz"] == "true";
    // src/exe/main.cu:55-60: anything but "unif" is the Gaussian start.
    const tsnecuda::TSNE_INIT init =
        v["init"] == "unif" ? tsnecuda::TSNE_INIT::UNIFORM : tsnecuda::TSNE_INIT::GAUSSIAN;
    const std::string data_set = v["data"];

    float *loaded = nullptr;      // delete[] at the end
    std::vector<float> simulated;
    float *points = nullptr;
    int n = 0, d = 0;
    if (data_set == "mnist") {
        int32_t images = 0, rows = 0, columns = 0;
        loaded = tsnecuda::util::LoadMnist(v["fname"], images, rows, columns);
        n = images;
        d = rows * columns;
    } else if (data_set == "cifar10") {
        loaded = tsnecuda::util::LoadCifar10(v["fname"]);
        n = 50000;
        d = 3 * 32 * 32;
    } else if (data_set == "cifar100") {
        loaded = tsnecuda::util::LoadCifar100(v["fname"]);
        n = 50000;
        d = 3 * 32 * 32;
    } else if (data_set == "sim") {
        // src/exe/main.cu:172-186: two clusters, N(-10, 1) for the first half of the values and N(10, 1) for
        // the rest, drawn in order from a default-seeded engine.
        if (num_points <= 0 || dim <= 0) {
            std::fprintf(stderr, "num-points and dim must be positive\n");
            return 1;
        }
        std::default_random_engine generator;
        std::normal_distribution<double> low(-10.0, 1.0), high(10.0, 1.0);
        simulated.resize((size_t)dim * num_points);
        const size_t half = (size_t)(num_points / 2) * dim;
        for (size_t i = 0; i < simulated.size(); ++i) simulated[i] = (float)(i < half ? low(generator) : high(generator));
        points = simulated.data();
        n = num_points;
        d = dim;
    } else {
        std::cout << "Dataset not recognized..." << std::endl;
        return 0;
    }
    if (data_set != "sim") {
        if (!loaded) return 1;
        points = loaded;
    }

    std::printf("Starting TSNE calculation with %u points.\n", (unsigned)n);
    std::fflush(stdout);
    tsnecuda::GpuOptions gpu_opt(device);
    tsnecuda::Options opt(nullptr, points, n, d);
    opt.perplexity = perplexity;
    opt.learning_rate = learning_rate;
    opt.early_exaggeration = early_ex;
    opt.iterations = steps;
    opt.iterations_no_progress = steps;
    opt.magnitude_factor = magnitude_factor;
    opt.initialization = init;
    opt.num_neighbors = neighbors;
    if (dump) opt.enable_dump("dump_ys.txt", 1);
    if (viz) opt.enable_viz(v["connection"]);
    tsnecuda::RunTsne(opt, gpu_opt);
    delete[] loaded;
    return 0;
}
