/*
 * tsnecuda::RunTsne, the C++ entry point of the pipeline (reference:
 * src/include/fit_tsne.h:33-35, src/fit_tsne.cu:16-627).
 */
#ifndef TSNECUDA_FIT_TSNE_H_
#define TSNECUDA_FIT_TSNE_H_

#include "options.h"

namespace tsnecuda {

// Runs kNN -> perplexity search -> symmetrisation -> opt.iterations gradient
// steps on gpu_opt.device and writes the embedding to opt.return_data.  Sets
// opt.trained and opt.trained_norm.  Invalid options print
// "E: Invalid options file. Terminating." and return without touching the
// result; an unusable initialisation or a GPU error prints a message and calls
// exit(1), as the reference does.
void RunTsne(Options &opt, GpuOptions &gpu_opt);

}  // namespace tsnecuda

#endif  // TSNECUDA_FIT_TSNE_H_
