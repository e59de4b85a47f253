/*
 * extern "C" entry point bound by the Python package through ctypes.
 * Byte-for-byte the signature of the reference's
 * src/include/ext/pymodule_ext.h:10-43 (implementation src/ext/pymodule_ext.cu:6-123).
 */
#ifndef TSNECUDA_PYMODULE_EXT_H_
#define TSNECUDA_PYMODULE_EXT_H_

#include <sys/types.h>
#ifndef __cplusplus
#include <stdbool.h>
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* result: (N, 2) float32 Fortran-ordered host buffer (xs then ys);
 * points: (N, D) float32 C-ordered host buffer; dims = {N, D};
 * initialization_type: 0 uniform, 1 gaussian, 2 resume (rejected), 3 vector
 * (preinit_data: (N, 2) float32 Fortran-ordered); return_style: 0 once,
 * 1 snapshots; distance_metric: 0 inner product, 1 L2 (recorded, not used). */
void pymodule_tsne(float *result, float *points, ssize_t *dims, float perplexity, float learning_rate,
                   float early_exaggeration, float magnitude_factor, int num_neighbors, int iterations,
                   int iterations_no_progress, int force_magnify_iters, float perplexity_search_epsilon,
                   float pre_exaggeration_momentum, float post_exaggeration_momentum, float theta, float epssq,
                   float min_gradient_norm, int initialization_type, float *preinit_data, bool dump_points,
                   char *dump_file, int dump_interval, bool use_interactive, char *viz_server, int viz_timeout,
                   int verbosity, int print_interval, int gpu_device, int return_style, int num_snapshots,
                   int distance_metric);

#ifdef __cplusplus
}
#endif

#endif /* TSNECUDA_PYMODULE_EXT_H_ */
