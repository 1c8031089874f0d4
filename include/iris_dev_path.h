/*
 * The hot path alone, as a static archive (iris_c_amd/libiris_dev_path.a, `make path`).
 *
 * For a host backend that keeps its own setup, memory entries, stream and other operators -- the reference's
 * backend object (iris_cuda.cu:117-230 for setup and memory, :456-1200 for the other operators) -- and takes
 * only the two hot-path operators from here. The archive defines
 *     iris_dev_head_norm_rope, iris_dev_attention                     (reference iris_dev.h:74-92)
 *     iris_dev_head_norm_rope_qk, iris_dev_head_norm_rope_qk_streams, iris_dev_attention_qnorm,
 *     iris_dev_last_error, iris_dev_last_kernel                       (additions, see iris_dev.h)
 * and the two entries below, and none of the other symbols of iris_dev.h, so it links next to a backend that
 * defines those itself.
 */
#ifndef IRIS_DEV_PATH_H
#define IRIS_DEV_PATH_H

#include "iris_dev.h"

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference. Hands over the hipStream_t (as void *) that the host's other device work
 * runs on; the operators enqueue there, in order with that work. Device 0 must be current. */
void iris_dev_path_attach(void *hip_stream);
/* Waits for that stream and frees the operators' private scratch (only allocated for layouts the matrix-core
 * kernels do not take directly). */
void iris_dev_path_detach(void);

#ifdef __cplusplus
}
#endif
#endif /* IRIS_DEV_PATH_H */
