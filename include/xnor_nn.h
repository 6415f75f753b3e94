/*
 * C entry points of the XNOR-Net binary-convolution primitive (MI355X / gfx950 build).
 *
 * Same six symbols, signatures and call protocol as mistler/xnor_nn
 * (reference include/xnor_nn.h:12-29); implemented by libxnor_nn.so with hand-written
 * HIP kernels.  Call protocol (reference example/simple_convolution.c:34-66):
 *
 *     xnor_nn_resources_t res = {0};
 *     xnor_nn_convolution_t c;
 *     xnor_nn_init_convolution(&c, xnor_nn_algorithm_bcast, ...);
 *     xnor_nn_allocate_resources(&c, res);
 *     res[xnor_nn_resource_user_weights] = w;  c.binarize_weights(&c, res);
 *     res[xnor_nn_resource_user_src] = x;  res[xnor_nn_resource_user_dst] = y;
 *     c.binarize_data(&c, res);  c.calculate_k(&c, res);  c.forward(&c, res);
 *     xnor_nn_free_resources(res);  xnor_nn_destroy_convolution(&c);
 */
#ifndef XNOR_NN_H
#define XNOR_NN_H

#include <stddef.h>

#include "xnor_nn_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces reference src/status.cpp:3-15.  Copies "success", "memory_error",
 * "bad_input" or "unimplemented" (with terminator) into msg; callers pass char[16]. */
void xnor_nn_get_status_message(char *msg, xnor_nn_status_t status);

/* Replaces reference src/memory.cpp:23-33.  Allocates DEVICE memory for slots 3..8
 * from c->resource_size[]; on failure releases what it got, leaves the slots null and
 * returns xnor_nn_error_memory. */
xnor_nn_status_t xnor_nn_allocate_resources(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res);

/* Replaces reference src/memory.cpp:35-39.  Frees slots 3..8 and nulls them;
 * safe on a zeroed table and when called twice. */
void xnor_nn_free_resources(xnor_nn_resources_t res);

/* Replaces reference src/binarize_weights_float.cpp:3-25 (training-side helper):
 * to[i] = (from[i] >= 0 ? 1 : -1) * mean(from).  Host or device pointers. */
void xnor_nn_binarize_weights_float(const xnor_nn_convolution_t *c,
        const float *from, float *to);

/* Replaces reference src/common_convolution.cpp:9-63.  Fills every field of *c,
 * computes oh/ow, builds the launch plan and installs the four executors.
 * Always returns xnor_nn_success, like the reference. */
xnor_nn_status_t xnor_nn_init_convolution(xnor_nn_convolution_t *c,
        const xnor_nn_algorithm_t algorithm,
        const xnor_nn_tensor_format_t src_fmt,
        const xnor_nn_tensor_format_t weights_fmt,
        const xnor_nn_tensor_format_t dst_fmt,
        int mb, int oc, int ic, int ih, int iw,
        int kh, int kw, int sh, int sw, int ph, int pw);

/* Replaces reference src/common_convolution.cpp:65-67.  Releases c->state
 * (plan, staging buffers) and nulls it. */
void xnor_nn_destroy_convolution(xnor_nn_convolution_t *c);

#ifdef __cplusplus
}
#endif
#endif /* XNOR_NN_H */
