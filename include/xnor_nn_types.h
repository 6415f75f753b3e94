/*
 * Public types of the XNOR-Net binary-convolution primitive (MI355X / gfx950 build).
 *
 * Binary-compatible with the descriptor, enums and resource table of mistler/xnor_nn
 * (reference include/xnor_nn_types.h:10-83): a program compiled against the reference
 * header links and runs against this library unchanged.  Enumerator values, field order
 * and field types are therefore fixed; everything else in this file is documentation of
 * what the HIP implementation does with them.
 */
#ifndef XNOR_NN_TYPES_H
#define XNOR_NN_TYPES_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes returned by every entry point and executor
 * (reference include/xnor_nn_types.h:10-15).  HIP runtime failures (allocation,
 * copy, launch) are reported as xnor_nn_error_memory. */
typedef enum {
    xnor_nn_success,              /* 0 */
    xnor_nn_error_memory,         /* 1: device/host allocation or HIP runtime failure */
    xnor_nn_error_invalid_input,  /* 2: a required descriptor or resource slot is null */
    xnor_nn_unimplemented,        /* 3: unknown tensor format / algorithm without GPU path */
} xnor_nn_status_t;

/* Algorithm selector (reference include/xnor_nn_types.h:17-22).  Only the bcast
 * XNOR/popcount pipeline has a GPU implementation; descriptors created with
 * xnor_nn_algorithm_reference get executors that return xnor_nn_unimplemented. */
typedef enum {
    xnor_nn_algorithm_reference = 0,
    xnor_nn_algorithm_bcast = 1,

    xnor_nn_algorithm_best = 1,
} xnor_nn_algorithm_t;

/* Index into xnor_nn_resources_t (reference include/xnor_nn_types.h:24-38).
 *
 *  user_src, user_weights, user_dst  caller-owned tensors, set by the caller before an
 *                                    executor runs.  They may be host pointers (staged
 *                                    through device buffers owned by the descriptor) or
 *                                    device pointers (used in place, no copy, asynchronous
 *                                    on the descriptor's stream).
 *  alpha .. operations_count         library-owned DEVICE buffers created by
 *                                    xnor_nn_allocate_resources(); read them back with
 *                                    the xnor_nn_hip_export_* helpers of xnor_nn_hip.h. */
typedef enum {
    xnor_nn_resource_user_src = 0,
    xnor_nn_resource_user_weights = 1,
    xnor_nn_resource_user_dst = 2,

    xnor_nn_resource_internal = 3, /* first library-owned slot */
    xnor_nn_resource_alpha = 3,            /* float[OC]            mean |w| per filter   */
    xnor_nn_resource_bin_src = 4,          /* packed sign bits of the input              */
    xnor_nn_resource_bin_weights = 5,      /* packed sign bits of the filters            */
    xnor_nn_resource_a = 6,                /* float[MB][IH][IW]    mean |x| over channels */
    xnor_nn_resource_k = 7,                /* float[MB][OH][OW]    box-filtered a         */
    xnor_nn_resource_operations_count = 8, /* int32[OH][OW]        IC * in-bounds taps    */

    xnor_nn_resource_number = 9,
} xnor_nn_resource_type_t;

/* Reference include/xnor_nn_types.h:40-45 (kept for source compatibility). */
typedef enum {
    xnor_nn_operation_convolution_forward = 0,
    xnor_nn_operation_binarize_weights = 1,
    xnor_nn_operation_binarize_data = 2,
    xnor_nn_operation_calculate_k = 3,
} xnor_nn_operation_t;

/* Tensor layouts (reference include/xnor_nn_types.h:47-52). */
typedef enum {
    xnor_nn_data_format_nchw = 0,
    xnor_nn_data_format_nhwc = 1,
    xnor_nn_weights_format_oihw = 2,
    xnor_nn_weights_format_hwio = 3,
} xnor_nn_tensor_format_t;

/* Caller-owned, zero-initialised table of resource pointers
 * (reference include/xnor_nn_types.h:54). */
typedef void *xnor_nn_resources_t[xnor_nn_resource_number];

typedef struct xnor_nn_convolution_ xnor_nn_convolution_t;

/* One pipeline stage (reference include/xnor_nn_types.h:58-59).  Reads and writes only
 * through res[]; self->state carries the launch plan, stream and staging buffers. */
typedef xnor_nn_status_t (*xnor_nn_executor_t)(const xnor_nn_convolution_t *self,
        xnor_nn_resources_t res);

/* Convolution descriptor, allocated by the caller and filled by
 * xnor_nn_init_convolution() (reference include/xnor_nn_types.h:61-83). */
struct xnor_nn_convolution_ {
    xnor_nn_algorithm_t algorithm;

    int mb;
    int ic, ih, iw;
    int oc, oh, ow;
    int sh, sw;
    int kh, kw;
    int ph, pw;

    xnor_nn_tensor_format_t src_format;
    xnor_nn_tensor_format_t weights_format;
    xnor_nn_tensor_format_t dst_format;

    /* byte sizes of the device buffers behind slots 3..8; slots 0..2 are not written */
    size_t resource_size[xnor_nn_resource_number];

    xnor_nn_executor_t binarize_weights; /* once per weight set                      */
    xnor_nn_executor_t binarize_data;    /* stage 1 of forward: sign bits (+ a)      */
    xnor_nn_executor_t calculate_k;      /* stage 2 of forward: a (if stale) and k   */
    xnor_nn_executor_t forward;          /* stage 3 of forward: XNOR/popcount conv   */

    void *state; /* opaque; released by xnor_nn_destroy_convolution() */
};

#ifdef __cplusplus
}
#endif
#endif /* XNOR_NN_TYPES_H */
