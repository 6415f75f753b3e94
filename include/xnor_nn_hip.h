/*
 * Extensions of the MI355X / gfx950 build of xnor_nn.  None of these exist in
 * mistler/xnor_nn; each comment names the reference behaviour it stands in for.
 *
 * Why they exist: in the reference, slots 3..8 of xnor_nn_resources_t are host memory
 * that callers and tests read directly (reference test/gtest/test_binarization.cpp:72-77).
 * Here they are device memory in a GPU-friendly word layout, so reading them goes
 * through the export helpers below, which return the reference's canonical host layout.
 */
#ifndef XNOR_NN_HIP_H
#define XNOR_NN_HIP_H

#include <stddef.h>
#include <stdint.h>

#include "xnor_nn_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* HIP stream (a hipStream_t passed as void*) on which the executors of this descriptor
 * launch; default: the null stream.  With device pointers in slots 0..2 the executors
 * only enqueue work and return; with host pointers they copy synchronously.
 * Stands in for the reference's implicit "runs on the calling thread + OpenMP team".
 * Threads: as in the reference (src/bcast_convolution.hpp:77-93) the executors keep nothing
 * between calls but the launch plan, so several host threads may run one descriptor, each
 * with a resource table of its own; calls on one descriptor are serialised internally (they
 * share its stream and, for host pointers, its staging buffers). */
xnor_nn_status_t xnor_nn_hip_set_stream(const xnor_nn_convolution_t *c, void *stream);

/* Stage fusion, on by default.  The reference's three per-forward stages each make a full
 * pass of their own (reference src/bcast_binarize_data.cpp:43-73,
 * src/bcast_calculate_k.cpp:42-85).  Here binarize_data also leaves mean|x| in res[a], and
 * the calculate_k that follows it immediately on the same res[user_src] and res[a] does not
 * read the input again; with the matrix-core convolution calculate_k also leaves its box
 * filter to forward, which sums K on the fly and stores the K plane.  What is handed over is
 * recorded against the device buffers of the resource table, so calls on other tables do
 * not interfere; any other executor on the table, freeing the table or destroying the
 * descriptor withdraws it.  A caller that changes the contents of user_src between
 * binarize_data and calculate_k, or that reads res[k] as a raw device pointer between
 * calculate_k and forward, switches fusion off (on = 0; the environment variable
 * XNOR_NN_HIP_SEPARATE_K=1, read when a descriptor is initialised, does the same for every
 * descriptor initialised while it is set): every executor then completes its own stage as
 * in the reference.  xnor_nn_hip_export_floats always returns the finished K plane.
 * The records are keyed on the addresses in slots `a` and `k`.  While fusion is on, buffers
 * that have been in those slots must therefore be released through xnor_nn_free_resources
 * (or after xnor_nn_destroy_convolution of every descriptor that used them): a caller that
 * brings its own `a`/`k` buffers and frees them behind the library's back leaves a record
 * that a later call on a recycled address would act on.
 * A box filter that is owed runs on the stream its mean|x| was written on, with the geometry
 * of the descriptor that owes it; when another descriptor's call triggers it (its table
 * names that K plane, or is about to overwrite that mean|x| plane) and that descriptor runs
 * on another stream, the two streams are ordered with events around the filter. */
xnor_nn_status_t xnor_nn_hip_set_stage_fusion(const xnor_nn_convolution_t *c, int on);

/* Block until everything enqueued by this descriptor's executors has finished. */
xnor_nn_status_t xnor_nn_hip_synchronize(const xnor_nn_convolution_t *c);

/* Bytes per packed word of the reference's CPU layout for this shape: 2 while
 * ic*kh*kw < 32767, else 4 (reference src/implementation.cpp:17-22,
 * src/convolution_traits.hpp:29-56).  Only the export helpers depend on it. */
int xnor_nn_hip_canonical_bici(const xnor_nn_convolution_t *c);

/* Copy res[bin_src] to host memory in the reference's layout
 * (reference src/bcast_binarize_data.cpp:43-73):
 *   dst[((mb*IH+ih)*IW+iw)*ABIC + b], bit (7-j) = 1 iff channel 8b+j has its sign bit
 *   clear; channels >= IC and pad bytes are 0; ABIC = ceil(ceil(IC/8)/bici)*bici.
 * dst_bytes must be MB*IH*IW*ABIC. */
xnor_nn_status_t xnor_nn_hip_export_bin_src(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, void *dst, size_t dst_bytes);

/* Copy res[bin_weights] to host memory in the reference's layout for a CPU that packs
 * `oci` filters per block (reference src/bcast_binarize_weights.cpp:54-93; oci = 16 for
 * int16 words / 8 for int32 words on a 256-bit CPU):
 *   dst[((((oco*KH+kh)*KW+kw)*ICO+ico)*oci+i)*bici + b], MSB-first, channels >= IC are 1.
 * oc must be a multiple of oci.  dst_bytes must be (OC/oci)*KH*KW*ICO*oci*bici. */
xnor_nn_status_t xnor_nn_hip_export_bin_weights(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int oci, void *dst, size_t dst_bytes);

/* Copy one of the float resources (xnor_nn_resource_alpha, _a, _k) to host memory,
 * shaped as in the reference (alpha[OC], a[MB][IH][IW], k[MB][OH][OW]). */
xnor_nn_status_t xnor_nn_hip_export_floats(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int slot, float *dst, size_t dst_bytes);

/* Copy res[operations_count] to host memory as int32[OH][OW]
 * (reference src/bcast_binarize_weights.cpp:126-142 stores int16 or int32). */
xnor_nn_status_t xnor_nn_hip_export_operations_count(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int32_t *dst, size_t dst_bytes);

/* Run the convolution stage but store the raw integer accumulators
 * popc[mb][oc][oh][ow] (int32, host or device pointer) instead of the scaled floats:
 * the `d_arr` values of reference src/default/bcast_convolution_default.cpp:64-91.
 * Needs res[bin_src] and res[bin_weights] only (the operation count that turns the
 * matrix-core kernel's 2*popc - n back into popc is derived from the geometry inside the
 * kernel); same kernel as forward, other epilogue. */
xnor_nn_status_t xnor_nn_hip_forward_popcount(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int32_t *popc);

/* Name of the kernel variant an executor of this descriptor launches (stage: one of
 * xnor_nn_operation_t), e.g. "conv_mfma_fp4_kernel<KS=6,PS=4+2>"; the counterpart of the
 * reference's XNOR_NN_VERBOSE line (reference src/utils/convolution_logger.hpp:99-152).
 * Returns the length written (without terminator). */
int xnor_nn_hip_kernel_name(const xnor_nn_convolution_t *c, int stage,
        char *buf, size_t buf_bytes);

/* Kernel durations as the GPU saw them, for benchmarks: with capacity > 0 every launch of
 * the binarize and of the convolution kernel by this descriptor's executors gets a pair of
 * HIP events attached to its own dispatch (hipExtLaunchKernel; no extra packets on the
 * stream), kept in a ring of `capacity` launches per stage; capacity = 0 switches timing
 * off.  xnor_nn_hip_kernel_times waits for the stream, writes the durations (milliseconds,
 * oldest first) of the launches of `stage` (xnor_nn_operation_binarize_data or
 * xnor_nn_operation_convolution_forward) since the last query into ms[0..max) and returns
 * how many it wrote, -1 on error.  The counterpart of the per-stage timers of reference
 * test/perf/test_simple_net.cpp:60-88. */
xnor_nn_status_t xnor_nn_hip_time_kernels(const xnor_nn_convolution_t *c, int capacity);
int xnor_nn_hip_kernel_times(const xnor_nn_convolution_t *c, int stage, float *ms, int max);

/* Compute units and peak engine clock (kHz) of the current HIP device, as the runtime
 * reports them; the figures the VALU roofline of the convolution kernel is priced with.
 * The reference's counterpart is its CPUID probe (reference src/utils/cpuid.hpp:119-168). */
xnor_nn_status_t xnor_nn_hip_device_info(int *compute_units, int *clock_khz);

/* Calibration for benchmarks, no counterpart in the reference: enqueues on `stream` (a
 * hipStream_t) one kernel that reads `bytes` (rounded down to 16) of device memory once, 16
 * bytes per lane and load, and keeps nothing.  Its duration beside the binarize kernel's on
 * the same bytes shows what the memory system, not the kernel, costs: the stages of this
 * library that stream the input are priced against the HBM peak, which no reader reaches. */
xnor_nn_status_t xnor_nn_hip_plain_read(const void *device_buffer, size_t bytes, void *stream);

/* Calibration for benchmarks, no counterpart in the reference: enqueues one kernel of
 * `workgroups` workgroups of four waves in which every wave issues 8 * iterations of the
 * convolution kernel's matrix instruction (FP4 32x32x64 = 131072 operations each) on
 * pseudo-random +-1 operands that stay in registers.  Its rate is what the matrix pipes
 * deliver on such data with no operand traffic at all, under the chip's own clock management:
 * the practical ceiling beside the published peak the convolution is priced against. */
#define XNOR_NN_HIP_MFMA_ONLY_OPS_PER_WAVE_ITERATION (8 * 131072LL)
xnor_nn_status_t xnor_nn_hip_mfma_only(int workgroups, int iterations, void *stream);

/* xnor_nn_binarize_weights_float (reference src/binarize_weights_float.cpp:3-25) for callers
 * that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  `from` and `to`
 * must both be device pointers to OC*IC*KH*KW floats; the call enqueues two kernels on the
 * descriptor's stream and returns (no allocation, no free, no memset, no synchronisation),
 * and writes the same bits as xnor_nn_binarize_weights_float.  The 256 partial sums live in
 * a 1 KB device array that is part of the library and stays on every GPU the library has
 * run on until the process ends (its device address is looked up once per GPU, by
 * xnor_nn_init_convolution or by the first call here, whichever comes first).  Every call on a GPU shares that array: calls that overlap
 * on one GPU (two streams, two threads) race on it and must be ordered by the caller.
 * More than XNOR_NN_HIP_NOALLOC_MAX_WEIGHTS weights, a null pointer, or a pointer to host
 * memory (the kernels would fault on it) is refused with xnor_nn_error_invalid_input and a
 * line on stderr; nothing is launched then. */
#define XNOR_NN_HIP_NOALLOC_MAX_WEIGHTS 2147483647LL /* the reference counts them in an int */
xnor_nn_status_t xnor_nn_hip_binarize_weights_float_noalloc(const xnor_nn_convolution_t *c,
        const float *from, float *to);

#ifdef __cplusplus
}
#endif
#endif /* XNOR_NN_HIP_H */
