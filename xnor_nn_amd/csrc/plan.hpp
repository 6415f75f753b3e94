// Launch plan and per-descriptor state of the gfx950 implementation.
//
// Takes the place of the reference's Implementation object behind c->state
// (reference src/implementation.hpp:11-27, src/bcast_convolution.cpp:58-117): instead of
// CPU blocking factors (BIC/ABIC/ICO/OCI/OCO) it records the device word layout, the
// launch geometry, the stream and the staging buffers used when the caller hands over
// host pointers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <mutex>
#include <vector>

#include "xnor_nn.h"

// Byte offset that the kernels give a buffer access they want the hardware to drop (a channel
// past the end, a dead pixel): it has to lie outside every buffer it is used with, so the
// kernels that use it take buffers below this size only.
#define XNOR_HIP_DROPPED_OFFSET 0xFFFFFFF0ull

namespace xnor_hip {

// n / d for 32-bit n by multiply-high and shifts; d is fixed on the host.
struct FastDiv {
    uint32_t mul, sh1, sh2, d;
    __host__ static FastDiv make(uint32_t d) {
        FastDiv f{0u, 0u, 0u, d};
        if (d <= 1) return f;
        uint32_t L = 0;
        while ((1ull << L) < d) L++;
        f.mul = (uint32_t)(((1ull << 32) * ((1ull << L) - d)) / d + 1);
        f.sh1 = 1;
        f.sh2 = L - 1;
        return f;
    }
    __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        const uint32_t t = __umulhi(n, mul);
#else
        const uint32_t t = (uint32_t)(((uint64_t)n * mul) >> 32);
#endif
        return (t + ((n - t) >> sh1)) >> sh2;
    }
};

// Geometry shared by all kernels.  Device layouts:
//   bin_src      uint32 [MB*IH*IW][XW]          word j, bit (31-b) = channel 32j+b has its
//                                               sign bit clear; channels >= IC are 0
//   bin_weights  uint32 [OCB][KH*KW][XW][Q]     same bit order; channels >= IC and
//                                               filters >= OC are all ones; followed (at
//                                               wfrag_offset) by the same signs as FP4
//                                               matrix-core fragments when use_mfma is set
//   alpha        float  [OC]
//   a            float  [MB*IH*IW]
//   k            float  [MB*OH*OW]
//   op count     int32  [OH*OW]
struct Geometry {
    int mb, ic, ih, iw, oc, oh, ow, kh, kw, sh, sw, ph, pw;
    int src_fmt, w_fmt, dst_fmt;
    int xw;       // 32-bit words per pixel = ceil(ic/32)
    int q;        // filters per wave in the convolution kernel
    int ocb;      // ceil(oc/q)
    int ihw, ohw; // ih*iw, oh*ow
    uint32_t npix_in, npix_out; // mb*ihw, mb*ohw
    int cus;                    // compute units of the device (256 if it cannot be asked)
    int use_mfma;               // 1: stage 3 runs the FP4 matrix-core kernel
    int mfma_ps;                // its tile size in 32-pixel blocks (1..4)
    int mfma_ps_small;          // > 0: a launch with two tile sizes; the later workgroups of an
                                // XCD take this many blocks (see the kernel)
    int mfma_groups;            // pixel groups per tile (1, 2, 4): with 128 / 64 filters or fewer
                                // the waves without filters take further pixel blocks instead
    uint32_t mfma_big_per_xcd;  // ... after this many workgroups with mfma_ps blocks,
    uint32_t mfma_blocks_per_xcd; // out of this many pixel blocks per XCD
    int mfma_persist;           // 1: two workgroups per CU stay and walk over the tiles, taking
    uint32_t mfma_tiles_per_round; // every mfma_tiles_per_round-th tile of their XCD
    uint32_t mfma_rounds;       // rounds of tiles a persistent workgroup walks at most
    int mfma_reverse;           // 1: the second workgroup of a CU walks its tiles last to first
    uint32_t mfma_stagger;      // ... and starts this many sleep periods late
    size_t wfrag_offset;        // byte offset of the FP4 weight fragments in bin_weights
    // the matrix-core kernel's variant and sizes, fixed once by mfma_plan: steps per tap (or
    // per pair of taps), tap pairing, channel parts, input pixels a tile stages at most, LDS
    // bytes per workgroup, bytes of the weight fragments
    int mfma_steps, mfma_pair, mfma_parts, mfma_rows;
    int mfma_small;             // 1: few tiles: the small-problem kernel (kernels_conv_small.hip),
    int mfma_small_rows;        // the input pixels one of its blocks stages at most
    uint32_t mfma_small_lds;    // and its LDS bytes per workgroup
    int stream_dst;             // 1: the matrix-core kernel stores its output with the nt bit
    uint32_t mfma_lds, mfma_wbytes;
    FastDiv div_ihw, div_iw, div_ohw, div_ow;
};

// First and last input pixel (flattened index) that a tile of the output pixels
// [p_first, p_end) can touch with an in-bounds tap: from the start of the first input row of
// its first pixel to the end of the last input row of its last pixel (with a stride above 1
// the span also holds the input pixels the stride skips).
__host__ __device__ inline void tile_span(const Geometry &g, uint32_t p_first, uint32_t p_end,
        int &lo, int &hi) {
    const uint32_t p_last = p_end - 1;
    const uint32_t i0 = g.div_ohw.div(p_first), i1 = g.div_ohw.div(p_last);
    const int oh0 = (int)g.div_ow.div(p_first - i0 * g.ohw);
    const int oh1 = (int)g.div_ow.div(p_last - i1 * g.ohw);
    int r0 = oh0 * g.sh - g.ph, r1 = oh1 * g.sh - g.ph + g.kh - 1;
    if (r0 < 0) r0 = 0;
    if (r0 > g.ih - 1) r0 = g.ih - 1;
    if (r1 > g.ih - 1) r1 = g.ih - 1;
    if (r1 < 0) r1 = 0;
    lo = (int)(i0 * g.ihw) + r0 * g.iw;
    hi = (int)(i1 * g.ihw) + r1 * g.iw + g.iw - 1;
    if (hi < lo) hi = lo;
}

// Optional timing of one launch: when both events are set the kernel is launched with them
// attached to its own dispatch, and their difference is the kernel's duration on the GPU (no
// marker packets on the stream, which would cost more than a short kernel takes).
struct KernelEvents {
    hipEvent_t start = nullptr, stop = nullptr;
};

template <class K, class... A>
inline void launch_kernel(K kernel, dim3 grid, dim3 block, size_t lds, hipStream_t s,
        const KernelEvents &ev, A... args) {
    if (ev.start != nullptr && ev.stop != nullptr)
        hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, s, ev.start, ev.stop, 0,
                args...);
    else
        hipLaunchKernelGGL(kernel, grid, block, lds, s, args...);
}

// Event pairs for xnor_nn_hip_time_kernels: one ring per timed stage.
struct KernelTimer {
    std::vector<KernelEvents> ring;
    size_t launches = 0; // since timing was switched on
    KernelEvents next() {
        if (ring.empty()) return KernelEvents{};
        return ring[launches++ % ring.size()];
    }
};

struct State {
    Geometry g;
    hipStream_t stream = nullptr;
    // Held for the length of every executor call: two host threads may share one descriptor
    // (each with a resource table of its own), and the staging buffers below, the stream and
    // the order in which a call's launches and copies are enqueued belong to one call at a
    // time.
    std::mutex mu;
    // staging buffers for host-side user tensors (allocated on first use)
    void *stage_src = nullptr, *stage_weights = nullptr, *stage_dst = nullptr;
    // partial sums of xnor_nn_binarize_weights_float (allocated on first use)
    float *float_parts = nullptr;
    // Stage fusion (xnor_nn_hip_set_stage_fusion): binarize_data hands mean|x| to the
    // calculate_k that follows it, and calculate_k leaves its box filter to the matrix-core
    // convolution.  What is handed over is recorded per resource table, not here (api.hip).
    bool fuse_stages = true;
    bool verbose = false;
    // Orders this descriptor's stream with another one (a box filter owed by a descriptor
    // that runs on another stream); created on first use, under mu.
    hipEvent_t order_before = nullptr, order_after = nullptr;
    KernelTimer time_binarize, time_convolution; // empty unless timing is switched on
};

inline State *state_of(const xnor_nn_convolution_t *c) {
    return reinterpret_cast<State *>(c->state);
}

// Kernel launchers (one per stage); each returns the hipError_t of the launch.
hipError_t launch_binarize_data(const Geometry &g, const float *x, uint32_t *bits,
        float *a_or_null, hipStream_t s, const KernelEvents &ev = KernelEvents{});
hipError_t launch_mean_abs(const Geometry &g, const float *x, float *a, hipStream_t s);
hipError_t launch_box_filter(const Geometry &g, const float *a, float *k, hipStream_t s);
// calibration: one pass of plain 16-byte reads over bytes / 16 * 16 bytes of device memory
hipError_t launch_plain_read(const void *buf, size_t bytes, hipStream_t s,
        const KernelEvents &ev = KernelEvents{});
hipError_t launch_binarize_weights(const Geometry &g, const float *w, uint32_t *bits,
        float *alpha, int32_t *opc, hipStream_t s);
hipError_t launch_convolution(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wbits, const float *alpha, const float *k, const int32_t *opc,
        float *dst, int32_t *popc_or_null, hipStream_t s,
        const KernelEvents &ev = KernelEvents{});
// sign(w) * mean(w); parts: weights_float_parts() floats of device memory for partial sums
int weights_float_parts();
hipError_t launch_weights_float(const float *from, float *to, size_t n, float *parts,
        hipStream_t s);
// device address of the library's own partial-sum array on the current GPU (static device
// memory: nothing is allocated)
hipError_t weights_float_scratch(float **out);
// Decides whether the matrix-core kernel takes the problem and fills use_mfma, mfma_ps and
// the mfma_* fields (everything the launch needs, so that a forward call computes nothing).
void mfma_plan(Geometry &g);
const char *mfma_kernel_name(const Geometry &g);
size_t mfma_weight_bytes(const Geometry &g);
hipError_t launch_pack_weights_fp4(const Geometry &g, const float *w, uint32_t *frag,
        hipStream_t s);
// With a_or_null set, the kernel ignores k, computes the K plane itself from mean|x| (the
// box filter of stage 2) and also stores it to k_out.
hipError_t launch_convolution_mfma(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wfrag, const float *alpha, const float *k,
        float *dst, int32_t *popc_or_null, const float *a_or_null, float *k_out,
        hipStream_t s, const KernelEvents &ev = KernelEvents{});
// calibration: `workgroups` x 4 waves, each issuing 8 * iterations FP4 matrix instructions
// (32x32x64) on register-resident +-1 operands
hipError_t launch_mfma_only(int workgroups, int iterations, hipStream_t s);
const char *convolution_kernel_name(const Geometry &g);
// The matrix-core kernel for launches of few tiles (filled in by mfma_plan: g.mfma_small).
bool small_kernel_applies(const Geometry &g, int *rows, uint32_t *lds);
hipError_t launch_convolution_small(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wfrag, const float *alpha, const float *k, float *dst,
        const float *a_or_null, float *k_out, hipStream_t s,
        const KernelEvents &ev = KernelEvents{});
const char *binarize_kernel_name(const Geometry &g);

int pick_q(int oc, int xw);

} // namespace xnor_hip
