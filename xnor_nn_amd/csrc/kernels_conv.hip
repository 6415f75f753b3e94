// Stage 3 of the forward pass: XNOR + popcount direct convolution with the fused
// alpha * k * (2*popc - n) epilogue (reference
// src/default/bcast_convolution_default.cpp:60-105 is the readable specification; the
// reference's AVX/SSE/NEON kernels compute the same values).
//
// Mapping.  A lane is one output pixel of the flattened (mb, oh, ow) index and keeps Q
// int32 accumulators, one per filter of the wave's filter group.  The packed filter
// words are wave-uniform, so they are fetched with scalar loads and used directly as the
// SGPR operand of v_xnor_b32; the popcount is v_bcnt_u32_b32, which adds into its third
// operand.  That is two VALU instructions per 32 binary multiply-accumulates per lane and
// nothing else in the inner loop.  Each lane loads the XW packed words of its input
// pixel once per tap (vector loads, L1/L2 resident: the packed input is 1/32 of the
// fp32 tensor) and reuses them for all Q filters.  Out-of-bounds taps are skipped by
// predication, exactly like the reference's `continue`, so no correction term exists.
#include "plan.hpp"

namespace xnor_hip {

namespace {

constexpr int WAVES = 4; // waves per workgroup; they share the pixel tile

template <int XW>
struct Words {
    uint32_t v[XW];
};

// Load the XW consecutive words of one packed pixel (16-byte vectors where XW allows).
template <int XW>
__device__ __forceinline__ void load_pixel(const uint32_t *__restrict__ p, uint32_t (&v)[XW]) {
    if constexpr (XW % 4 == 0) {
        const uint4 *q = reinterpret_cast<const uint4 *>(p);
#pragma unroll
        for (int i = 0; i < XW / 4; i++) {
            const uint4 t = q[i];
            v[4 * i + 0] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else if constexpr (XW % 2 == 0) {
        const uint2 *q = reinterpret_cast<const uint2 *>(p);
#pragma unroll
        for (int i = 0; i < XW / 2; i++) {
            const uint2 t = q[i];
            v[2 * i + 0] = t.x; v[2 * i + 1] = t.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < XW; i++) v[i] = p[i];
    }
}

// XW > 0: words per pixel fixed at compile time (fully unrolled).
// XW == 0: runtime word count (any shape).
template <int XW, int Q, bool RAW>
__global__ __launch_bounds__(64 * WAVES)
void conv_xnor_popc_kernel(const uint32_t *__restrict__ xbits,
        const uint32_t *__restrict__ wbits, const float *__restrict__ alpha,
        const float *__restrict__ kplane, const int32_t *__restrict__ opc,
        float *__restrict__ dst, int32_t *__restrict__ popc, const Geometry g) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ob = blockIdx.y * WAVES + wave; // filter group of this wave (uniform)
    if (ob >= g.ocb) return;

    const uint32_t p = blockIdx.x * 64 + lane;
    const bool live = p < g.npix_out;
    const uint32_t pc = live ? p : g.npix_out - 1;
    const uint32_t img = g.div_ohw.div(pc);
    const uint32_t rem = pc - img * g.ohw;
    const int oh = (int)g.div_ow.div(rem);
    const int ow = (int)rem - oh * g.ow;
    const int ih0 = oh * g.sh - g.ph;
    const int iw0 = ow * g.sw - g.pw;
    const int xw = XW > 0 ? XW : g.xw;

    const uint32_t *ximg = xbits + (size_t)img * g.ihw * xw;
    const uint32_t *wgrp = wbits + (size_t)ob * g.kh * g.kw * xw * Q;

    int acc[Q];
#pragma unroll
    for (int q = 0; q < Q; q++) acc[q] = 0;

    for (int kh = 0; kh < g.kh; kh++) {
        const int ih = ih0 + kh;
        const bool row_ok = (unsigned)ih < (unsigned)g.ih;
        for (int kw = 0; kw < g.kw; kw++) {
            const int iw = iw0 + kw;
            const uint32_t *wtap = wgrp + (size_t)(kh * g.kw + kw) * xw * Q;
            if (row_ok && (unsigned)iw < (unsigned)g.iw) {
                const uint32_t *xp = ximg + (size_t)(ih * g.iw + iw) * xw;
                if constexpr (XW > 0) {
                    uint32_t xv[XW];
                    load_pixel<XW>(xp, xv);
#pragma unroll
                    for (int j = 0; j < XW; j++) {
#pragma unroll
                        for (int q = 0; q < Q; q++)
                            acc[q] += __builtin_popcount(~(xv[j] ^ wtap[j * Q + q]));
                    }
                } else {
                    for (int j = 0; j < xw; j++) {
                        const uint32_t xv = xp[j];
#pragma unroll
                        for (int q = 0; q < Q; q++)
                            acc[q] += __builtin_popcount(~(xv ^ wtap[j * Q + q]));
                    }
                }
            }
        }
    }

    if (!live) return;
    const int oc0 = ob * Q;
    if constexpr (RAW) {
#pragma unroll
        for (int q = 0; q < Q; q++)
            if (oc0 + q < g.oc)
                popc[((size_t)img * g.oc + oc0 + q) * g.ohw + rem] = acc[q];
    } else {
        // dst = fl(fl((float)(2*popc - n) * alpha) * k), products rounded separately
        const int n = opc[rem];
        const float kv = kplane[p];
        if (g.dst_fmt == xnor_nn_data_format_nchw) {
            float *out = dst + ((size_t)img * g.oc + oc0) * g.ohw + rem;
#pragma unroll
            for (int q = 0; q < Q; q++)
                if (oc0 + q < g.oc)
                    out[(size_t)q * g.ohw] =
                        __fmul_rn(__fmul_rn((float)(2 * acc[q] - n), alpha[oc0 + q]), kv);
        } else {
            float *out = dst + (size_t)p * g.oc + oc0;
#pragma unroll
            for (int q = 0; q < Q; q++)
                if (oc0 + q < g.oc)
                    out[q] = __fmul_rn(__fmul_rn((float)(2 * acc[q] - n), alpha[oc0 + q]), kv);
        }
    }
}

template <int XW, int Q>
hipError_t launch_variant(const Geometry &g, const uint32_t *xbits, const uint32_t *wbits,
        const float *alpha, const float *k, const int32_t *opc, float *dst, int32_t *popc,
        hipStream_t s, const KernelEvents &ev) {
    const dim3 grid((g.npix_out + 63) / 64, (g.ocb + WAVES - 1) / WAVES);
    const dim3 block(64 * WAVES);
    if (popc)
        launch_kernel(conv_xnor_popc_kernel<XW, Q, true>, grid, block, 0, s, ev, xbits,
                wbits, alpha, k, opc, dst, popc, g);
    else
        launch_kernel(conv_xnor_popc_kernel<XW, Q, false>, grid, block, 0, s, ev, xbits,
                wbits, alpha, k, opc, dst, popc, g);
    return hipGetLastError();
}

} // namespace

// Filters per wave.  16 keeps the accumulators and one tap-word of weights (16 SGPRs)
// comfortably inside the register files.
int pick_q(int oc, int xw) {
    (void)xw;
    return oc >= 16 ? 16 : 8;
}

const char *convolution_kernel_name(const Geometry &g) {
    static thread_local char name[64];
    if (g.use_mfma) return mfma_kernel_name(g);
    const int xw = (g.xw == 3 || g.xw == 8 || g.xw == 12 || g.xw == 16) ? g.xw : 0;
    snprintf(name, sizeof name, "conv_xnor_popc_kernel<XW=%d,Q=%d>", xw, g.q);
    return name;
}

hipError_t launch_convolution(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wbits, const float *alpha, const float *k, const int32_t *opc,
        float *dst, int32_t *popc, hipStream_t s, const KernelEvents &ev) {
#define XNOR_CASE(XW_, Q_) \
    if (g.q == Q_ && (XW_ == 0 || g.xw == XW_)) \
        return launch_variant<XW_, Q_>(g, xbits, wbits, alpha, k, opc, dst, popc, s, ev);
    XNOR_CASE(3, 16)
    XNOR_CASE(8, 16)
    XNOR_CASE(12, 16)
    XNOR_CASE(16, 16)
    XNOR_CASE(0, 16)
    XNOR_CASE(0, 8)
#undef XNOR_CASE
    return hipErrorInvalidValue;
}

} // namespace xnor_hip
