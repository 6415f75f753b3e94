// Stage 1 and stage 2 of the forward pass: sign-bit packing of the input, mean |x| over
// channels (the "A" plane) and its box filter (the "K" plane).
//
// Semantics follow reference src/bcast_binarize_data.cpp:43-73 and
// src/bcast_calculate_k.cpp:42-85.  Both float reductions are evaluated in exactly the
// reference's order with separately rounded products and sums (no FMA contraction), so
// a and k come out bit-identical to the CPU library.
#include "plan.hpp"

namespace xnor_hip {

namespace {

constexpr int TILE = 64;       // pixels per workgroup = lanes per wave
constexpr int MAX_WAVES = 16;  // 1024 threads

__device__ __forceinline__ uint32_t fbits(float v) { return __float_as_uint(v); }

// Mask that keeps the n most significant bits of a word (n in 1..32).
__device__ __forceinline__ uint32_t top_bits(int n) {
    return n >= 32 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu >> n);
}

// NCHW input.  One workgroup = 64 consecutive pixels of the flattened (mb, ih, iw) index;
// wave w of the group owns the 32-channel slices w, w+NW, ... of those pixels.  A lane is
// a pixel, so every load instruction reads 64 consecutive floats of one channel plane.
// All 32 loads of a slice are issued before the first use.  Sign bits are shifted into
// the lane's word with one funnel shift per element (a ballot would produce
// pixel-major masks of one channel, i.e. the transpose of what is stored).
//
// mean|x| must be summed over channels in order.  The slices therefore hand the running
// sum from wave to wave through LDS: slice s adds its 32 terms after slice s-1 has
// published its result.  Loads of all slices are in flight during that chain.
//
// The packed words of the tile are staged in LDS and written as one contiguous run.
template <bool WRITE_BITS, bool WRITE_A>
__global__ __launch_bounds__(TILE * MAX_WAVES)
void binarize_nchw_kernel(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry g, const float inv_ic, const int rounds) {
    extern __shared__ uint32_t lds[];
    float *chain = reinterpret_cast<float *>(lds); // [TILE]
    uint32_t *stage = lds + TILE;                  // [TILE][xw]

    const int lane = threadIdx.x & (TILE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;

    const uint32_t p = blockIdx.x * TILE + lane;
    const bool live = p < g.npix_in;
    const uint32_t pc = live ? p : g.npix_in - 1;
    const uint32_t img = g.div_ihw.div(pc);
    const uint32_t hw = pc - img * g.ihw;
    const float *base = x + (size_t)img * g.ic * g.ihw + hw;

    if (wave == 0) chain[lane] = 0.f;

    for (int r = 0; r < rounds; r++) {
        const int slice = r * nw + wave; // wave-uniform
        const int c0 = slice * 32;
        const bool has = c0 < g.ic;
        float t[32];
        uint32_t neg = 0; // sign bits, first channel ends up in the MSB
        if (has) {
            const float *col = base + (size_t)c0 * g.ihw;
            float v[32];
            if (c0 + 32 <= g.ic) {
#pragma unroll
                for (int i = 0; i < 32; i++) v[i] = col[(size_t)i * g.ihw];
            } else {
#pragma unroll
                for (int i = 0; i < 32; i++)
                    v[i] = (c0 + i < g.ic) ? col[(size_t)i * g.ihw] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < 32; i++) {
                neg = __builtin_amdgcn_alignbit(neg, fbits(v[i]), 31);
                t[i] = __fmul_rn(__builtin_fabsf(v[i]), inv_ic);
            }
            const int n = min(32, g.ic - c0);
            if (WRITE_BITS) stage[lane * g.xw + slice] = (~neg) & top_bits(n);
        }
        // ordered hand-over of the running sum: slice s goes after slice s-1
        for (int s = 0; s < nw; s++) {
            if (s == wave && has) {
                float acc = chain[lane];
#pragma unroll
                for (int i = 0; i < 32; i++) acc = __fadd_rn(acc, t[i]);
                chain[lane] = acc;
            }
            __syncthreads();
        }
    }

    const size_t tile_words = (size_t)TILE * g.xw;
    const size_t first = (size_t)blockIdx.x * tile_words;
    const size_t total = (size_t)g.npix_in * g.xw;
    if (WRITE_BITS)
        for (uint32_t i = threadIdx.x; i < tile_words; i += blockDim.x)
            if (first + i < total) bits[first + i] = stage[i];
    if (WRITE_A && wave == 0 && live) a[p] = chain[lane];
}

// Any source layout, one lane per pixel, channels visited in order.  Used for NHWC input
// (reference src/bcast_binarize_data.cpp:56-57, src/bcast_calculate_k.cpp:59-60).
template <bool WRITE_BITS, bool WRITE_A>
__global__ __launch_bounds__(256)
void binarize_generic_kernel(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry g, const float inv_ic) {
    const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= g.npix_in) return;
    const uint32_t img = g.div_ihw.div(p);
    const uint32_t hw = p - img * g.ihw;
    size_t idx, step;
    if (g.src_fmt == xnor_nn_data_format_nchw) {
        idx = (size_t)img * g.ic * g.ihw + hw;
        step = g.ihw;
    } else {
        idx = (size_t)p * g.ic;
        step = 1;
    }
    float acc = 0.f;
    for (int j = 0; j < g.xw; j++) {
        uint32_t neg = 0;
        const int n = min(32, g.ic - 32 * j);
        for (int i = 0; i < n; i++) {
            const float v = x[idx];
            idx += step;
            neg = __builtin_amdgcn_alignbit(neg, fbits(v), 31);
            acc = __fadd_rn(acc, __fmul_rn(__builtin_fabsf(v), inv_ic));
        }
        if (WRITE_BITS) bits[(size_t)p * g.xw + j] = (~(neg << (32 - n))) & top_bits(n);
    }
    if (WRITE_A) a[p] = acc;
}

// K plane: k = sum over in-bounds taps, row-major, of fl(a * KHW)
// (reference src/bcast_calculate_k.cpp:69-85).  One lane per output pixel.
__global__ __launch_bounds__(256)
void box_filter_kernel(const float *__restrict__ a, float *__restrict__ k,
        const Geometry g, const float inv_khw) {
    const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= g.npix_out) return;
    const uint32_t img = g.div_ohw.div(p);
    const uint32_t rem = p - img * g.ohw;
    const int oh = (int)g.div_ow.div(rem);
    const int ow = (int)rem - oh * g.ow;
    const float *plane = a + (size_t)img * g.ihw;
    float acc = 0.f;
    for (int kh = 0; kh < g.kh; kh++) {
        const int ih = oh * g.sh - g.ph + kh;
        if (ih < 0 || ih >= g.ih) continue;
        for (int kw = 0; kw < g.kw; kw++) {
            const int iw = ow * g.sw - g.pw + kw;
            if (iw < 0 || iw >= g.iw) continue;
            acc = __fadd_rn(acc, __fmul_rn(plane[ih * g.iw + iw], inv_khw));
        }
    }
    k[p] = acc;
}

int data_waves(const Geometry &g) { return g.xw < MAX_WAVES ? g.xw : MAX_WAVES; }

} // namespace

const char *binarize_kernel_name(const Geometry &g) {
    return g.src_fmt == xnor_nn_data_format_nchw ? "binarize_nchw_kernel"
                                                 : "binarize_generic_kernel";
}

hipError_t launch_binarize_data(const Geometry &g, const float *x, uint32_t *bits,
        float *a_or_null, hipStream_t s) {
    const float inv_ic = 1.f / g.ic;
    if (g.src_fmt == xnor_nn_data_format_nchw) {
        const int nw = data_waves(g);
        const int rounds = (g.xw + nw - 1) / nw;
        const unsigned blocks = (g.npix_in + TILE - 1) / TILE;
        const size_t lds = sizeof(uint32_t) * (TILE + (size_t)TILE * g.xw);
        if (a_or_null)
            hipLaunchKernelGGL((binarize_nchw_kernel<true, true>), dim3(blocks),
                    dim3(nw * TILE), lds, s, x, bits, a_or_null, g, inv_ic, rounds);
        else
            hipLaunchKernelGGL((binarize_nchw_kernel<true, false>), dim3(blocks),
                    dim3(nw * TILE), lds, s, x, bits, a_or_null, g, inv_ic, rounds);
    } else {
        const unsigned blocks = (g.npix_in + 255) / 256;
        if (a_or_null)
            hipLaunchKernelGGL((binarize_generic_kernel<true, true>), dim3(blocks),
                    dim3(256), 0, s, x, bits, a_or_null, g, inv_ic);
        else
            hipLaunchKernelGGL((binarize_generic_kernel<true, false>), dim3(blocks),
                    dim3(256), 0, s, x, bits, a_or_null, g, inv_ic);
    }
    return hipGetLastError();
}

hipError_t launch_mean_abs(const Geometry &g, const float *x, float *a, hipStream_t s) {
    const float inv_ic = 1.f / g.ic;
    if (g.src_fmt == xnor_nn_data_format_nchw) {
        const int nw = data_waves(g);
        const int rounds = (g.xw + nw - 1) / nw;
        const unsigned blocks = (g.npix_in + TILE - 1) / TILE;
        const size_t lds = sizeof(uint32_t) * (TILE + (size_t)TILE * g.xw);
        hipLaunchKernelGGL((binarize_nchw_kernel<false, true>), dim3(blocks),
                dim3(nw * TILE), lds, s, x, nullptr, a, g, inv_ic, rounds);
    } else {
        const unsigned blocks = (g.npix_in + 255) / 256;
        hipLaunchKernelGGL((binarize_generic_kernel<false, true>), dim3(blocks), dim3(256),
                0, s, x, nullptr, a, g, inv_ic);
    }
    return hipGetLastError();
}

hipError_t launch_box_filter(const Geometry &g, const float *a, float *k, hipStream_t s) {
    const float inv_khw = 1.f / g.kh / g.kw; // two divisions, like the reference
    const unsigned blocks = (g.npix_out + 255) / 256;
    hipLaunchKernelGGL(box_filter_kernel, dim3(blocks), dim3(256), 0, s, a, k, g, inv_khw);
    return hipGetLastError();
}

} // namespace xnor_hip
