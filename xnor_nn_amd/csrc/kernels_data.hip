// Stage 1 and stage 2 of the forward pass: sign-bit packing of the input, mean |x| over
// channels (the "A" plane) and its box filter (the "K" plane).
//
// Semantics follow reference src/bcast_binarize_data.cpp:43-73 and
// src/bcast_calculate_k.cpp:42-85.  Both float reductions are evaluated in exactly the
// reference's order with separately rounded products and sums (no FMA contraction), so
// a and k come out bit-identical to the CPU library.
#include <cstdlib>

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
// wave w of the group owns S consecutive 32-channel slices per round (slices
// (r*NW + w)*S .. +S-1 in round r).  A lane is a pixel, so every load instruction reads 64
// consecutive floats of one channel plane.  All 32*S loads of a wave are issued before
// the first use.  Sign bits are shifted into the lane's word with one funnel shift per
// element (a ballot would produce pixel-major masks of one channel, i.e. the transpose
// of what is stored).
//
// mean|x| must be summed over channels in order.  The waves therefore hand the running
// sum from one to the next through LDS: wave w adds its terms after wave w-1 has published
// its result.  The loads of every wave are in flight during that chain.
//
// The packed words of the tile are staged in LDS and written as one contiguous run.
//
// Workgroup b works on tile (b % 8) * tiles_per_xcd + b / 8: workgroups are dealt to the
// eight XCDs round-robin, so this gives each XCD one contiguous range of tiles and the
// cache lines that straddle two neighbouring tiles (a channel plane is rarely a multiple
// of 128 bytes) are fetched into one L2 instead of two.
template <int S, bool WRITE_BITS, bool WRITE_A>
__global__ __launch_bounds__(TILE * MAX_WAVES / S)
void binarize_nchw_kernel(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry g, const float inv_ic, const int rounds,
        const uint32_t ntiles, const uint32_t tiles_per_xcd) {
    extern __shared__ uint32_t lds[];
    float *chain = reinterpret_cast<float *>(lds); // [TILE]
    uint32_t *stage = lds + TILE;                  // [TILE][xw]

    const uint32_t tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= ntiles) return;

    const int lane = threadIdx.x & (TILE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;

    const uint32_t p = tile * TILE + lane;
    const bool live = p < g.npix_in;
    const uint32_t pc = live ? p : g.npix_in - 1;
    const uint32_t img = g.div_ihw.div(pc);
    const uint32_t hw = pc - img * g.ihw;
    const float *base = x + (size_t)img * g.ic * g.ihw + hw;

    if (wave == 0) chain[lane] = 0.f;

    for (int r = 0; r < rounds; r++) {
        const int slice0 = (r * nw + wave) * S; // wave-uniform
        const int c0 = slice0 * 32;
        const bool has = c0 < g.ic;
        float t[32 * S];
        if (has) {
            const float *col = base + (size_t)c0 * g.ihw;
            if (c0 + 32 * S <= g.ic) {
#pragma unroll
                for (int i = 0; i < 32 * S; i++) t[i] = col[(size_t)i * g.ihw];
            } else {
#pragma unroll
                for (int i = 0; i < 32 * S; i++)
                    t[i] = (c0 + i < g.ic) ? col[(size_t)i * g.ihw] : 0.f;
            }
#pragma unroll
            for (int sl = 0; sl < S; sl++) {
                uint32_t neg = 0; // sign bits, first channel ends up in the MSB
#pragma unroll
                for (int i = 0; i < 32; i++) {
                    neg = __builtin_amdgcn_alignbit(neg, fbits(t[32 * sl + i]), 31);
                    t[32 * sl + i] = __fmul_rn(__builtin_fabsf(t[32 * sl + i]), inv_ic);
                }
                const int n = g.ic - (c0 + 32 * sl);
                if (WRITE_BITS && n > 0)
                    stage[lane * g.xw + slice0 + sl] = (~neg) & top_bits(n);
            }
        }
        // ordered hand-over of the running sum: wave s goes after wave s-1
        for (int s = 0; s < nw; s++) {
            if (s == wave && has) {
                float acc = chain[lane];
#pragma unroll
                for (int i = 0; i < 32 * S; i++) acc = __fadd_rn(acc, t[i]);
                chain[lane] = acc;
            }
            __syncthreads();
        }
    }

    const size_t tile_words = (size_t)TILE * g.xw;
    const size_t first = (size_t)tile * tile_words;
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

// Slices per wave.  Two slices per wave halve the waves of a workgroup but need over 100
// VGPRs, which leaves no more workgroups resident than one slice per wave does; measured
// equal or slower on MI355X, so one is used.
int slices_per_wave(const Geometry &g) {
    if (const char *e = getenv("XNOR_NN_HIP_BIN_S")) return atoi(e) == 2 ? 2 : 1;
    (void)g;
    return 1;
}

template <int S, bool WRITE_BITS, bool WRITE_A>
void launch_nchw(const Geometry &g, const float *x, uint32_t *bits, float *a, hipStream_t s) {
    const int max_waves = MAX_WAVES / S;
    const int need = (g.xw + S - 1) / S;
    const int nw = need < max_waves ? need : max_waves;
    const int rounds = (need + nw - 1) / nw;
    const uint32_t ntiles = (g.npix_in + TILE - 1) / TILE;
    const uint32_t per_xcd = (ntiles + 7) / 8;
    const size_t lds = sizeof(uint32_t) * (TILE + (size_t)TILE * g.xw);
    hipLaunchKernelGGL((binarize_nchw_kernel<S, WRITE_BITS, WRITE_A>), dim3(per_xcd * 8),
            dim3(nw * TILE), lds, s, x, bits, a, g, 1.f / g.ic, rounds, ntiles, per_xcd);
}

template <bool WRITE_BITS, bool WRITE_A>
void launch_nchw(const Geometry &g, const float *x, uint32_t *bits, float *a, hipStream_t s) {
    if (slices_per_wave(g) == 2) launch_nchw<2, WRITE_BITS, WRITE_A>(g, x, bits, a, s);
    else launch_nchw<1, WRITE_BITS, WRITE_A>(g, x, bits, a, s);
}

} // namespace

const char *binarize_kernel_name(const Geometry &g) {
    return g.src_fmt == xnor_nn_data_format_nchw ? "binarize_nchw_kernel"
                                                 : "binarize_generic_kernel";
}

hipError_t launch_binarize_data(const Geometry &g, const float *x, uint32_t *bits,
        float *a_or_null, hipStream_t s) {
    const float inv_ic = 1.f / g.ic;
    if (g.src_fmt == xnor_nn_data_format_nchw) {
        if (a_or_null) launch_nchw<true, true>(g, x, bits, a_or_null, s);
        else launch_nchw<true, false>(g, x, bits, nullptr, s);
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
        launch_nchw<false, true>(g, x, nullptr, a, s);
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
