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
constexpr int MAX_WAVES = 12;  // waves per workgroup
constexpr int TURN_ROW = 36;   // floats per pixel row of the NHWC turn-around buffer (32 + 4)
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t fbits(float v) { return __float_as_uint(v); }

// Mask that keeps the n most significant bits of a word (n in 1..32).
__device__ __forceinline__ uint32_t top_bits(int n) {
    return n >= 32 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu >> n);
}

// NCHW input.  A tile is 64 consecutive pixels of the flattened (mb, ih, iw) index; wave w of
// the workgroup owns the 32-channel slices w, w + NW, ... of it.  A lane is a pixel, so every
// load instruction reads 64 consecutive floats of one channel plane.  All 32 loads of a slice
// are issued before the first use.  Sign bits are shifted into the lane's word with one
// funnel shift per element (a ballot would produce pixel-major masks of one channel, i.e.
// the transpose of what is stored).
//
// mean|x| must be summed over channels in order.  The waves therefore hand the running
// sum from one to the next through LDS: wave w adds its terms after wave w-1 has published
// its result.  The packed words of the tile are staged in LDS and written as one
// contiguous run.
//
// One workgroup per tile.  (A persistent grid that issues the loads of its next tile before
// it processes the current one was measured and is not used: at these sizes the kernel is
// bound by the transfer plus one pass of the sum through the waves, and the hardware's own
// workgroup scheduling does as well as the hand-made pipeline.)
//
// Workgroups are dealt to the eight XCDs round-robin.  XCD x owns the contiguous range of
// tiles [x * tiles_per_xcd, (x+1) * tiles_per_xcd): the cache lines that straddle two
// neighbouring tiles (a channel plane is rarely a multiple of 128 bytes) are fetched into
// one L2 instead of two.  Workgroup b takes local tile b / 8 of XCD b % 8.
//
// NHWC input (channel count a multiple of 4) runs the same tile: the 32 values of a slice are
// then 128 contiguous bytes of a pixel.  A wave fetches them eight lanes to a pixel, so that
// every load instruction reads eight whole cache lines, and turns the block around through
// LDS into the lane = pixel layout (one lane per pixel straight from memory, 64 partial
// cache lines per instruction, took 19.7 us where this takes 13.5 us, the NCHW kernel 13.3).
template <bool NHWC, bool WRITE_BITS, bool WRITE_A>
__device__ __forceinline__
void binarize_tile(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry &g, const float inv_ic, const int rounds,
        const uint32_t ntiles, const uint32_t tiles_per_xcd) {
    extern __shared__ uint32_t lds[];
    float *chain = reinterpret_cast<float *>(lds); // [TILE]
    uint32_t *stage = lds + TILE;                  // [TILE][xw]
    // NHWC: [waves][32 pixels][TURN_ROW floats], 16-byte aligned
    float *turn = reinterpret_cast<float *>(lds + ((TILE + TILE * g.xw + 3) & ~3));

    const int lane = threadIdx.x & (TILE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;
    const uint32_t tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= ntiles) return;

    // the whole input as one raw buffer (the host side checks that it is below 4 GiB)
    const __amdgpu_buffer_rsrc_t src = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(x), 0, (int)((uint32_t)g.npix_in * (uint32_t)g.ic * 4u),
            0x00020000);
    // slice (r * nw + wave) of a tile: 32 channel values of this lane's pixel
    auto load_slice = [&](float (&t)[32], uint32_t tile, int r) {
        const uint32_t p = tile * TILE + lane;
        const uint32_t pc = p < g.npix_in ? p : g.npix_in - 1;
        const uint32_t img = g.div_ihw.div(pc);
        const uint32_t hw = pc - img * g.ihw;
        const int c0 = (r * nw + wave) * 32; // wave-uniform
        if (c0 >= g.ic) return;
        if constexpr (NHWC) {
            // Load i of the wave reads the slice of pixels 8i .. 8i+7 of the tile: eight
            // lanes per pixel, 16 bytes each, i.e. eight whole cache lines per instruction.
            // The wave then turns the 64 x 128 bytes around through its own piece of LDS
            // (32 pixels at a time, rows of 144 bytes so that neither side has bank
            // conflicts) to end up with the lane = pixel layout of the rest of the kernel.
            typedef float v4f __attribute__((ext_vector_type(4)));
            const int piece = lane & 7;
            const int c = c0 + 4 * piece; // IC is a multiple of 4: a piece is inside or outside
            v4f v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t q = tile * TILE + 8 * i + (lane >> 3);
                const uint32_t qc = q < g.npix_in ? q : g.npix_in - 1;
                // a piece past the last channel gets an offset outside the buffer: reads +0
                const uint32_t off = c < g.ic ? qc * (uint32_t)g.ic * 4u + (uint32_t)c * 4u
                                              : 0xFFFFFFF0u;
                v[i] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
                        src, off, 0, 0));
            }
            float *mine = turn + wave * (32 * TURN_ROW);
#pragma unroll
            for (int half = 0; half < 2; half++) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    *reinterpret_cast<v4f *>(mine + (8 * i + (lane >> 3)) * TURN_ROW + 4 * piece)
                        = v[4 * half + i];
                if ((lane >> 5) == half) {
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const v4f r = *reinterpret_cast<const v4f *>(
                                mine + (lane & 31) * TURN_ROW + 4 * u);
#pragma unroll
                        for (int e = 0; e < 4; e++) t[4 * u + e] = r[e];
                    }
                }
            }
            return;
        }
        // Buffer loads: one VGPR holds the lane's byte offset for all 32 loads, the channel
        // plane is a scalar offset (no 64-bit address arithmetic per load, fewer VGPRs).
        const uint32_t lane_off = (img * (uint32_t)(g.ic * g.ihw) + hw) * 4u;
        const uint32_t plane_bytes = (uint32_t)g.ihw * 4u;
        if (c0 + 32 <= g.ic) {
#pragma unroll
            for (int i = 0; i < 32; i++)
                t[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                        src, lane_off, (uint32_t)(c0 + i) * plane_bytes, 0));
        } else {
            // last, ragged slice: a channel past the end gets an offset outside the buffer and
            // reads +0 (no branch per load); its bit is masked out of the word below and |+0|
            // leaves the running sum as it is
#pragma unroll
            for (int i = 0; i < 32; i++)
                t[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                        src, c0 + i < g.ic ? lane_off : 0xFFFFFFF0u,
                        c0 + i < g.ic ? (uint32_t)(c0 + i) * plane_bytes : 0u, 0));
        }
    };

    // everything after the loads of the first pass over the slices (r = 0); t holds them
    auto process = [&](float (&t)[32], uint32_t tile) {
        const uint32_t p = tile * TILE + lane;
        if (wave == 0) chain[lane] = 0.f;
        for (int r = 0; r < rounds; r++) {
            if (r > 0) load_slice(t, tile, r);
            const int slice = r * nw + wave; // wave-uniform
            const int c0 = slice * 32;
            const bool has = c0 < g.ic;
            if (has) {
                uint32_t neg = 0; // sign bits, first channel ends up in the MSB
#pragma unroll
                for (int i = 0; i < 32; i++) {
                    neg = __builtin_amdgcn_alignbit(neg, fbits(t[i]), 31);
                    t[i] = __fmul_rn(__builtin_fabsf(t[i]), inv_ic);
                }
                if (WRITE_BITS) stage[lane * g.xw + slice] = (~neg) & top_bits(g.ic - c0);
            }
            // ordered hand-over of the running sum: wave s goes after wave s-1
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
        const size_t first = (size_t)tile * tile_words;
        const size_t total = (size_t)g.npix_in * g.xw;
        if (WRITE_BITS)
            for (uint32_t i = threadIdx.x; i < tile_words; i += blockDim.x)
                if (first + i < total) bits[first + i] = stage[i];
        if (WRITE_A && wave == 0 && p < g.npix_in) a[p] = chain[lane];
    };

    float t[32];
    load_slice(t, tile, 0);
    process(t, tile);
}

template <bool WRITE_BITS, bool WRITE_A>
__global__ __launch_bounds__(TILE * 16)
void binarize_nchw_kernel(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry g, const float inv_ic, const int rounds,
        const uint32_t ntiles, const uint32_t tiles_per_xcd) {
    binarize_tile<false, WRITE_BITS, WRITE_A>(x, bits, a, g, inv_ic, rounds, ntiles,
            tiles_per_xcd);
}

template <bool WRITE_BITS, bool WRITE_A>
__global__ __launch_bounds__(TILE * 16)
void binarize_nhwc_tiled_kernel(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry g, const float inv_ic, const int rounds,
        const uint32_t ntiles, const uint32_t tiles_per_xcd) {
    binarize_tile<true, WRITE_BITS, WRITE_A>(x, bits, a, g, inv_ic, rounds, ntiles,
            tiles_per_xcd);
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

// NHWC input with IC a multiple of 4 and too many channels for the tiled kernel's LDS: a lane
// is a pixel and walks over its channels, which
// are contiguous, in order, 32 at a time (one packed word): eight 16-byte buffer loads per
// word, the loads of the next three words in flight while the current one is folded into
// the sign word and the running mean|x| (reference src/bcast_binarize_data.cpp:56-57,
// src/bcast_calculate_k.cpp:59-60).  The lanes of a wave read addresses IC*4 bytes apart,
// so every load touches 64 cache lines, but each line is used completely by the loads that
// follow, and HBM traffic is the algorithmic minimum.
template <bool WRITE_BITS, bool WRITE_A>
__global__ __launch_bounds__(256)
void binarize_nhwc_kernel(const float *__restrict__ x, uint32_t *__restrict__ bits,
        float *__restrict__ a, const Geometry g, const float inv_ic) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t pc = p < g.npix_in ? p : g.npix_in - 1;
    const __amdgpu_buffer_rsrc_t src = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(x), 0, (int)((uint32_t)g.npix_in * (uint32_t)g.ic * 4u),
            0x00020000);
    const uint32_t lane_off = pc * (uint32_t)g.ic * 4u;
    // 32 channels starting at c0; channels >= IC read as +0 (sign bit clear, |x| = 0: they
    // are masked out of the word and add nothing to the sum)
    auto fetch = [&](v4f (&v)[8], int c0) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int c = c0 + 4 * u; // uniform
            v[u] = c < g.ic ? __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
                                      src, lane_off, (uint32_t)c * 4u, 0))
                            : v4f{0.f, 0.f, 0.f, 0.f};
        }
    };
    float acc = 0.f;
    auto fold = [&](const v4f (&v)[8], int j) { // word j: sign bits and the running sum
        if (j >= g.xw) return; // uniform
        uint32_t neg = 0; // sign bits, first channel ends up in the MSB
        const int n = min(32, g.ic - 32 * j);
#pragma unroll
        for (int u = 0; u < 8; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float val = v[u][e];
                neg = __builtin_amdgcn_alignbit(neg, fbits(val), 31);
                if (4 * u + e < n) // uniform; a sum must not see the padding's +0 terms
                    acc = __fadd_rn(acc, __fmul_rn(__builtin_fabsf(val), inv_ic));
            }
        if (WRITE_BITS && p < g.npix_in) bits[(size_t)p * g.xw + j] = (~neg) & top_bits(n);
    };
    // four register sets used in turn: three words are in flight while one is folded
    v4f b0[8], b1[8], b2[8], b3[8];
    fetch(b0, 0);
    fetch(b1, 32);
    fetch(b2, 64);
    for (int j = 0; j < g.xw; j += 4) {
        fetch(b3, 32 * (j + 3));
        fold(b0, j);
        fetch(b0, 32 * (j + 4));
        fold(b1, j + 1);
        fetch(b1, 32 * (j + 5));
        fold(b2, j + 2);
        fetch(b2, 32 * (j + 6));
        fold(b3, j + 3);
    }
    if (WRITE_A && p < g.npix_in) a[p] = acc;
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

// Calibration only: reads a buffer once, 16 bytes per lane and load, four loads in flight per
// lane, and keeps nothing.  What this takes is what the memory system allows a kernel that
// does no work at all on the same bytes.
__global__ __launch_bounds__(256)
void plain_read_kernel(const v4u *__restrict__ x, const size_t n16) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    v4u acc = {0u, 0u, 0u, 0u};
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const v4u v0 = x[i], v1 = x[i + stride], v2 = x[i + 2 * stride], v3 = x[i + 3 * stride];
        acc ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < n16; i += stride) acc ^= x[i];
    asm volatile("" : : "v"(acc)); // the loads have a use
}

template <bool NHWC, bool WRITE_BITS, bool WRITE_A>
void launch_tiled(const Geometry &g, const float *x, uint32_t *bits, float *a, hipStream_t s,
        const KernelEvents &ev) {
    // At most twelve waves per workgroup, the slices split evenly over the rounds: with more
    // waves the hand-over chain of one workgroup gets long and too few workgroups are
    // resident to cover it (512 input channels: 14.1 us with 16 waves, 10.4 us with 2 x 8;
    // 384 channels: 12 x 1 and 6 x 2 are equal at MB 256, 12 x 1 is 5% faster at MB 1024).
    // XNOR_NN_HIP_BIN_WAVES overrides the cap for measurements.
    const int need = g.xw;
    int cap = MAX_WAVES;
    if (const char *e = getenv("XNOR_NN_HIP_BIN_WAVES")) {
        const int v = atoi(e);
        if (v >= 1 && v <= 16) cap = v;
    }
    const int rounds = (need + cap - 1) / cap;
    const int nw = (need + rounds - 1) / rounds;
    const uint32_t ntiles = (g.npix_in + TILE - 1) / TILE;
    const uint32_t per_xcd = (ntiles + 7) / 8;
    size_t lds = sizeof(uint32_t) * (TILE + (size_t)TILE * g.xw);
    if (NHWC) lds = ((lds + 15) & ~(size_t)15) + sizeof(float) * nw * 32 * TURN_ROW;
    if (NHWC)
        launch_kernel(binarize_nhwc_tiled_kernel<WRITE_BITS, WRITE_A>, dim3(per_xcd * 8),
                dim3(nw * TILE), lds, s, ev, x, bits, a, g, 1.f / g.ic, rounds, ntiles, per_xcd);
    else
        launch_kernel(binarize_nchw_kernel<WRITE_BITS, WRITE_A>, dim3(per_xcd * 8),
                dim3(nw * TILE), lds, s, ev, x, bits, a, g, 1.f / g.ic, rounds, ntiles, per_xcd);
}

// NHWC input runs the tiled kernel unless its LDS (chain, packed words, turn-around rows) would
// not fit 64 KB (more than about a thousand channels); XNOR_NN_HIP_NHWC=lane forces the
// one-lane-per-pixel kernel (for measurements).
bool nhwc_by_lane(const Geometry &g) {
    const char *e = getenv("XNOR_NN_HIP_NHWC");
    if (e && e[0] == 'l') return true;
    const int rounds = (g.xw + MAX_WAVES - 1) / MAX_WAVES;
    const int nw = (g.xw + rounds - 1) / rounds;
    return sizeof(uint32_t) * (TILE + (size_t)TILE * g.xw) + 16
        + sizeof(float) * nw * 32 * TURN_ROW > 64 * 1024;
}

} // namespace

// The tiled kernel addresses the input with 32-bit byte offsets and stages the packed words
// of a tile in LDS (64 KB at most: up to 8160 channels); deeper or larger inputs run the
// generic kernel.  A channel past the end of a ragged slice is read through the byte offset
// 0xFFFFFFF0, which has to lie outside the buffer for the load to return +0: the input must
// end below that offset.
static bool tiled_nchw(const Geometry &g) {
    return g.src_fmt == xnor_nn_data_format_nchw
        && (uint64_t)g.npix_in * (uint64_t)g.ic * 4u < XNOR_HIP_DROPPED_OFFSET
        && sizeof(uint32_t) * (TILE + (size_t)TILE * g.xw) <= 64 * 1024;
}

// The NHWC kernel reads 16 bytes per load at 32-bit byte offsets (and drops pieces past the
// last channel the same way).
static bool vector_nhwc(const Geometry &g) {
    return g.src_fmt == xnor_nn_data_format_nhwc && (g.ic & 3) == 0
        && (uint64_t)g.npix_in * (uint64_t)g.ic * 4u < XNOR_HIP_DROPPED_OFFSET;
}

const char *binarize_kernel_name(const Geometry &g) {
    return tiled_nchw(g) ? "binarize_nchw_kernel"
        : !vector_nhwc(g) ? "binarize_generic_kernel"
        : nhwc_by_lane(g) ? "binarize_nhwc_kernel" : "binarize_nhwc_tiled_kernel";
}

hipError_t launch_binarize_data(const Geometry &g, const float *x, uint32_t *bits,
        float *a_or_null, hipStream_t s, const KernelEvents &ev) {
    const float inv_ic = 1.f / g.ic;
    if (tiled_nchw(g)) {
        if (a_or_null) launch_tiled<false, true, true>(g, x, bits, a_or_null, s, ev);
        else launch_tiled<false, true, false>(g, x, bits, nullptr, s, ev);
    } else if (vector_nhwc(g) && !nhwc_by_lane(g)) {
        if (a_or_null) launch_tiled<true, true, true>(g, x, bits, a_or_null, s, ev);
        else launch_tiled<true, true, false>(g, x, bits, nullptr, s, ev);
    } else if (vector_nhwc(g)) {
        const unsigned blocks = (g.npix_in + 255) / 256;
        if (a_or_null)
            launch_kernel(binarize_nhwc_kernel<true, true>, dim3(blocks), dim3(256), 0, s, ev,
                    x, bits, a_or_null, g, inv_ic);
        else
            launch_kernel(binarize_nhwc_kernel<true, false>, dim3(blocks), dim3(256), 0, s, ev,
                    x, bits, a_or_null, g, inv_ic);
    } else {
        const unsigned blocks = (g.npix_in + 255) / 256;
        if (a_or_null)
            launch_kernel(binarize_generic_kernel<true, true>, dim3(blocks), dim3(256), 0, s,
                    ev, x, bits, a_or_null, g, inv_ic);
        else
            launch_kernel(binarize_generic_kernel<true, false>, dim3(blocks), dim3(256), 0, s,
                    ev, x, bits, a_or_null, g, inv_ic);
    }
    return hipGetLastError();
}

hipError_t launch_mean_abs(const Geometry &g, const float *x, float *a, hipStream_t s) {
    const float inv_ic = 1.f / g.ic;
    if (tiled_nchw(g)) {
        launch_tiled<false, false, true>(g, x, nullptr, a, s, KernelEvents{});
    } else if (vector_nhwc(g) && !nhwc_by_lane(g)) {
        launch_tiled<true, false, true>(g, x, nullptr, a, s, KernelEvents{});
    } else if (vector_nhwc(g)) {
        const unsigned blocks = (g.npix_in + 255) / 256;
        hipLaunchKernelGGL((binarize_nhwc_kernel<false, true>), dim3(blocks), dim3(256), 0, s,
                x, nullptr, a, g, inv_ic);
    } else {
        const unsigned blocks = (g.npix_in + 255) / 256;
        hipLaunchKernelGGL((binarize_generic_kernel<false, true>), dim3(blocks), dim3(256),
                0, s, x, nullptr, a, g, inv_ic);
    }
    return hipGetLastError();
}

hipError_t launch_plain_read(const void *buf, size_t bytes, hipStream_t s,
        const KernelEvents &ev) {
    launch_kernel(plain_read_kernel, dim3(2048), dim3(256), 0, s, ev,
            static_cast<const v4u *>(buf), bytes / 16);
    return hipGetLastError();
}

hipError_t launch_box_filter(const Geometry &g, const float *a, float *k, hipStream_t s) {
    const float inv_khw = 1.f / g.kh / g.kw; // two divisions, like the reference
    const unsigned blocks = (g.npix_out + 255) / 256;
    hipLaunchKernelGGL(box_filter_kernel, dim3(blocks), dim3(256), 0, s, a, k, g, inv_khw);
    return hipGetLastError();
}

} // namespace xnor_hip
