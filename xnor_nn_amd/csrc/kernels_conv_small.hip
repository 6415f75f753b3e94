// Stage 3 on the matrix cores for launches of few tiles (small batches): the same FP4
// implicit GEMM as kernels_conv_mfma.hip, cut the other way.
// Semantics: reference src/default/bcast_convolution_default.cpp:60-105.
//
// The large-launch kernel gives a workgroup 32*PS pixels x 256 filters and every wave all
// taps of its 64 filters: at minibatch 1 of AlexNet conv4 that is 6 workgroups on a chip of
// 256 compute units, each wave walking 54 steps one behind the other with the latency of a
// weight fetch between the groups.  Here a workgroup is one block of 32 pixels x ONE block of
// 32 filters, and its four waves split the (tap, channel step) sequence between them: 48
// workgroups for that problem, 13 or 14 matrix instructions per wave.  The partial sums are
// exact integers in FP32, so the four waves' accumulators add up to the same bits in any
// order; they meet in LDS and every wave scales and stores a quarter of the block.
//
// Nothing is hand-scheduled: a wave asks for its first weight fragments before it stages
// the input (they arrive meanwhile), keeps a ring of eight fragments in flight and leaves
// the waits to the compiler.
#include <cstdlib>

#include "plan.hpp"

namespace xnor_hip {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int SMALL_ROW_PAD = 16;     // spare bytes per LDS row, as in the large-launch kernel
constexpr int SMALL_TABLE_BYTES = 1024;
constexpr int SMALL_RING = 8;         // weight fragments in flight per wave
constexpr uint32_t SMALL_DROP = 0xFFFFFFF0u;

__device__ __forceinline__ v16f small_mfma_fp4(const v4i a, const v4i b, const v16f c) {
    const v8i a8 = {a.x, a.y, a.z, a.w, 0, 0, 0, 0};
    const v8i b8 = {b.x, b.y, b.z, b.w, 0, 0, 0, 0};
    // cbsz = blgp = 4: FP4 (E2M1) operands; zero scale operands select the unscaled form
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c, 4, 4, 0, 0, 0, 0);
}

// FP4 codes of eight channels from one byte of packed sign bits (bit 7 = first channel,
// set = sign bit clear = +1): nibble i = channel i, +1 -> 0x2, -1 -> 0xA.
__device__ __forceinline__ uint32_t small_fp4_of_byte(uint32_t byte) {
    uint32_t out = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
        out |= (((byte >> (7 - i)) & 1u) ? 0x2u : 0xAu) << (4 * i);
    return out;
}

// LDS: [table 1 KB][rows: zero row + max_rows rows of ks*32 + 16 bytes][mean|x| of the staged
// pixels + one slot of zero][partial sums: 4 waves x 12 registers x 64 lanes]
__global__ __launch_bounds__(256)
void conv_mfma_fp4_small_kernel(const uint32_t *__restrict__ xbits, const v4i *__restrict__ wfrag,
        const float *__restrict__ alpha, const float *__restrict__ kplane,
        float *__restrict__ dst, const Geometry g, const int max_rows, const int ks,
        const int subs, const uint32_t wfrag_bytes, const float *__restrict__ a_plane,
        float *__restrict__ k_out, const float inv_khw, const FastDiv div_xw) {
    extern __shared__ unsigned char smem[];
    uint32_t *table = reinterpret_cast<uint32_t *>(smem);
    unsigned char *rows = smem + SMALL_TABLE_BYTES;
    const int row_bytes = ks * 32 + SMALL_ROW_PAD;
    float *a_lds = reinterpret_cast<float *>(rows + (size_t)(1 + max_rows) * row_bytes);
    float *parts = a_lds + ((max_rows + 1 + 3) & ~3);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t block = blockIdx.x / (uint32_t)subs;
    const int sub = (int)(blockIdx.x - block * (uint32_t)subs); // 32-filter block
    const uint32_t p_first = block * 32u, p_limit = g.npix_out;
    const int taps = g.kh * g.kw, nsteps = taps * ks;
    // this wave's share of the steps
    const int s_lo = (wave * nsteps) / 4, s_hi = ((wave + 1) * nsteps) / 4;

    // ---- weight fragments: [32-filter block][tap][step][lane]; the first ring is asked for now
    const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<v4i *>(wfrag), 0, (int)wfrag_bytes, 0x00020000);
    const uint32_t wvoff = (uint32_t)lane * 16u;
    const uint32_t wbase = (uint32_t)sub * (uint32_t)nsteps * 1024u;
    auto fragment = [&](int s) { // a step past the wave's share reads outside the buffer: zeros
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wbuf,
                s < s_hi ? wvoff : SMALL_DROP, s < s_hi ? wbase + (uint32_t)s * 1024u : 0u, 0));
    };
    v4i ring[SMALL_RING];
#pragma unroll
    for (int i = 0; i < SMALL_RING; i++) ring[i] = fragment(s_lo + i);

    // the alphas of the four filters this lane will scale (registers 4*wave .. +3 of the block:
    // filters 8*wave + 4*(lane/32) + 0..3), asked for now so that the epilogue does not wait
    const int f0 = sub * 32 + 8 * wave + 4 * (lane >> 5);
    float al[4];
#pragma unroll
    for (int ii = 0; ii < 4; ii++) al[ii] = f0 + ii < g.oc ? alpha[f0 + ii] : 0.f;

    // ---- the block's pixels, one per lane (both halves of the wave hold the same 32)
    int lo, hi;
    tile_span(g, p_first, min(p_first + 32u, p_limit), lo, hi);
    const int nrows = min(hi - lo + 1, max_rows);
    const uint32_t pix = p_first + (lane & 31);
    const bool live = pix < p_limit;
    const uint32_t pc = live ? pix : p_limit - 1;
    const uint32_t img = g.div_ohw.div(pc), rem = pc - img * g.ohw;
    const int oh = (int)g.div_ow.div(rem), ow = (int)rem - oh * g.ow;
    const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw; // input pixel of tap (0,0)
    const int in0 = (int)(img * g.ihw) + ih0 * g.iw + iw0 - lo;
    auto run_of_bits = [](int first, int last) -> uint32_t { // bits first..last, clipped
        if (first < 0) first = 0;
        if (last > 31) last = 31;
        if (last < first) return 0u;
        return (0xFFFFFFFFu >> (31 - last)) & (0xFFFFFFFFu << first);
    };
    const uint32_t rowmask = live ? run_of_bits(-ih0, g.ih - 1 - ih0) : 0u;
    const uint32_t colmask = run_of_bits(-iw0, g.iw - 1 - iw0);
    // byte offsets into `rows`: the zero row, and the row of tap (0,0) of the lane's pixel
    // (the upper half of the wave reads the second 32 channels of a step)
    const int zero_off = (lane >> 5) * 16;
    const int base_off = zero_off + (1 + in0) * row_bytes;

    // ---- staging: table, zero row, mean|x|, FP4 rows
    const bool fuse_k = a_plane != nullptr; // uniform
    const float k_read = fuse_k ? 0.f : kplane[live ? pix : 0]; // asked for early
    table[tid] = small_fp4_of_byte(tid);
    for (int i = tid; i < row_bytes / 4; i += 256) reinterpret_cast<uint32_t *>(rows)[i] = 0;
    if (fuse_k) {
        for (int i = tid; i < nrows; i += 256) a_lds[i] = a_plane[lo + i];
        if (tid == 0) a_lds[max_rows] = 0.f;
    }
    const int nitems = nrows * g.xw;
    const uint32_t *run = xbits + (size_t)lo * g.xw;
    uint32_t word[4];
#pragma unroll
    for (int u = 0; u < 4; u++) word[u] = u * 256 + tid < nitems ? run[u * 256 + tid] : 0u;
    __syncthreads();
    auto expand = [&](int i, uint32_t w) { // item i of the run -> 32 FP4 codes of its row
        const int r = (int)div_xw.div((uint32_t)i), j = i - r * g.xw;
        v4i q;
        q.x = table[w >> 24];
        q.y = table[(w >> 16) & 0xFF];
        q.z = table[(w >> 8) & 0xFF];
        q.w = table[w & 0xFF];
        *reinterpret_cast<v4i *>(rows + (size_t)(1 + r) * row_bytes + j * 16) = q;
    };
#pragma unroll
    for (int u = 0; u < 4; u++)
        if (u * 256 + tid < nitems) expand(u * 256 + tid, word[u]);
    for (int i = 1024 + tid; i < nitems; i += 256) expand(i, run[i]);
    __syncthreads();

    // ---- this wave's steps: two accumulators in turn (the sums are exact, any order)
    v16f acc0, acc1;
#pragma unroll
    for (int i = 0; i < 16; i++) acc0[i] = acc1[i] = 0.f;
    int tap = s_lo / ks, cs = s_lo - tap * ks; // uniform
    auto row_of_tap = [&](int t) {
        const int kh = t / g.kw, kw = t - kh * g.kw;
        const uint32_t ok = (rowmask >> kh) & (colmask >> kw) & 1u;
        return ok ? base_off + (kh * g.iw + kw) * row_bytes : zero_off;
    };
    int rowoff = row_of_tap(tap < taps ? tap : 0);
    for (int s = s_lo; s < s_hi; s += SMALL_RING) {
#pragma unroll
        for (int i = 0; i < SMALL_RING; i++) {
            if (s + i < s_hi) { // uniform
                const v4i b = *reinterpret_cast<const v4i *>(rows + rowoff + cs * 32);
                if (i & 1) acc1 = small_mfma_fp4(ring[i], b, acc1);
                else acc0 = small_mfma_fp4(ring[i], b, acc0);
                ring[i] = fragment(s + i + SMALL_RING);
                if (++cs == ks) {
                    cs = 0;
                    tap++;
                    rowoff = row_of_tap(tap < taps ? tap : 0);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) acc0[i] += acc1[i];

    // ---- the four partial sums meet in LDS: wave w keeps registers 4w .. 4w+3 (filters
    // 8w + 4*(lane/32) + 0..3 of the block) and gets the other waves' values for them
#pragma unroll
    for (int q = 0; q < 4; q++) {
        if (q == wave) continue; // uniform
        const int slot = wave < q ? wave : wave - 1; // 0..2 among the three givers of quarter q
#pragma unroll
        for (int ii = 0; ii < 4; ii++)
            parts[((q * 3 + slot) * 4 + ii) * 64 + lane] = acc0[4 * q + ii];
    }
    // ---- K of the lane's pixel, while the other waves finish their steps: the box filter's
    // own order (in-bounds taps, row-major, every product rounded, then added: reference
    // src/bcast_calculate_k.cpp:69-85), unless it came from the K plane
    float kv = k_read;
    if (fuse_k) {
        for (int kh = 0; kh < g.kh; kh++)
            for (int kw = 0; kw < g.kw; kw++) {
                const bool ok = (rowmask >> kh) & (colmask >> kw) & 1u;
                // a tap outside the image reads the slot that holds zero: + 0 changes nothing
                kv = __fadd_rn(kv, __fmul_rn(a_lds[ok ? in0 + kh * g.iw + kw : max_rows], inv_khw));
            }
        if (sub == 0 && wave == 0 && lane < 32 && live) k_out[pix] = kv;
    }

    __syncthreads();
    float sum[4];
#pragma unroll
    for (int ii = 0; ii < 4; ii++) {
        float v = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (q == wave) v = acc0[4 * q + ii]; // uniform
#pragma unroll
        for (int slot = 0; slot < 3; slot++) v += parts[((wave * 3 + slot) * 4 + ii) * 64 + lane];
        sum[ii] = v; // = 2*popc - n, exactly
    }

    // ---- epilogue: dst = fl(fl((float)(2*popc - n) * alpha) * k), every product rounded
    const bool nchw = g.dst_fmt == xnor_nn_data_format_nchw;
#pragma unroll
    for (int ii = 0; ii < 4; ii++) {
        const int f = f0 + ii;
        if (f < g.oc && live) {
            const float out = __fmul_rn(__fmul_rn(sum[ii], al[ii]), kv);
            const size_t at = nchw ? ((size_t)img * g.oc + f) * g.ohw + rem
                                   : (size_t)pix * g.oc + f;
            dst[at] = out;
        }
    }
}

} // namespace

// Which problems take this kernel: one channel part, no tap pairing (the fragment layout of
// paired taps is walked differently), and few enough (pixel block, filter block) pairs that
// the large-launch kernel would leave most of the chip idle.  XNOR_NN_HIP_MFMA_SMALL=0|1
// overrides the size rule (for measurements).
bool small_kernel_applies(const Geometry &g, int *rows_out, uint32_t *lds_out) {
    if (!g.use_mfma || g.mfma_pair || g.mfma_parts > 1) return false;
    const uint32_t blocks = (g.npix_out + 31) / 32;
    const uint32_t subs = (uint32_t)(g.oc + 31) / 32;
    // measured on AlexNet conv4 (8 filter blocks): minibatch 1 / 2 / 4 / 8, i.e. 48 to 344
    // pairs, 6.2 / 6.2 / 6.3 / 7.1 us against 7.4 / 7.5 / 7.6 / 7.9 us for the large-launch
    // kernel; minibatch 16 (680 pairs) 8.4 against 8.1 us, minibatch 32 13.5 against 8.7 us
    // With long walks (48 steps and more: conv4's 54, 72 for 512 channels) the split of the steps
    // over four waves still pays at up to two pairs per compute unit: conv4 minibatch 12 (512
    // pairs) 7.2 against 7.6 us, 512 -> 512 channels on 28x28 minibatch 1 (400 pairs) 8.0 against
    // 8.6, on 14x14 minibatch 4 7.6 against 8.4, on 7x7 minibatch 20 (496 pairs) 7.5 against
    // 8.5; with 36 steps (256 channels) the large-launch kernel is ahead there (6.9 against 7.2).
    const uint64_t pairs = (uint64_t)blocks * subs;
    const int walk = g.kh * g.kw * g.mfma_steps;
    bool take = pairs <= (uint64_t)g.cus + (uint64_t)g.cus / 2
        || (walk >= 48 && pairs <= 2 * (uint64_t)g.cus);
    // a tile size, tile mix or persistent workgroups asked for by name mean the other kernel
    if (getenv("XNOR_NN_HIP_MFMA_PS") || getenv("XNOR_NN_HIP_MFMA_MIX")
            || getenv("XNOR_NN_HIP_MFMA_PERSIST"))
        take = false;
    if (const char *e = getenv("XNOR_NN_HIP_MFMA_SMALL")) take = e[0] == '1';
    if (!take) return false;
    // input pixels a block of 32 output pixels touches at most (blocks start at multiples of 32)
    int most = 1;
    const uint32_t look = blocks < (uint32_t)g.ohw + 1 ? blocks : (uint32_t)g.ohw + 1;
    auto see = [&](uint32_t b) {
        int lo, hi;
        tile_span(g, b * 32u, b * 32u + 32u < g.npix_out ? b * 32u + 32u : g.npix_out, lo, hi);
        if (hi - lo + 1 > most) most = hi - lo + 1;
    };
    for (uint32_t b = 0; b < look; b++) see(b);
    see(blocks - 1);
    const size_t row_bytes = (size_t)g.mfma_steps * 32 + SMALL_ROW_PAD;
    const size_t lds = SMALL_TABLE_BYTES + (1 + (size_t)most) * row_bytes
        + (((size_t)most + 1 + 3) & ~(size_t)3) * 4 + 4 * 3 * 4 * 64 * 4;
    if (lds > 64 * 1024) return false;
    if (rows_out) *rows_out = most;
    if (lds_out) *lds_out = (uint32_t)lds;
    return true;
}

hipError_t launch_convolution_small(const Geometry &g, const uint32_t *xbits,
        const uint32_t *wfrag, const float *alpha, const float *k, float *dst,
        const float *a_or_null, float *k_out, hipStream_t s, const KernelEvents &ev) {
    const uint32_t blocks = (g.npix_out + 31) / 32;
    const int subs = (g.oc + 31) / 32;
    launch_kernel(conv_mfma_fp4_small_kernel, dim3(blocks * (uint32_t)subs), dim3(256),
            (size_t)g.mfma_small_lds, s, ev, xbits, reinterpret_cast<const v4i *>(wfrag), alpha, k,
            dst, g, g.mfma_small_rows, g.mfma_steps, subs, g.mfma_wbytes, a_or_null, k_out,
            1.f / g.kh / g.kw, FastDiv::make((uint32_t)g.xw));
    return hipGetLastError();
}

} // namespace xnor_hip
