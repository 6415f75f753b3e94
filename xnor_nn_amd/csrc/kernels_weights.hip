// Once-per-weight-set stage: sign-bit packing of the filters, alpha = mean |w| per filter
// and the per-output-pixel operation counts
// (reference src/bcast_binarize_weights.cpp:54-142), plus the float sign(w)*mean(w)
// helper (reference src/binarize_weights_float.cpp:3-25).  None of this is on the
// per-forward path, so the kernels favour exact reference order over speed.
#include <mutex>

#include "plan.hpp"

// Partial sums for callers that may not allocate (xnor_nn_hip_binarize_weights_float_noalloc):
// 256 floats per GPU for as long as the process lives.  In host code the name is only a
// handle; the device address comes from hipGetSymbolAddress, once per device
// (weights_float_scratch below), and kernels get that address as an argument.
static __device__ __align__(256) float scratch[256];

namespace xnor_hip {

namespace {

__device__ __forceinline__ size_t w_index(const Geometry &g, int oc, int ic, int kh, int kw) {
    if (g.w_fmt == xnor_nn_weights_format_oihw)
        return (((size_t)oc * g.ic + ic) * g.kh + kh) * g.kw + kw;
    return (((size_t)kh * g.kw + kw) * g.ic + ic) * g.oc + oc;
}

// One thread per packed word of the device layout [OCB][KH*KW][XW][Q].
// Channels >= IC (and whole filters >= OC) are written as ones so that
// popcount(xnor(0, 1)) adds nothing (reference src/bcast_binarize_weights.cpp:80-88).
__global__ __launch_bounds__(256)
void pack_weights_kernel(const float *__restrict__ w, uint32_t *__restrict__ bits,
        const Geometry g) {
    const int taps = g.kh * g.kw;
    const size_t total = (size_t)g.ocb * taps * g.xw * g.q;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int qi = (int)(i % g.q);
    const int j = (int)((i / g.q) % g.xw);
    const int tap = (int)((i / ((size_t)g.q * g.xw)) % taps);
    const int ob = (int)(i / ((size_t)g.q * g.xw * taps));
    const int oc = ob * g.q + qi;
    const int kh = tap / g.kw, kw = tap % g.kw;
    uint32_t word = 0;
    for (int b = 0; b < 32; b++) {
        const int c = 32 * j + b;
        uint32_t bit = 1u;
        if (oc < g.oc && c < g.ic)
            bit = (~__float_as_uint(w[w_index(g, oc, c, kh, kw)])) >> 31;
        word = (word << 1) | bit;
    }
    bits[i] = word;
}

// alpha[oc] = sum over (ic, kh, kw), nested in that order, of fl(|w| * chw)
// (reference src/bcast_binarize_weights.cpp:95-115): two kernels, one per weight layout.
//
// OIHW weights: a filter is one contiguous row of n = IC*KH*KW floats
// already in summation order.  One wave per ALPHA_F filters.  The rows are read ALPHA_CHUNK
// elements at a time with coalesced loads (all lanes read consecutive elements of one
// filter), passed through LDS and summed in order by lane f for filter f; the loads of the
// next chunk are in flight while the current one is summed.  Few filters per wave and long
// chunks: the sum is a serial chain either way, and this shape keeps many bytes in flight
// per wave and spreads the filters over many CUs.
constexpr int ALPHA_F = 8;
constexpr int ALPHA_CHUNK = 512;

__global__ __launch_bounds__(64)
void alpha_oihw_kernel(const float *__restrict__ w, float *__restrict__ alpha, const int oc_n,
        const int n, const float chw) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    // rows of ALPHA_CHUNK + 4 floats: 16-byte aligned, and the eight summing lanes start four
    // banks apart, so their 16-byte reads do not collide
    __shared__ __attribute__((aligned(16))) float tile[ALPHA_F][ALPHA_CHUNK + 4];
    constexpr int PER_LANE = ALPHA_CHUNK / 64;
    const int lane = threadIdx.x;
    const int f0 = blockIdx.x * ALPHA_F;
    const int nf = min(ALPHA_F, oc_n - f0);
    float acc = 0.f;
    float cur[ALPHA_F][PER_LANE], nxt[ALPHA_F][PER_LANE]; // element c0 + 64*u + lane of filter f
    auto fetch = [&](float (&v)[ALPHA_F][PER_LANE], int c0) {
#pragma unroll
        for (int f = 0; f < ALPHA_F; f++)
#pragma unroll
            for (int u = 0; u < PER_LANE; u++) {
                const int e = c0 + 64 * u + lane;
                v[f][u] = (f < nf && e < n) ? w[(size_t)(f0 + f) * n + e] : 0.f;
            }
    };
    fetch(cur, 0);
    for (int c0 = 0; c0 < n; c0 += ALPHA_CHUNK) {
        if (c0 + ALPHA_CHUNK < n) fetch(nxt, c0 + ALPHA_CHUNK);
#pragma unroll
        for (int f = 0; f < ALPHA_F; f++)
#pragma unroll
            for (int u = 0; u < PER_LANE; u++)
                tile[f][64 * u + lane] = __fmul_rn(__builtin_fabsf(cur[f][u]), chw);
        __syncthreads();
        // Elements past the end of the row were stored as +0, and s + 0 == s for these
        // non-negative sums, so whole batches can be read before they are added in order.
        // Two register sets of 16 values: one is read from LDS while the other is added.
        if (lane < ALPHA_F) {
            const v4f *row = reinterpret_cast<const v4f *>(tile[lane]);
            v4f a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; u++) a[u] = row[u];
            for (int j = 0; j < ALPHA_CHUNK / 16; j += 2) {
#pragma unroll
                for (int u = 0; u < 4; u++) b[u] = row[4 * (j + 1) + u];
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) acc = __fadd_rn(acc, a[u][e]);
                if (j + 2 < ALPHA_CHUNK / 16) {
#pragma unroll
                    for (int u = 0; u < 4; u++) a[u] = row[4 * (j + 2) + u];
                }
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int e = 0; e < 4; e++) acc = __fadd_rn(acc, b[u][e]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int f = 0; f < ALPHA_F; f++)
#pragma unroll
            for (int u = 0; u < PER_LANE; u++) cur[f][u] = nxt[f][u];
    }
    if (lane < nf) alpha[f0 + lane] = acc;
}

// Weights in which the filters are the contiguous index (HWIO): element t of
// the summation order (t = (ic*KH + kh)*KW + kw) of 64 consecutive filters is one coalesced
// load, a lane is a filter.  With one wave per 64 filters and a load per addition the kernel
// waited for memory 3456 times in a row (800 us for 256 x 3456 weights); here eight waves
// fetch the next ALPHA_T elements into registers while wave 0 adds the current ones, in
// order, out of LDS.
constexpr int ALPHA_T = 256;

__global__ __launch_bounds__(512)
void alpha_strided_kernel(const float *__restrict__ w, float *__restrict__ alpha,
        const Geometry g, const float chw, const FastDiv div_taps, const FastDiv div_kw) {
    __shared__ float tile[ALPHA_T][64];
    constexpr int PER_WAVE = ALPHA_T / 8;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int oc = blockIdx.x * 64 + lane;
    const int ocl = oc < g.oc ? oc : g.oc - 1;
    const int taps = g.kh * g.kw, n = g.ic * taps;
    float next[PER_WAVE];
    auto fetch = [&](int c) { // this wave's rows of chunk c: t = c*ALPHA_T + wave*PER_WAVE + u
#pragma unroll
        for (int u = 0; u < PER_WAVE; u++) {
            const int t = c * ALPHA_T + wave * PER_WAVE + u; // wave-uniform
            const int tc = t < n ? t : n - 1;
            const int ic = (int)div_taps.div((uint32_t)tc), tap = tc - ic * taps;
            const int kh = (int)div_kw.div((uint32_t)tap), kw = tap - kh * g.kw;
            const float v = w[w_index(g, ocl, ic, kh, kw)];
            next[u] = t < n ? __fmul_rn(__builtin_fabsf(v), chw) : 0.f; // +0 adds nothing
        }
    };
    auto publish = [&]() {
#pragma unroll
        for (int u = 0; u < PER_WAVE; u++) tile[wave * PER_WAVE + u][lane] = next[u];
    };
    const int chunks = (n + ALPHA_T - 1) / ALPHA_T;
    float acc = 0.f;
    fetch(0);
    publish();
    __syncthreads();
    for (int c = 0; c < chunks; c++) {
        if (c + 1 < chunks) fetch(c + 1);
        if (wave == 0) {
            for (int r = 0; r < ALPHA_T; r += 16) {
                float v[16];
#pragma unroll
                for (int u = 0; u < 16; u++) v[u] = tile[r + u][lane];
#pragma unroll
                for (int u = 0; u < 16; u++) acc = __fadd_rn(acc, v[u]);
            }
        }
        __syncthreads(); // the chunk has been added: its rows may be overwritten
        if (c + 1 < chunks) publish();
        __syncthreads();
    }
    if (wave == 0 && oc < g.oc) alpha[oc] = acc;
}

// opc[oh][ow] = IC * number of in-bounds taps (reference
// src/bcast_binarize_weights.cpp:126-142).
__global__ __launch_bounds__(256)
void op_count_kernel(int32_t *__restrict__ opc, const Geometry g) {
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= g.ohw) return;
    const int oh = p / g.ow, ow = p % g.ow;
    int taps = 0;
    for (int kh = 0; kh < g.kh; kh++) {
        const int ih = oh * g.sh - g.ph + kh;
        if (ih < 0 || ih >= g.ih) continue;
        for (int kw = 0; kw < g.kw; kw++) {
            const int iw = ow * g.sw - g.pw + kw;
            if (iw < 0 || iw >= g.iw) continue;
            taps++;
        }
    }
    opc[p] = taps * g.ic;
}

// Deterministic two-level sum for the float-weights helper (reference
// src/binarize_weights_float.cpp:14-20 adds every weight into one float; its OpenMP loop
// has no reduction clause, so only its one-thread result is defined, and a sum in another
// fixed order is within rounding of it).  Level 1: workgroup p of PARTS sums the contiguous
// slice p, thread t taking elements t, t + 256, ... of it (coalesced) and the 256 thread
// sums meeting in a fixed tree.  Level 2: every workgroup of the second kernel adds the PARTS
// partial sums in the same fixed tree, so all of them multiply by the same mean.
constexpr int PARTS = 256; // also the length of `scratch` above

__device__ __forceinline__ float tree_sum_256(float v, float *lds) {
    const int t = threadIdx.x;
    lds[t] = v;
    __syncthreads();
#pragma unroll
    for (int half = 128; half >= 1; half >>= 1) {
        if (t < half) lds[t] = __fadd_rn(lds[t], lds[t + half]);
        __syncthreads();
    }
    return lds[0];
}

__global__ __launch_bounds__(256)
void partial_sum_kernel(const float *__restrict__ from, float *__restrict__ parts,
        const size_t n) {
    __shared__ float lds[256];
    const size_t per = (n + PARTS - 1) / PARTS;
    const size_t lo = (size_t)blockIdx.x * per;
    const size_t hi = lo + per < n ? lo + per : n;
    float acc = 0.f;
    for (size_t i = lo + threadIdx.x; i < hi; i += 256) acc = __fadd_rn(acc, from[i]);
    const float sum = tree_sum_256(acc, lds);
    if (threadIdx.x == 0) parts[blockIdx.x] = sum;
}

__global__ __launch_bounds__(256)
void sign_times_mean_kernel(const float *__restrict__ from, float *__restrict__ to,
        const float *__restrict__ parts, const size_t n, const float inv_n) {
    __shared__ float lds[256];
    const float mean = __fmul_rn(tree_sum_256(parts[threadIdx.x], lds), inv_n);
    // four consecutive elements per thread
    const size_t i0 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
#pragma unroll
    for (int u = 0; u < 4; u++)
        if (i0 + u < n) to[i0 + u] = from[i0 + u] >= 0.f ? mean : -mean;
}

} // namespace

hipError_t launch_binarize_weights(const Geometry &g, const float *w, uint32_t *bits,
        float *alpha, int32_t *opc, hipStream_t s) {
    const size_t words = (size_t)g.ocb * g.kh * g.kw * g.xw * g.q;
    hipLaunchKernelGGL(pack_weights_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256),
            0, s, w, bits, g);
    const float chw = 1.f / (g.ic * g.kh * g.kw);
    if (g.w_fmt == xnor_nn_weights_format_oihw)
        hipLaunchKernelGGL(alpha_oihw_kernel, dim3((g.oc + ALPHA_F - 1) / ALPHA_F), dim3(64), 0,
                s, w, alpha,
                g.oc, g.ic * g.kh * g.kw, chw);
    else
        hipLaunchKernelGGL(alpha_strided_kernel, dim3((g.oc + 63) / 64), dim3(512), 0, s, w,
                alpha, g, chw, FastDiv::make((uint32_t)(g.kh * g.kw)),
                FastDiv::make((uint32_t)g.kw));
    hipLaunchKernelGGL(op_count_kernel, dim3((g.ohw + 255) / 256), dim3(256), 0, s, opc, g);
    return hipGetLastError();
}

int weights_float_parts() { return PARTS; }

// parts: PARTS floats of device memory.
hipError_t launch_weights_float(const float *from, float *to, size_t n, float *parts,
        hipStream_t s) {
    hipLaunchKernelGGL(partial_sum_kernel, dim3(PARTS), dim3(256), 0, s, from, parts, n);
    hipLaunchKernelGGL(sign_times_mean_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256),
            0, s, from, to, parts, n, 1.f / (float)n);
    return hipGetLastError();
}

// Device address of this GPU's copy of `scratch`, looked up on the first call on a device
// (with that device current) and kept.
hipError_t weights_float_scratch(float **out) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static float *addr[MAX_DEVICES];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (addr[dev] == nullptr) {
        float *p = nullptr;
        e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (p == nullptr) return hipErrorInvalidSymbol;
        addr[dev] = p;
    }
    *out = addr[dev];
    return hipSuccess;
}

} // namespace xnor_hip
