/*
 * CPU oracle for the XNOR-Net bcast forward path.  TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of what mistler/xnor_nn computes on its bcast path, written to be
 * read next to the reference and used as the checker in tests/, in the smoke check and as
 * the optional CPU-baseline leg of the benchmark.  Nothing in the shipped library links,
 * loads or calls this file; the product path is HIP only.
 *
 * Pinning status (what proves each function, apart from this text):
 *   xo_binarize_data     byte-for-byte against the compiled reference (oracle/_ref) on the
 *                        reference's 94 test shapes and the five benchmark shapes; closed
 *                        form bit = !signbit under the index formula of the reference's
 *                        own checker (reference test/gtest/common.hpp:68-98); +0/-0/NaN.
 *   xo_calculate_k       bit-for-bit against oracle/_ref; known answers a == 1,
 *                        k = {4,6,4,6,9,6,4,6,4}/9 (reference
 *                        test/gtest/test_data_bin_reference.cpp:43-53); float64 means.
 *   xo_binarize_weights  byte-for-byte against oracle/_ref (bits incl. the all-ones tail,
 *                        alpha, operation counts); reference checker formula
 *                        (reference test/gtest/common.hpp:101-144); alpha = {1,1}
 *                        (reference test/gtest/test_weights_bin_reference.cpp:50);
 *                        sum(op_c) = IC * in-bounds taps.
 *   xo_convolution       bit-for-bit dst against oracle/_ref (AVX kernels); the 18-value
 *                        known-answer forward (reference
 *                        test/gtest/test_convolution_reference_forward.cpp:58-73);
 *                        brute-force +-1 dot products from the raw floats.
 *   xo_binarize_weights_float
 *                        bit-for-bit against oracle/_ref run on ONE OpenMP thread (the
 *                        reference adds into a shared variable from a parallel loop without
 *                        a reduction, reference src/binarize_weights_float.cpp:17-19, so
 *                        only its one-thread result is defined); closed forms (all ones,
 *                        alternating signs, -0.0 counts as >= 0); float64 mean.
 * No function is "parity unpinned".
 *
 * Floating point: every product and every sum is rounded to float separately and in the
 * reference's order.  Build with -ffp-contract=off and without -ffast-math; the
 * reference's translation units for these stages are compiled for baseline x86-64,
 * which has no fused multiply-add (reference src/CMakeLists.txt:60-69).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { XO_NCHW = 0, XO_NHWC = 1, XO_OIHW = 2, XO_HWIO = 3 };

typedef struct {
    int mb, ic, ih, iw;
    int oc, oh, ow;
    int kh, kw, sh, sw, ph, pw;
    int src_fmt, w_fmt, dst_fmt;
} xo_shape_t;

static int div_up(int a, int b) { return (a + b - 1) / b; }

/* Output extent.  The reference computes BOTH oh and ow with pw
 * (reference src/common_convolution.cpp:16-17, src/utils/utils.hpp:7-13). */
void xo_shape_init(xo_shape_t *s, int src_fmt, int w_fmt, int dst_fmt,
        int mb, int oc, int ic, int ih, int iw,
        int kh, int kw, int sh, int sw, int ph, int pw) {
    s->mb = mb; s->ic = ic; s->ih = ih; s->iw = iw; s->oc = oc;
    s->kh = kh; s->kw = kw; s->sh = sh; s->sw = sw; s->ph = ph; s->pw = pw;
    s->oh = (ih + 2 * pw - kh) / sh + 1;
    s->ow = (iw + 2 * pw - kw) / sw + 1;
    s->src_fmt = src_fmt; s->w_fmt = w_fmt; s->dst_fmt = dst_fmt;
}

/* Bytes per packed word: int16 words while ic*kh*kw < 32767, else int32 words
 * (reference src/implementation.cpp:17-22 tries Short first;
 *  src/convolution_traits.hpp:29-56). */
int xo_bici(const xo_shape_t *s) {
    return (s->ic * s->kh * s->kw < 32767) ? 2 : 4;
}

/* Blocking (reference src/bcast_convolution.hpp:51-70). */
int xo_bic(const xo_shape_t *s) { return div_up(s->ic, 8); }
int xo_abic(const xo_shape_t *s) {
    int b = xo_bici(s);
    return div_up(xo_bic(s), b) * b;
}
int xo_ico(const xo_shape_t *s) { return div_up(div_up(s->ic, xo_bici(s)), 8); }
/* oci = vector bytes / bici on the CPU (16 or 8 for 256-bit AVX); a free parameter here. */
int xo_oco(const xo_shape_t *s, int oci) { return div_up(s->oc, oci); }

size_t xo_bin_src_bytes(const xo_shape_t *s) {
    return (size_t)s->mb * s->ih * s->iw * xo_abic(s);
}
size_t xo_bin_weights_bytes(const xo_shape_t *s, int oci) {
    return (size_t)xo_oco(s, oci) * s->kh * s->kw * xo_ico(s) * oci * xo_bici(s);
}

static size_t src_index(const xo_shape_t *s, int mb, int c, int h, int w) {
    if (s->src_fmt == XO_NCHW)
        return (((size_t)mb * s->ic + c) * s->ih + h) * s->iw + w;
    return (((size_t)mb * s->ih + h) * s->iw + w) * s->ic + c;
}

static size_t w_index(const xo_shape_t *s, int oc, int ic, int kh, int kw) {
    if (s->w_fmt == XO_OIHW)
        return (((size_t)oc * s->ic + ic) * s->kh + kh) * s->kw + kw;
    return (((size_t)kh * s->kw + kw) * s->ic + ic) * s->oc + oc;
}

static unsigned sign_clear(const float *p) {
    uint32_t u;
    memcpy(&u, p, 4);
    return (~u) >> 31; /* 1 when the IEEE sign bit is 0: +0 -> 1, -0 -> 0 */
}

/* Stage 1 (reference src/bcast_binarize_data.cpp:43-73).
 * out[((mb*IH+ih)*IW+iw)*ABIC + b], bit (7-j) = sign-clear of channel 8b+j;
 * channels >= IC and the bytes BIC..ABIC-1 are 0. */
void xo_binarize_data(const xo_shape_t *s, const float *x, uint8_t *out) {
    const int BIC = xo_bic(s), ABIC = xo_abic(s);
#pragma omp parallel for collapse(2) schedule(static)
    for (int mb = 0; mb < s->mb; mb++)
    for (int ih = 0; ih < s->ih; ih++)
    for (int iw = 0; iw < s->iw; iw++) {
        uint8_t *px = out + (((size_t)mb * s->ih + ih) * s->iw + iw) * ABIC;
        for (int b = 0; b < ABIC; b++) {
            unsigned byte = 0;
            for (int j = 0; j < 8; j++) {
                int c = 8 * b + j;
                unsigned bit = (b < BIC && c < s->ic)
                    ? sign_clear(x + src_index(s, mb, c, ih, iw)) : 0u;
                byte = (byte << 1) | bit;
            }
            px[b] = (uint8_t)byte;
        }
    }
}

/* Stage 2 (reference src/bcast_calculate_k.cpp:42-85).
 * a = sum over channels, in order, of fl(|x| * C), C = 1.f/IC;
 * k = sum over in-bounds taps, row-major, of fl(a * KHW), KHW = (1.f/KH)/KW. */
void xo_calculate_k(const xo_shape_t *s, const float *x, float *a, float *k) {
    const float C = 1.f / s->ic;
    const float KHW = 1.f / s->kh / s->kw;
#pragma omp parallel for collapse(2) schedule(static)
    for (int mb = 0; mb < s->mb; mb++)
    for (int ih = 0; ih < s->ih; ih++)
    for (int iw = 0; iw < s->iw; iw++) {
        float acc = 0.f;
        for (int c = 0; c < s->ic; c++) {
            float t = fabsf(x[src_index(s, mb, c, ih, iw)]) * C;
            acc = acc + t;
        }
        a[((size_t)mb * s->ih + ih) * s->iw + iw] = acc;
    }
#pragma omp parallel for collapse(2) schedule(static)
    for (int mb = 0; mb < s->mb; mb++)
    for (int oh = 0; oh < s->oh; oh++)
    for (int ow = 0; ow < s->ow; ow++) {
        float acc = 0.f;
        for (int kh = 0; kh < s->kh; kh++)
        for (int kw = 0; kw < s->kw; kw++) {
            int ih = oh * s->sh - s->ph + kh;
            int iw = ow * s->sw - s->pw + kw;
            if (ih < 0 || iw < 0 || ih >= s->ih || iw >= s->iw) continue;
            float t = a[((size_t)mb * s->ih + ih) * s->iw + iw] * KHW;
            acc = acc + t;
        }
        k[((size_t)mb * s->oh + oh) * s->ow + ow] = acc;
    }
}

/* Stage 3 (reference src/bcast_binarize_weights.cpp:54-142).
 * bits : out[((((oco*KH+kh)*KW+kw)*ICO+ico)*OCI+oci)*BICI+b] holds channels
 *        (ico*BICI+b)*8 .. +7 of filter oco*OCI+oci, MSB first; channels >= IC are 1.
 * alpha: sum over (ic, kh, kw), nested in that order, of fl(|w| * chw), chw = 1.f/(IC*KH*KW).
 * opc  : IC * number of in-bounds taps of output pixel (oh, ow). */
void xo_binarize_weights(const xo_shape_t *s, int oci_n, const float *w,
        uint8_t *out, float *alpha, int32_t *opc) {
    const int BICI = xo_bici(s), ICO = xo_ico(s), OCO = xo_oco(s, oci_n);
#pragma omp parallel for collapse(2) schedule(static)
    for (int oco = 0; oco < OCO; oco++)
    for (int kh = 0; kh < s->kh; kh++)
    for (int kw = 0; kw < s->kw; kw++)
    for (int ico = 0; ico < ICO; ico++)
    for (int oci = 0; oci < oci_n; oci++)
    for (int b = 0; b < BICI; b++) {
        unsigned byte = 0;
        int oc = oco * oci_n + oci;
        for (int j = 0; j < 8; j++) {
            int c = (ico * BICI + b) * 8 + j;
            unsigned bit = (c < s->ic && oc < s->oc)
                ? sign_clear(w + w_index(s, oc, c, kh, kw)) : 1u;
            byte = (byte << 1) | bit;
        }
        out[((((size_t)(oco * s->kh + kh) * s->kw + kw) * ICO + ico) * oci_n + oci) * BICI + b]
            = (uint8_t)byte;
    }

    const float chw = 1.f / (s->ic * s->kh * s->kw);
#pragma omp parallel for schedule(static)
    for (int oc = 0; oc < s->oc; oc++) {
        float acc = 0.f;
        for (int ic = 0; ic < s->ic; ic++)
        for (int kh = 0; kh < s->kh; kh++)
        for (int kw = 0; kw < s->kw; kw++) {
            float t = fabsf(w[w_index(s, oc, ic, kh, kw)]) * chw;
            acc = acc + t;
        }
        alpha[oc] = acc;
    }

    for (int oh = 0; oh < s->oh; oh++)
    for (int ow = 0; ow < s->ow; ow++) {
        int n = 0;
        for (int kh = 0; kh < s->kh; kh++)
        for (int kw = 0; kw < s->kw; kw++) {
            int ih = oh * s->sh - s->ph + kh;
            int iw = ow * s->sw - s->pw + kw;
            if (ih < 0 || iw < 0 || ih >= s->ih || iw >= s->iw) continue;
            n += s->ic;
        }
        opc[oh * s->ow + ow] = n;
    }
}

static uint32_t load_word(const uint8_t *p, int bici) {
    if (bici == 2) { uint16_t v; memcpy(&v, p, 2); return v; }
    uint32_t v; memcpy(&v, p, 4); return v;
}

/* Stage 4 (reference src/default/bcast_convolution_default.cpp:60-105; the AVX, SSE and
 * NEON kernels compute the same values).  For every output element:
 *   popc = sum over in-bounds taps and packed words of popcount(~(src ^ weights)),
 *          taken on BICI-byte words; out-of-bounds taps are skipped;
 *   dst  = fl(fl((float)(2*popc - opc[oh,ow]) * alpha[oc]) * k[mb,oh,ow]).
 * popc (optional) receives the raw accumulators as [mb][oc][oh][ow]. */
void xo_convolution(const xo_shape_t *s, int oci_n,
        const uint8_t *bsrc, const uint8_t *bw,
        const float *alpha, const float *k, const int32_t *opc,
        int32_t *popc, float *dst) {
    const int BICI = xo_bici(s), ICO = xo_ico(s), OCO = xo_oco(s, oci_n);
    const uint32_t wmask = (BICI == 2) ? 0xFFFFu : 0xFFFFFFFFu;
#pragma omp parallel for collapse(3) schedule(static)
    for (int mb = 0; mb < s->mb; mb++)
    for (int oco = 0; oco < OCO; oco++)
    for (int oh = 0; oh < s->oh; oh++)
    for (int ow = 0; ow < s->ow; ow++)
    for (int oci = 0; oci < oci_n; oci++) {
        const int oc = oco * oci_n + oci;
        if (oc >= s->oc) continue;
        int acc = 0;
        for (int kh = 0; kh < s->kh; kh++)
        for (int kw = 0; kw < s->kw; kw++) {
            int ih = oh * s->sh - s->ph + kh;
            int iw = ow * s->sw - s->pw + kw;
            if (ih < 0 || iw < 0 || ih >= s->ih || iw >= s->iw) continue;
            const uint8_t *sp = bsrc
                + (((size_t)mb * s->ih + ih) * s->iw + iw) * ICO * BICI;
            const uint8_t *wp = bw
                + ((size_t)(oco * s->kh + kh) * s->kw + kw) * ICO * oci_n * BICI;
            for (int ico = 0; ico < ICO; ico++) {
                uint32_t a = load_word(sp + (size_t)ico * BICI, BICI);
                uint32_t b = load_word(wp + ((size_t)ico * oci_n + oci) * BICI, BICI);
                acc += __builtin_popcount((~(a ^ b)) & wmask);
            }
        }
        size_t pix = ((size_t)mb * s->oh + oh) * s->ow + ow;
        size_t di = (s->dst_fmt == XO_NCHW)
            ? (((size_t)mb * s->oc + oc) * s->oh + oh) * s->ow + ow
            : pix * s->oc + oc;
        if (popc)
            popc[(((size_t)mb * s->oc + oc) * s->oh + oh) * s->ow + ow] = acc;
        if (dst) {
            float v = (float)(acc * 2 - opc[oh * s->ow + ow]);
            v = v * alpha[oc];
            v = v * k[pix];
            dst[di] = v;
        }
    }
}

/* Float "binarized" weights for a framework's backward pass
 * (reference src/binarize_weights_float.cpp:3-25), in the order one thread runs it:
 *   alpha = fl(sum over i in index order of from[i]) -- the weights themselves, not |w| --
 *   alpha = fl(alpha * cckhw), cckhw = 1.f / elems;
 *   to[i] = fl((from[i] >= 0.f ? 1.f : -1.f) * alpha)   (-0.0f compares >= 0). */
void xo_binarize_weights_float(const xo_shape_t *s, const float *from, float *to) {
    const int elems = s->oc * s->ic * s->kh * s->kw;
    const float cckhw = 1.f / elems;
    float alpha = 0.f;
    for (int i = 0; i < elems; i++) alpha += from[i];
    alpha *= cckhw;
    for (int i = 0; i < elems; i++) to[i] = (from[i] >= .0f ? 1.f : -1.f) * alpha;
}
