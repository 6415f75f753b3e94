/* Runs the C oracle (oracle/xnor_oracle.c, compiled into this program) under the address and
 * undefined-behaviour sanitizers over small and ragged shapes in every layout, with exactly
 * sized heap buffers: an index that leaves a tensor, a shift by the word size or a signed
 * overflow in the restatement ends the program with a report.  Also checks one invariant
 * that needs no reference: an all-ones input against all-ones weights gives
 * dst = n * 1 * taps/(KH*KW) exactly where the divisions are exact.
 * Built and run by tests/test_oracle.py (host only). */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "../oracle/xnor_oracle.c"

static float *floats(size_t n, unsigned seed, int ones) {
    float *p = malloc(n * sizeof(float) + (n == 0));
    for (size_t i = 0; i < n; i++) {
        seed = seed * 1664525u + 1013904223u;
        p[i] = ones ? 1.f : ((int)(seed >> 8) % 2001 - 1000) / 1000.f;
        if (!ones && i % 7 == 3) p[i] = 0.f;
        if (!ones && i % 11 == 5) p[i] = -0.f;
    }
    return p;
}

static int run(int src_fmt, int w_fmt, int dst_fmt, int mb, int oc, int ic, int ih, int iw,
        int kh, int kw, int sh, int sw, int ph, int pw, int ones) {
    xo_shape_t s;
    xo_shape_init(&s, src_fmt, w_fmt, dst_fmt, mb, oc, ic, ih, iw, kh, kw, sh, sw, ph, pw);
    if (s.oh < 1 || s.ow < 1) return 0;
    const int oci = 32 / xo_bici(&s);
    if (oc % oci) return 0; /* the reference's own restriction on its packed layout */
    const size_t nx = (size_t)mb * ic * ih * iw, nw = (size_t)oc * ic * kh * kw;
    const size_t nout = (size_t)mb * oc * s.oh * s.ow;
    float *x = floats(nx, 1u + ic, ones), *w = floats(nw, 7u + oc, ones);
    uint8_t *bx = malloc(xo_bin_src_bytes(&s)), *bw = malloc(xo_bin_weights_bytes(&s, oci));
    float *a = malloc((size_t)mb * ih * iw * 4), *k = malloc((size_t)mb * s.oh * s.ow * 4);
    float *alpha = malloc((size_t)oc * 4), *dst = malloc(nout * 4), *wf = malloc(nw * 4 + 4);
    int32_t *opc = malloc((size_t)s.oh * s.ow * 4), *popc = malloc(nout * 4);
    xo_binarize_data(&s, x, bx);
    xo_calculate_k(&s, x, a, k);
    xo_binarize_weights(&s, oci, w, bw, alpha, opc);
    xo_convolution(&s, oci, bx, bw, alpha, k, opc, popc, dst);
    xo_binarize_weights_float(&s, w, wf);
    int bad = 0;
    if (ones) { /* every valid tap agrees on every channel */
        for (size_t i = 0; i < nout && !bad; i++) {
            /* the raw accumulators are laid out [mb][oc][oh][ow] whatever dst_fmt says */
            if (popc[i] != opc[i % ((size_t)s.oh * s.ow)]) bad = 1;
        }
    }
    free(x); free(w); free(bx); free(bw); free(a); free(k); free(alpha); free(dst); free(wf);
    free(opc); free(popc);
    return bad;
}

int main(void) {
    static const int shapes[][11] = { /* mb oc ic ih iw kh kw sh sw ph pw */
        {1, 16, 1, 1, 1, 1, 1, 1, 1, 0, 0}, {2, 16, 3, 4, 6, 3, 3, 1, 1, 1, 1},
        {1, 32, 33, 6, 6, 5, 5, 1, 1, 2, 2}, {3, 16, 40, 9, 11, 3, 3, 2, 2, 1, 1},
        {1, 16, 70, 7, 5, 3, 3, 2, 3, 1, 1}, {2, 48, 96, 13, 13, 5, 5, 1, 1, 2, 2},
        {1, 16, 24, 12, 12, 7, 7, 3, 3, 3, 3}, {1, 8, 3700, 3, 3, 3, 3, 1, 1, 1, 1},
        {2, 16, 64, 5, 9, 1, 1, 1, 1, 0, 0}, {1, 16, 16, 8, 8, 4, 4, 1, 1, 0, 0},
        {1, 16, 8, 10, 10, 3, 3, 1, 1, 0, 1}, /* ph != pw: both extents follow pw */
    };
    int cases = 0, bad = 0;
    for (size_t i = 0; i < sizeof shapes / sizeof shapes[0]; i++)
        for (int f = 0; f < 8; f++)
            for (int ones = 0; ones < 2; ones++) {
                const int *t = shapes[i];
                bad += run(f & 1 ? XO_NHWC : XO_NCHW, f & 2 ? XO_HWIO : XO_OIHW,
                        f & 4 ? XO_NHWC : XO_NCHW, t[0], t[1], t[2], t[3], t[4], t[5], t[6],
                        t[7], t[8], t[9], t[10], ones);
                cases++;
            }
    printf("%d cases, %d bad\n", cases, bad);
    return bad != 0;
}
