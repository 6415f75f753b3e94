"""Randomised parity run on the GPU, outside the pytest suite: python tests/stress_random.py SEED SECONDS

Draws convolution problems (channel counts around the 32/64/1024 boundaries up to 2048,
kernels 1..9, strides 1..4, paddings 0..4, images up to 43 x 43, every layout combination,
inputs with exact zeros of both signs) until the time is up and compares dst and the raw
popcounts with the C oracle bit for bit.  Prints the case before running it and, at the end,
how many cases each kernel variant took."""
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
import numpy as np
import checkers, shapes
from util import oracle_shape
from xnor_nn_amd import Convolution, capi, synth
oracle = checkers.Oracle()
rng = np.random.default_rng(int(sys.argv[1]) if len(sys.argv) > 1 else 1)
budget = float(sys.argv[2]) if len(sys.argv) > 2 else 60
t_end = time.time() + budget
n = 0; names = {}
while time.time() < t_end:
    kh, kw = int(rng.integers(1, 10)), int(rng.integers(1, 10))
    ph, pw = int(rng.integers(0, 5)), int(rng.integers(0, 5))
    sh, sw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
    ih = int(rng.integers(max(1, kh - 2 * pw), 44)); iw = int(rng.integers(max(1, kw - 2 * pw), 44))
    ic = int(rng.choice([1, 3, 4, 31, 32, 33, 64, 65, 96, 100, 128, 160, 200, 256, 257, 320, 384, 448, 512, 513, 640, 700, 1000, 1024, 1028, 1500, 2048]))
    oc = int(rng.choice([1, 7, 16, 31, 32, 33, 64, 65, 100, 128, 130, 256, 260, 384, 512, 600]))
    mb = int(rng.integers(1, 7))
    oh = (ih + 2 * pw - kh) // sh + 1; ow = (iw + 2 * pw - kw) // sw + 1
    if oh < 1 or ow < 1 or ih + 2 * ph < kh: continue
    if mb * ic * ih * iw > 6e6 or mb * oc * oh * ow > 6e6 or oc * ic * kh * kw > 6e6: continue
    if mb * oc * oh * ow * ic * kh * kw > 4e10: continue
    fmts = (int(rng.choice([capi.FMT_NCHW, capi.FMT_NHWC])), int(rng.choice([capi.FMT_OIHW, capi.FMT_HWIO])), int(rng.choice([capi.FMT_NCHW, capi.FMT_NHWC])))
    d = dict(mb=mb, ic=ic, oc=oc, ih=ih, iw=iw, kh=kh, kw=kw, sh=sh, sw=sw, ph=ph, pw=pw)
    x = synth.normal(1000 + n, mb * ic * ih * iw).reshape(mb, ic, ih, iw); x.ravel()[::7] = 0.0; x.ravel()[3::11] = -0.0
    w = synth.normal(5000 + n, oc * ic * kh * kw, 0.05).reshape(oc, ic, kh, kw)
    xs = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if fmts[0] == capi.FMT_NHWC else x
    ws = np.ascontiguousarray(w.transpose(2, 3, 1, 0)) if fmts[1] == capi.FMT_HWIO else w
    s = oracle_shape(oracle, d, fmts)
    want = oracle.forward(s, xs, ws)
    print('case', n, d, fmts, flush=True)
    conv = Convolution(capi.ALGORITHM_BCAST, fmts[0], fmts[1], fmts[2], mb, oc, ic, ih, iw, kh, kw, sh, sw, ph, pw, ws)
    dst = np.empty(want['dst'].shape, np.float32)
    conv.forward(xs, dst)
    kn = (conv.kernel_name(0).split('<')[0] + '<' + conv.kernel_name(0).split('<')[1].split(',')[0], conv.kernel_name(2))
    names[kn] = names.get(kn, 0) + 1
    ok = np.array_equal(dst.view(np.uint32), want['dst'].view(np.uint32)) and np.array_equal(conv.forward_popcount(), want['popc'])
    conv.close()
    if not ok:
        print('MISMATCH', d, fmts, kn); sys.exit(1)
    n += 1
print('cases', n, 'all bit-exact')
for k, v in sorted(names.items(), key=lambda kv: -kv[1]): print('  ', v, k)
