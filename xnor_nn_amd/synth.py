"""Bit-reproducible synthetic tensors for the binary-convolution workloads.

The generator is a counter-based integer hash (the splitmix64 finaliser) evaluated per
flat element index, so a tensor does not depend on the host, on thread counts or on any
libm: normal deviates are Irwin-Hall sums of twelve 16-bit uniforms (exact in float32),
scaled by one float32 multiply.  The same (seed, shape) always yields the same bits, which
is what lets committed digests stand in for the reference's outputs.
"""
import numpy as np

_GOLD = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)

SEED_SRC = 1234
SEED_WEIGHTS = 4321


def _mix(counter):
    """splitmix64 output function on an array of uint64 counters."""
    z = counter.copy()
    z ^= z >> np.uint64(30)
    z *= _M1
    z ^= z >> np.uint64(27)
    z *= _M2
    z ^= z >> np.uint64(31)
    return z


def _hash(seed, idx, lane, lanes):
    with np.errstate(over="ignore"):
        ctr = (idx * np.uint64(lanes) + np.uint64(lane + 1)) * _GOLD + np.uint64(seed)
        return _mix(ctr)


def normal(seed, n, sigma=1.0, chunk=1 << 22):
    """n float32 values ~ N(0, sigma^2): ((sum of 12 u16) - 393210) * 2^-16 * sigma."""
    out = np.empty(n, dtype=np.float32)
    s32 = np.float32(sigma)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        idx = np.arange(lo, hi, dtype=np.uint64)
        total = np.zeros(hi - lo, dtype=np.int64)
        for lane in range(3):
            h = _hash(seed, idx, lane, 4)
            for sh in (0, 16, 32, 48):
                total += ((h >> np.uint64(sh)) & np.uint64(0xFFFF)).astype(np.int64)
        v = ((total - 393210).astype(np.float32)) * np.float32(2.0 ** -16)
        out[lo:hi] = v * s32 if sigma != 1.0 else v
    return out


def uniform_pm1(seed, n, chunk=1 << 22):
    """n float32 values uniform on [-1, 1): (u24 - 2^23) * 2^-23."""
    out = np.empty(n, dtype=np.float32)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        idx = np.arange(lo, hi, dtype=np.uint64)
        h = _hash(seed, idx, 0, 4)
        u = (h >> np.uint64(40)).astype(np.int64) - (1 << 23)
        out[lo:hi] = u.astype(np.float32) * np.float32(2.0 ** -23)
    return out


def zero_mask(seed, n, one_in=10, chunk=1 << 22):
    """Boolean mask, True for about 1/one_in of the elements."""
    out = np.empty(n, dtype=bool)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        idx = np.arange(lo, hi, dtype=np.uint64)
        h = _hash(seed, idx, 3, 4)
        out[lo:hi] = (h % np.uint64(one_in)) == 0
    return out


# The five workloads: (name, mb, ic, ih, iw, oc, kh, kw, sh, sw, ph, pw, src kind, w sigma)
WORKLOADS = {
    "alexnet_conv4_mb1":   dict(mb=1,   ic=384, ih=13, iw=13, oc=256, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1, src="normal",       wsigma=0.05),
    "alexnet_conv4_mb256": dict(mb=256, ic=384, ih=13, iw=13, oc=256, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1, src="normal",       wsigma=0.05),
    "alexnet_conv2_mb128": dict(mb=128, ic=96,  ih=27, iw=27, oc=256, kh=5, kw=5, sh=1, sw=1, ph=2, pw=2, src="normal",       wsigma=0.05),
    "resnet_3x3_mb64":     dict(mb=64,  ic=256, ih=56, iw=56, oc=256, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1, src="uniform",      wsigma=0.02),
    "vgg_512_mb32":        dict(mb=32,  ic=512, ih=28, iw=28, oc=512, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1, src="normal_zeros", wsigma=0.02),
}


def make_src(kind, n, seed=SEED_SRC):
    if kind == "normal":
        return normal(seed, n)
    if kind == "uniform":
        return uniform_pm1(seed, n)
    if kind == "normal_zeros":
        x = normal(seed, n)
        x[zero_mask(seed, n)] = np.float32(0.0)  # literal +0.0f, never x*0
        return x
    raise ValueError(kind)


def make_workload(name, mb=None):
    """Return (dims dict, src NCHW float32, weights OIHW float32) for a named workload."""
    d = dict(WORKLOADS[name])
    if mb is not None:
        d["mb"] = mb
    src = make_src(d["src"], d["mb"] * d["ic"] * d["ih"] * d["iw"])
    w = normal(SEED_WEIGHTS, d["oc"] * d["ic"] * d["kh"] * d["kw"], d["wsigma"])
    return d, src.reshape(d["mb"], d["ic"], d["ih"], d["iw"]), \
        w.reshape(d["oc"], d["ic"], d["kh"], d["kw"])


def reference_test_src(mb, ic, ih, iw):
    """Closed-form input of the reference's own tests
    (reference test/gtest/test_convolution_compare_with_reference.cpp:9-17):
    0.33f + 0.0023f*(19 - (iw+ih+ic+mb%37)), evaluated in float32 like the C expression."""
    m, c, h, w = np.meshgrid(np.arange(mb), np.arange(ic), np.arange(ih), np.arange(iw),
                             indexing="ij")
    t = (19 - (w + h + c + m % 37)).astype(np.float32)
    return (np.float32(0.33) + np.float32(0.0023) * t).astype(np.float32)


def reference_test_weights(oc, ic, kh, kw):
    """Closed-form weights of the reference's own tests
    (reference test/gtest/test_convolution_compare_with_reference.cpp:19-27):
    0.18f + 0.017f*(11 - (kw+kh+ic+oc%23))."""
    o, c, h, w = np.meshgrid(np.arange(oc), np.arange(ic), np.arange(kh), np.arange(kw),
                             indexing="ij")
    t = (11 - (w + h + c + o % 23)).astype(np.float32)
    return (np.float32(0.18) + np.float32(0.017) * t).astype(np.float32)
