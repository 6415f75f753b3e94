"""Helpers shared by the test modules."""
import hashlib

import numpy as np


def sha256(arr):
    return hashlib.sha256(np.ascontiguousarray(arr).tobytes()).hexdigest()


def oracle_shape(oracle, d, fmts=None):
    from xnor_nn_amd import capi
    fmts = fmts or (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW)
    return oracle.shape(d["mb"], d["oc"], d["ic"], d["ih"], d["iw"], d["kh"], d["kw"],
                        d["sh"], d["sw"], d["ph"], d["pw"], *fmts)


def brute_force_dot(x, w, d):
    """sum over in-bounds taps and channels of sgn(x)*sgn(w) with sgn = +1 when the sign
    bit is clear, computed from the raw floats in int64 (independent of any packing)."""
    sx = np.where(np.signbit(x), -1, 1).astype(np.int64)
    sw = np.where(np.signbit(w), -1, 1).astype(np.int64)
    mb, ic, ih, iw = x.shape
    oc = w.shape[0]
    oh = (ih + 2 * d["pw"] - d["kh"]) // d["sh"] + 1
    ow = (iw + 2 * d["pw"] - d["kw"]) // d["sw"] + 1
    out = np.zeros((mb, oc, oh, ow), dtype=np.int64)
    n = np.zeros((oh, ow), dtype=np.int64)
    for kh in range(d["kh"]):
        for kw in range(d["kw"]):
            for o_h in range(oh):
                i_h = o_h * d["sh"] - d["ph"] + kh
                if i_h < 0 or i_h >= ih:
                    continue
                for o_w in range(ow):
                    i_w = o_w * d["sw"] - d["pw"] + kw
                    if i_w < 0 or i_w >= iw:
                        continue
                    out[:, :, o_h, o_w] += sx[:, :, i_h, i_w] @ sw[:, :, kh, kw].T
                    n[o_h, o_w] += ic
    return out, n


def relative_error(actual, expected):
    a = np.asarray(actual, dtype=np.float64)
    e = np.asarray(expected, dtype=np.float64)
    denom = np.maximum(np.abs(e), np.finfo(np.float32).tiny)
    return float(np.max(np.abs(a - e) / denom)) if a.size else 0.0
