"""The entry point that allocates nothing: xnor_nn_hip_binarize_weights_float_noalloc against
xnor_nn_binarize_weights_float, through the C ABI, bit for bit."""
import ctypes as C

import numpy as np
import pytest

from xnor_nn_amd import capi, synth

pytestmark = pytest.mark.gpu


def descriptor(lib, oc, ic, kh, kw):
    c = capi.ConvolutionDesc()
    assert lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW,
                                        capi.FMT_OIHW, capi.FMT_NCHW, 1, oc, ic, 13, 13, kh, kw,
                                        1, 1, 1, 1) == capi.SUCCESS
    return c


def test_no_alloc_entry_point_matches_the_allocating_one(gpu):
    """Two calls in a row, the second on a smaller weight tensor (the partial sums of the
    first call are still in the shared array), then the first size again."""
    import torch
    lib = capi.load()
    for oc, ic, kh, kw in ((256, 384, 3, 3), (48, 33, 5, 5), (256, 384, 3, 3), (1, 1, 1, 1)):
        n = oc * ic * kh * kw
        w = synth.normal(900 + oc, n, 0.05).reshape(oc, ic, kh, kw)
        w.ravel()[::97] = -0.0
        wt = torch.from_numpy(w).to(gpu)
        c = descriptor(lib, oc, ic, kh, kw)
        want = torch.empty_like(wt)
        lib.xnor_nn_binarize_weights_float(C.byref(c), wt.data_ptr(), want.data_ptr())
        got = torch.full_like(wt, float("nan"))
        torch.cuda.synchronize()
        assert lib.xnor_nn_hip_binarize_weights_float_noalloc(
            C.byref(c), wt.data_ptr(), got.data_ptr()) == capi.SUCCESS
        assert lib.xnor_nn_hip_synchronize(C.byref(c)) == capi.SUCCESS
        torch.cuda.synchronize()
        g, e = got.cpu().numpy(), want.cpu().numpy()
        assert np.array_equal(g.view(np.uint32), e.view(np.uint32)), (oc, ic, kh, kw)
        # and what the values have to be: +mean(w) where w >= 0 (a negative zero counts as
        # positive), -mean(w) elsewhere
        mean = float(np.mean(w.astype(np.float64)))
        m = g[w >= 0][0] if np.any(w >= 0) else -g[w < 0][0]
        assert np.all(g[w >= 0] == m) and np.all(g[w < 0] == -m)
        assert abs(float(m) - mean) <= 1e-6 * float(np.mean(np.abs(w)))
        lib.xnor_nn_destroy_convolution(C.byref(c))


def test_no_alloc_entry_point_refuses_what_it_cannot_take(gpu):
    import torch
    lib = capi.load()
    c = descriptor(lib, 16, 8, 3, 3)
    t = torch.zeros(16 * 8 * 9, dtype=torch.float32, device=gpu)
    fn = lib.xnor_nn_hip_binarize_weights_float_noalloc
    assert fn(C.byref(c), None, t.data_ptr()) == capi.ERROR_INVALID_INPUT
    assert fn(C.byref(c), t.data_ptr(), None) == capi.ERROR_INVALID_INPUT
    assert fn(None, t.data_ptr(), t.data_ptr()) == capi.ERROR_INVALID_INPUT
    lib.xnor_nn_destroy_convolution(C.byref(c))
    # more weights than the limit: refused before anything touches the pointers
    big = capi.ConvolutionDesc()
    big.oc, big.ic, big.kh, big.kw = 65536, 65536, 1, 1
    assert fn(C.byref(big), t.data_ptr(), t.data_ptr()) == capi.ERROR_INVALID_INPUT
