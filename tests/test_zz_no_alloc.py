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
    # host memory on either side: refused on the host, nothing is launched
    host = np.zeros(16 * 8 * 9, np.float32)
    assert fn(C.byref(c), host.ctypes.data, t.data_ptr()) == capi.ERROR_INVALID_INPUT
    assert fn(C.byref(c), t.data_ptr(), host.ctypes.data) == capi.ERROR_INVALID_INPUT
    torch.cuda.synchronize()
    lib.xnor_nn_destroy_convolution(C.byref(c))
    # more weights than the limit: refused before anything touches the pointers
    big = capi.ConvolutionDesc()
    big.oc, big.ic, big.kh, big.kw = 65536, 65536, 1, 1
    assert fn(C.byref(big), t.data_ptr(), t.data_ptr()) == capi.ERROR_INVALID_INPUT


def test_no_alloc_entry_point_allocates_nothing(gpu):
    """What the entry point is for.  (1) Free device memory is the same before and after a
    call.  (2) The call can be captured in a HIP graph (capture refuses allocation, free and
    synchronisation) on a side stream, and every replay, with eager calls on other weights
    in between, writes what the allocating entry point writes."""
    import torch
    lib = capi.load()
    oc, ic, kh, kw = 64, 96, 3, 3
    n = oc * ic * kh * kw
    w1 = synth.normal(931, n, 0.05).reshape(oc, ic, kh, kw)
    w2 = (w1[::-1] * np.float32(-0.5) + np.float32(0.01)).copy()
    c = descriptor(lib, oc, ic, kh, kw)
    w1t, w2t = torch.from_numpy(w1).to(gpu), torch.from_numpy(w2).to(gpu)
    src = w1t.clone()
    want1, want2 = torch.empty_like(w1t), torch.empty_like(w1t)
    lib.xnor_nn_binarize_weights_float(C.byref(c), w1t.data_ptr(), want1.data_ptr())
    lib.xnor_nn_binarize_weights_float(C.byref(c), w2t.data_ptr(), want2.data_ptr())
    got = torch.zeros_like(w1t)
    fn = lib.xnor_nn_hip_binarize_weights_float_noalloc
    assert fn(C.byref(c), src.data_ptr(), got.data_ptr()) == capi.SUCCESS  # warm: symbol looked up
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert fn(C.byref(c), src.data_ptr(), got.data_ptr()) == capi.SUCCESS
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(got, want1)
    side = torch.cuda.Stream()
    assert lib.xnor_nn_hip_set_stream(C.byref(c), C.c_void_p(side.cuda_stream)) == capi.SUCCESS
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert fn(C.byref(c), src.data_ptr(), got.data_ptr()) == capi.SUCCESS
    other = torch.zeros_like(w1t)
    for i in range(3):
        src.copy_(w1t if i % 2 == 0 else w2t)
        got.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want1 if i % 2 == 0 else want2), i
        with torch.cuda.stream(side):  # an eager call on the same shared partial sums
            assert fn(C.byref(c), w2t.data_ptr(), other.data_ptr()) == capi.SUCCESS
        side.synchronize()
        assert torch.equal(other, want2), i
    lib.xnor_nn_destroy_convolution(C.byref(c))
