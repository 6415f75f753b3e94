"""Parity of the HIP path against the CPU oracle and the committed digests of the upstream
library's outputs.  Everything goes through the C ABI of libxnor_nn.so.

Bar: packed tensors, operation counts and integer popcount accumulators bit-exact; the
float tensors (a, k, alpha, dst) are computed in the reference's summation order and are
asserted bit-exact as well, which is stricter than the 1e-5 relative tolerance allowed for
them (the tolerance check is kept in `check_floats` for the error message only)."""
import os

import numpy as np
import pytest

import shapes
from util import oracle_shape, relative_error, sha256
from xnor_nn_amd import Convolution, capi, synth

pytestmark = pytest.mark.gpu
REL_TOL = 1e-5

NCHW = (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW)


def make(d, w, fmts=NCHW):
    return Convolution(capi.ALGORITHM_BCAST, fmts[0], fmts[1], fmts[2],
                       d["mb"], d["oc"], d["ic"], d["ih"], d["iw"], d["kh"], d["kw"],
                       d["sh"], d["sw"], d["ph"], d["pw"], w)


def check_floats(name, got, want):
    err = relative_error(got, want)
    assert err <= REL_TOL, "%s: relative error %.3e > %.0e" % (name, err, REL_TOL)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
        "%s within tolerance (%.3e) but not bit-identical" % (name, err)


def run_and_compare(oracle, d, x, w, fmts=NCHW, device_tensors=False, gpu=None):
    """Full pipeline on the GPU vs the oracle, every intermediate."""
    s = oracle_shape(oracle, d, fmts)
    want = oracle.forward(s, x, w)
    dshape = want["dst"].shape
    if device_tensors:
        import torch
        xt = torch.from_numpy(x).to(gpu)
        wt = torch.from_numpy(w).to(gpu)
        dt = torch.empty(dshape, dtype=torch.float32, device=gpu)
        conv = make(d, wt, fmts)
        conv.forward(xt, dt)
        conv.synchronize()
        dst = dt.cpu().numpy()
    else:
        dst = np.full(dshape, np.nan, dtype=np.float32)
        conv = make(d, w, fmts)
        conv.forward(x, dst)
    assert np.array_equal(conv.export_bin_src(), want["bin_src"]), "bin_src"
    assert np.array_equal(conv.export_operations_count(), want["opc"]), "operations_count"
    if d["oc"] % oracle.default_oci(s) == 0:
        assert np.array_equal(conv.export_bin_weights(), want["bin_weights"]), "bin_weights"
    check_floats("alpha", conv.export_floats(capi.RES_ALPHA), want["alpha"])
    check_floats("a", conv.export_floats(capi.RES_A), want["a"])
    check_floats("k", conv.export_floats(capi.RES_K), want["k"])
    assert np.array_equal(conv.forward_popcount(), want["popc"]), "popcount accumulators"
    check_floats("dst", dst, want["dst"])
    conv.close()
    return dst, want


@pytest.mark.parametrize("t", shapes.COMPARE_WITH_REFERENCE, ids=shapes.shape_id)
def test_reference_test_matrix(oracle, golden, t):
    """The shape matrix and closed-form inputs of the reference's differential test
    (reference test/gtest/test_convolution_compare_with_reference.cpp:9-27,82-217), host
    pointers like the reference's tests; also against the upstream digests."""
    d = shapes.as_dims(t)
    x = synth.reference_test_src(d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.reference_test_weights(d["oc"], d["ic"], d["kh"], d["kw"])
    dst, _ = run_and_compare(oracle, d, x, w)
    assert sha256(dst) == golden["reference_test_shapes"][shapes.shape_id(t)]["sha256"]["dst"]


@pytest.mark.parametrize("name,mb", [
    ("alexnet_conv4_mb1", None), ("alexnet_conv4_mb256", 16), ("alexnet_conv2_mb128", 4),
    ("resnet_3x3_mb64", 2), ("vgg_512_mb32", 2)])
def test_workloads_reduced_batch(oracle, gpu, name, mb):
    """The five benchmark workloads at a small batch, device-resident tensors."""
    d, x, w = synth.make_workload(name, mb)
    run_and_compare(oracle, d, x, w, device_tensors=True, gpu=gpu)


@pytest.mark.parametrize("name", list(synth.WORKLOADS))
def test_workloads_full_size_digests(oracle, golden, gpu, name):
    """Benchmark sizes: every tensor the GPU produced hashes to what the upstream library
    produced on the same seeded inputs (tests/golden/golden.json), and to the oracle."""
    import torch
    d, x, w = synth.make_workload(name)
    g = golden["workloads"][name]["sha256"]
    xt = torch.from_numpy(x).to(gpu)
    wt = torch.from_numpy(w).to(gpu)
    dt = torch.empty((d["mb"], d["oc"], d["ih"], d["iw"]), dtype=torch.float32, device=gpu)
    conv = make(d, wt)
    conv.forward(xt, dt)
    conv.synchronize()
    assert sha256(conv.export_bin_src()) == g["bin_src"]
    assert sha256(conv.export_bin_weights()) == g["bin_weights"]
    assert sha256(conv.export_operations_count()) == g["opc"]
    assert sha256(conv.export_floats(capi.RES_ALPHA)) == g["alpha"]
    assert sha256(conv.export_floats(capi.RES_A)) == g["a"]
    assert sha256(conv.export_floats(capi.RES_K)) == g["k"]
    dst = dt.cpu().numpy()
    assert sha256(dst) == g["dst"]
    # integer accumulators against the oracle, and the size-independent identity
    # 2*popc - n == dst / (alpha*k) up to the two roundings
    s = oracle_shape(oracle, d)
    want = oracle.forward(s, x, w)
    pt = torch.empty((d["mb"], d["oc"], d["ih"], d["iw"]), dtype=torch.int32, device=gpu)
    conv.forward_popcount(pt)
    conv.synchronize()
    assert np.array_equal(pt.cpu().numpy(), want["popc"])
    assert np.array_equal(dst.view(np.uint32), want["dst"].view(np.uint32))
    conv.close()


@pytest.mark.parametrize("fmts", [
    (capi.FMT_NHWC, capi.FMT_OIHW, capi.FMT_NCHW),
    (capi.FMT_NCHW, capi.FMT_HWIO, capi.FMT_NCHW),
    (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC),
    (capi.FMT_NHWC, capi.FMT_HWIO, capi.FMT_NHWC),
])
@pytest.mark.parametrize("t", [(3, 40, 32, 9, 11, 3, 3, 1, 1, 1, 1),
                               (2, 96, 48, 13, 13, 5, 5, 1, 1, 2, 2),
                               # full 64-filter waves (16-byte NHWC stores), IC = 3 words + 4
                               (3, 256, 100, 13, 13, 3, 3, 1, 1, 1, 1),
                               # IC not a multiple of 4: the generic NHWC kernel
                               (1, 12, 37, 6, 7, 3, 3, 1, 1, 1, 1)], ids=shapes.shape_id)
def test_tensor_formats(oracle, fmts, t):
    """NHWC input, HWIO weights and NHWC output (reference
    src/bcast_binarize_data.cpp:56-57, src/bcast_binarize_weights.cpp:71-72,
    src/default/bcast_convolution_default.cpp:97-99)."""
    d = shapes.as_dims(t)
    x = synth.normal(31, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.normal(32, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    if fmts[0] == capi.FMT_NHWC:
        x = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    if fmts[1] == capi.FMT_HWIO:
        w = np.ascontiguousarray(w.transpose(2, 3, 1, 0))
    run_and_compare(oracle, d, x, w, fmts)


@pytest.mark.parametrize("t", [
    (1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0),        # smallest possible problem
    (2, 5, 3, 4, 6, 3, 3, 1, 1, 1, 1),        # oc below one filter group
    (1, 70, 20, 7, 5, 3, 3, 2, 2, 1, 1),      # stride 2, ic and oc ragged
    (3, 33, 17, 6, 6, 5, 5, 1, 1, 2, 2),      # one bit past a word
    (1, 1100, 16, 3, 3, 3, 3, 1, 1, 1, 1),    # more than 1024 channels: two parts of 12 steps
    (1, 3700, 16, 3, 3, 3, 3, 1, 1, 1, 1),    # ic*kh*kw > 32767: int32 words upstream
    (1, 4100, 16, 3, 3, 3, 3, 1, 1, 1, 1),    # more than 4096 channels: XNOR/popcount kernel
    (5, 64, 64, 5, 9, 1, 1, 1, 1, 0, 0),      # 1x1 filter
    (2, 16, 32, 8, 8, 3, 3, 1, 1, 0, 0),      # no padding
    (1, 24, 16, 12, 12, 7, 7, 3, 3, 3, 3),    # big filter, stride 3
    (2, 160, 100, 9, 9, 3, 3, 1, 1, 1, 1),    # 3 channel steps of 64, ragged filter count
    (2, 288, 300, 7, 7, 3, 3, 1, 1, 1, 1),    # 5 steps (run as 6), more than 256 filters
    (1, 448, 70, 6, 6, 3, 3, 1, 1, 1, 1),     # 7 steps (run as 8)
    (7, 64, 40, 10, 10, 3, 3, 1, 1, 2, 2),    # padding larger than the usual "same"
    (2, 32, 64, 16, 16, 4, 4, 1, 1, 0, 0),    # even filter size, output smaller than input
    (1, 640, 32, 5, 5, 3, 3, 1, 1, 1, 1),     # more than 512 channels: 12 steps, quarter-tap groups
    (2, 1024, 70, 7, 7, 1, 1, 1, 1, 0, 0),    # 1x1 over 1024 channels: 16 steps
    (1, 1000, 40, 6, 6, 3, 3, 1, 1, 1, 1),    # 16 steps with a ragged last word, 3x3
    (3, 768, 260, 9, 9, 3, 3, 2, 2, 1, 1),    # 12 steps, stride 2, more than 256 filters
], ids=shapes.shape_id)
def test_edge_shapes(oracle, t):
    d = shapes.as_dims(t)
    x = synth.normal(41, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::5] = 0.0
    x.ravel()[2::9] = -0.0
    w = synth.normal(42, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    w.ravel()[::13] = -0.0
    run_and_compare(oracle, d, x, w)


@pytest.mark.parametrize("ps", ["1", "2", "3", "4"])
def test_matrix_core_tile_sizes(oracle, gpu, monkeypatch, ps):
    """Every tile size of the matrix-core kernel on a workload whose last tile is ragged."""
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_PS", ps)
    d, x, w = synth.make_workload("alexnet_conv4_mb256", 5)
    run_and_compare(oracle, d, x, w, device_tensors=True, gpu=gpu)
    d, x, w = synth.make_workload("vgg_512_mb32", 1)
    run_and_compare(oracle, d, x, w, device_tensors=True, gpu=gpu)
    # paired taps over three words, and 12 steps per tap
    d, x, w = synth.make_workload("alexnet_conv2_mb128", 2)
    assert make(d, w).kernel_name(0) == "conv_mfma_fp4_kernel<KS=3,PS=%s,PAIR>" % ps
    run_and_compare(oracle, d, x, w, device_tensors=True, gpu=gpu)
    d = shapes.as_dims((2, 768, 70, 14, 14, 3, 3, 1, 1, 1, 1))
    x = synth.normal(75, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.normal(76, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    assert make(d, w).kernel_name(0) == "conv_mfma_fp4_kernel<KS=12,PS=%s,GROUPS=2>" % ps  # 70 filters
    run_and_compare(oracle, d, x, w)


@pytest.mark.parametrize("pair", ["0", "1"])
@pytest.mark.parametrize("t", [
    (2, 96, 64, 13, 13, 5, 5, 1, 1, 2, 2),     # 3 words, 25 taps (odd: last pair has one tap)
    (3, 32, 70, 9, 11, 3, 3, 1, 1, 1, 1),      # 1 word: two taps per matrix instruction
    (1, 20, 33, 8, 8, 2, 2, 1, 1, 0, 0),       # 1 ragged word, even number of taps
    (2, 160, 40, 10, 10, 3, 3, 2, 2, 1, 1),    # 5 words, stride 2
    (1, 150, 300, 7, 6, 4, 3, 1, 1, 1, 1),     # 5 words (ragged), more than 256 filters
], ids=shapes.shape_id)
def test_tap_pairing(oracle, monkeypatch, t, pair):
    """Odd numbers of 32-channel words per pixel: the matrix-core kernel with and without
    two taps sharing their steps (XNOR_NN_HIP_MFMA_PAIR forces either)."""
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_PAIR", pair)
    d = shapes.as_dims(t)
    x = synth.normal(71, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.normal(72, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    name = make(d, w).kernel_name(0)
    assert name.startswith("conv_mfma") and (",PAIR" in name) == (pair == "1"), name
    run_and_compare(oracle, d, x, w)


def test_popcount_kernel_still_matches(oracle, gpu, monkeypatch):
    """The XNOR/popcount kernel (the general fallback) on shapes the matrix-core kernel
    would otherwise take."""
    monkeypatch.setenv("XNOR_NN_HIP_CONV", "valu")
    for name, mb in (("alexnet_conv4_mb256", 4), ("alexnet_conv2_mb128", 2)):
        d, x, w = synth.make_workload(name, mb)
        conv_name = make(d, w).kernel_name(0)
        assert conv_name.startswith("conv_xnor_popc"), conv_name
        run_and_compare(oracle, d, x, w, device_tensors=True, gpu=gpu)
    # strides above 1, ragged channel and filter counts
    for t in ((1, 70, 20, 7, 5, 3, 3, 2, 2, 1, 1), (1, 24, 16, 12, 12, 7, 7, 3, 3, 3, 3),
              (2, 96, 64, 28, 28, 3, 3, 2, 2, 1, 1)):
        d = shapes.as_dims(t)
        x = synth.normal(51, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
            d["mb"], d["ic"], d["ih"], d["iw"])
        w = synth.normal(52, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
            d["oc"], d["ic"], d["kh"], d["kw"])
        run_and_compare(oracle, d, x, w)


@pytest.mark.parametrize("t", [
    (2, 96, 64, 28, 28, 3, 3, 2, 2, 1, 1),     # ResNet-style 3x3 stride 2
    (3, 128, 64, 28, 28, 1, 1, 2, 2, 0, 0),    # 1x1 stride 2 shortcut
    (2, 64, 96, 27, 27, 5, 5, 2, 2, 2, 2),     # 5x5 stride 2, ragged channels
    (1, 32, 130, 31, 29, 3, 3, 3, 2, 1, 1),    # different strides per axis
    (2, 64, 64, 23, 23, 7, 7, 4, 4, 2, 2),     # 7x7 stride 4
], ids=shapes.shape_id)
def test_strided_shapes_on_the_matrix_core_kernel(oracle, t):
    """Strides above 1 run the matrix-core kernel too (the staged span of input pixels then
    also holds the ones the stride skips)."""
    d = shapes.as_dims(t)
    x = synth.normal(61, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.normal(62, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    conv_name = make(d, w).kernel_name(0)
    assert conv_name.startswith("conv_mfma"), conv_name
    run_and_compare(oracle, d, x, w)


@pytest.mark.parametrize("t", [
    (1, 512, 64, 112, 112, 3, 3, 1, 1, 1, 1),  # 258 staged pixels of 272 bytes
    (1, 1024, 40, 56, 56, 3, 3, 1, 1, 1, 1),   # 16 steps per tap on a 56 x 56 image
    (1, 256, 32, 60, 60, 7, 7, 2, 2, 3, 3),    # 7 x 7 stride 2: seven image rows and more
    (1, 96, 70, 120, 120, 11, 11, 4, 4, 2, 2), # 11 x 11 stride 4, paired taps
], ids=shapes.shape_id)
def test_tiles_that_need_more_than_64_kb_of_lds(oracle, t):
    """The matrix-core kernel keeps every input pixel a tile touches in LDS; a gfx950
    workgroup may use up to 160 KB of it, which has to be asked for above 64 KB."""
    d = shapes.as_dims(t)
    x = synth.normal(81, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.normal(82, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    conv_name = make(d, w).kernel_name(0)
    assert conv_name.startswith("conv_mfma"), conv_name
    run_and_compare(oracle, d, x, w)


@pytest.mark.parametrize("t,parts", [
    ((2, 2048, 130, 7, 7, 1, 1, 1, 1, 0, 0), ("KS=16", "PARTS=2")),   # ResNet-50 style 1x1
    ((1, 1536, 64, 9, 8, 3, 3, 1, 1, 1, 1), ("KS=12", "PARTS=2")),    # 24 steps, no padding
    ((1, 2500, 40, 6, 6, 3, 3, 2, 2, 1, 1), ("KS=16", "PARTS=3")),    # 40 steps (run as 48), stride 2
    ((1, 4096, 300, 4, 4, 2, 2, 1, 1, 0, 0), ("KS=16", "PARTS=4")),  # the most the kernel takes
    ((3, 1100, 70, 12, 12, 3, 3, 1, 1, 1, 1), ("KS=12", "PARTS=2")),   # several tiles per image
], ids=lambda v: shapes.shape_id(v) if len(v) == 11 else "-".join(v))
@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
def test_more_than_1024_channels_on_the_matrix_core_kernel(oracle, t, parts, layout):
    """Above 1024 input channels the kernel walks every tap once per part of 768 or 1024
    channels; the fragments of a part follow those of the part before."""
    d = shapes.as_dims(t)
    x = synth.normal(91, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::6] = 0.0
    w = synth.normal(92, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    fmts = (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW)
    if layout == "nhwc":
        fmts = (capi.FMT_NHWC, capi.FMT_HWIO, capi.FMT_NHWC)
        x = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
        w = np.ascontiguousarray(w.transpose(2, 3, 1, 0))
    conv_name = make(d, w, fmts).kernel_name(0)
    assert conv_name.startswith("conv_mfma") and all(p in conv_name for p in parts), conv_name
    run_and_compare(oracle, d, x, w, fmts)


@pytest.mark.parametrize("by_lane", [False, True])
@pytest.mark.parametrize("t", [
    (3, 384, 64, 13, 13, 3, 3, 1, 1, 1, 1),    # twelve slices, one round; ragged last tile
    (2, 512, 32, 9, 7, 3, 3, 1, 1, 1, 1),      # sixteen slices in two rounds of eight waves
    (5, 100, 16, 6, 5, 1, 1, 1, 1, 0, 0),      # last slice holds 4 channels: 7 of 8 pieces empty
    (1, 36, 16, 10, 10, 3, 3, 1, 1, 1, 1),     # one full slice and one piece
    (1, 4, 8, 17, 3, 1, 1, 1, 1, 0, 0),        # a single piece, 51 pixels
    (2, 800, 16, 5, 5, 3, 3, 1, 1, 1, 1),      # 25 slices in three rounds
], ids=shapes.shape_id)
def test_nhwc_input_kernels(oracle, monkeypatch, t, by_lane):
    """Channels-last input: the tiled kernel (whole cache lines per load, turned around through
    LDS) and the one-lane-per-pixel kernel it falls back to for very deep inputs."""
    if by_lane:
        monkeypatch.setenv("XNOR_NN_HIP_NHWC", "lane")
    d = shapes.as_dims(t)
    x = synth.normal(97, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ih"], d["iw"], d["ic"])
    x.ravel()[::5] = 0.0
    x.ravel()[1::7] = -0.0
    w = synth.normal(98, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    fmts = (capi.FMT_NHWC, capi.FMT_OIHW, capi.FMT_NCHW)
    name = make(d, w, fmts).kernel_name(2)
    assert name == ("binarize_nhwc_kernel" if by_lane else "binarize_nhwc_tiled_kernel"), name
    run_and_compare(oracle, d, x, w, fmts)


def _random_case(rng):
    kh, kw = int(rng.integers(1, 8)), int(rng.integers(1, 8))
    ph, pw = int(rng.integers(0, 4)), int(rng.integers(0, 4))
    sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    # the reference derives oh AND ow from pw, so keep both extents consistent with that
    ih = int(rng.integers(max(1, kh - 2 * pw), 22))
    iw = int(rng.integers(max(1, kw - 2 * pw), 22))
    ic = int(rng.choice([1, 3, 31, 32, 33, 64, 65, 96, 100, 128, 160, 200, 257]))
    oc = int(rng.choice([1, 7, 16, 31, 32, 33, 64, 65, 100, 130, 256, 260]))
    mb = int(rng.integers(1, 5))
    fmts = (int(rng.choice([capi.FMT_NCHW, capi.FMT_NHWC])),
            int(rng.choice([capi.FMT_OIHW, capi.FMT_HWIO])),
            int(rng.choice([capi.FMT_NCHW, capi.FMT_NHWC])))
    return (mb, ic, oc, ih, iw, kh, kw, sh, sw, ph, pw), fmts


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_strides_and_layouts(oracle, seed):
    """Seeded random problems (channel counts around the 32/64 boundaries, kernels 1..7,
    strides 1..3, paddings 0..3, all layout combinations), ten per seed, every intermediate
    against the oracle.  Inputs carry exact zeros of both signs."""
    rng = np.random.default_rng(1000 + seed)
    done = 0
    while done < 10:
        t, fmts = _random_case(rng)
        d = shapes.as_dims(t)
        oh = (d["ih"] + 2 * d["pw"] - d["kh"]) // d["sh"] + 1
        ow = (d["iw"] + 2 * d["pw"] - d["kw"]) // d["sw"] + 1
        if oh < 1 or ow < 1 or d["ih"] + 2 * d["ph"] < d["kh"]:
            continue
        x = synth.normal(7000 + 100 * seed + done, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
            d["mb"], d["ic"], d["ih"], d["iw"])
        x.ravel()[::7] = 0.0
        x.ravel()[3::11] = -0.0
        w = synth.normal(9000 + 100 * seed + done, d["oc"] * d["ic"] * d["kh"] * d["kw"],
                         0.05).reshape(d["oc"], d["ic"], d["kh"], d["kw"])
        if fmts[0] == capi.FMT_NHWC:
            x = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
        if fmts[1] == capi.FMT_HWIO:
            w = np.ascontiguousarray(w.transpose(2, 3, 1, 0))
        try:
            run_and_compare(oracle, d, x, w, fmts)
        except AssertionError as e:
            raise AssertionError("case %s formats %s: %s" % (shapes.shape_id(t), fmts, e))
        done += 1


@pytest.mark.parametrize("case", ["conv4", "tile_above_64_kb"])
def test_forward_pass_captured_in_a_hip_graph(oracle, gpu, case):
    """The three executors enqueue kernels only (no allocation, no memset, no host
    synchronisation when the tensors are on the device), so a caller may capture them in a
    HIP graph.  Every replay, with eager passes and synchronisations in between, must give
    the eager result bit for bit.  The second case is a tile that has to ask for more than
    64 KB of LDS at every launch, captured ones included."""
    import torch
    if case == "conv4":
        d, x, w = synth.make_workload("alexnet_conv4_mb256", 24)
    else:
        d = shapes.as_dims((2, 512, 64, 112, 112, 3, 3, 1, 1, 1, 1))
        x = synth.normal(95, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
            d["mb"], d["ic"], d["ih"], d["iw"])
        w = synth.normal(96, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
            d["oc"], d["ic"], d["kh"], d["kw"])
    x2 = np.ascontiguousarray(x[::-1])
    s = oracle_shape(oracle, d)
    want, want2 = oracle.forward(s, x, w)["dst"], oracle.forward(s, x2, w)["dst"]
    side = torch.cuda.Stream()
    xt = torch.from_numpy(x).to(gpu)
    x2t = torch.from_numpy(x2).to(gpu)
    yt = torch.empty(want.shape, dtype=torch.float32, device=gpu)
    conv = make(d, torch.from_numpy(w).to(gpu))
    conv.set_stream(side)

    def step():
        conv.stage("binarize_data", src=xt, dst=yt)
        conv.stage("calculate_k")
        conv.stage("forward")

    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        step() # eager pass first: the staging state of the descriptor is settled
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    for i in range(4):
        yt.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(yt.cpu().numpy().view(np.uint32), want.view(np.uint32)), i
        # eager work of the same descriptor on other data between the replays
        with torch.cuda.stream(side):
            conv.stage("binarize_data", src=x2t, dst=yt)
            conv.stage("calculate_k")
            conv.stage("forward")
        side.synchronize()
        assert np.array_equal(yt.cpu().numpy().view(np.uint32), want2.view(np.uint32)), i
    conv.close()


def test_known_answer_forward_on_gpu():
    """The reference's 18 precomputed outputs
    (reference test/gtest/test_convolution_reference_forward.cpp:20-73), tolerance 1e-3."""
    from test_oracle import KA_DIMS, KA_DST, KA_SRC, KA_W
    conv = make(KA_DIMS, KA_W)
    dst = np.zeros((1, 2, 3, 3), np.float32)
    conv.forward(KA_SRC, dst)
    assert np.allclose(dst, KA_DST, atol=1e-3, rtol=0)
    conv.close()


def test_calculate_k_alone_matches_fused_path(oracle, gpu):
    """calculate_k called without a preceding binarize_data reads the input itself; both
    routes give the same bits."""
    import torch
    d, x, w = synth.make_workload("alexnet_conv4_mb256", 8)
    s = oracle_shape(oracle, d)
    a_want, k_want = oracle.calculate_k(s, x)
    xt = torch.from_numpy(x).to(gpu)
    conv = make(d, w)
    conv.stage("calculate_k", src=xt)
    assert np.array_equal(conv.export_floats(capi.RES_A), a_want)
    assert np.array_equal(conv.export_floats(capi.RES_K), k_want)
    conv.stage("binarize_data", src=xt)
    conv.stage("calculate_k", src=xt)
    assert np.array_equal(conv.export_floats(capi.RES_K), k_want)
    conv.close()


@pytest.mark.parametrize("exe", ["simple_convolution_c", "simple_convolution_cpp"])
def test_upstream_example_programs_run_unchanged(gpu, exe):
    """The reference's own example programs (reference example/simple_convolution.c and
    .cpp: host buffers, algorithm "best", three forward passes), compiled unchanged against
    include/ and linked to this library by `make -C oracle examples`, run to completion.
    The C program prints the status string of its last call."""
    import subprocess
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "oracle", "_ref", "examples", exe)
    if not os.path.exists(path):
        pytest.skip("example programs not built (upstream sources were not mounted)")
    out = subprocess.run([path], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, (out.stdout, out.stderr)
    if exe.endswith("_c"):
        assert out.stdout.strip() == "success"


@pytest.mark.parametrize("exe", ["test_only_convolution", "test_simple_net"])
def test_upstream_performance_programs_run_unchanged(gpu, exe):
    """The reference's performance programs (reference test/perf/test_only_convolution.cpp:
    8192 forward calls with only user_dst set; test/perf/test_simple_net.cpp: every stage of
    seven layer shapes on host buffers, AlexNet conv1 with stride 4 among them), compiled
    unchanged and linked to this library by `make -C oracle examples`.  Both end by printing
    the status string of their last call."""
    import subprocess
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "oracle", "_ref", "examples", exe)
    if not os.path.exists(path):
        pytest.skip("performance programs not built (upstream sources were not mounted)")
    out = subprocess.run([path], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, (out.stdout[-2000:], out.stderr[-2000:])
    assert out.stdout.strip().endswith("success"), out.stdout[-500:]


def test_device_info(gpu):
    """xnor_nn_hip_device_info: compute units and clock of the current device, what the
    benchmark prices the XNOR/popcount kernel's ceiling with."""
    import ctypes as C
    cus, khz = C.c_int(0), C.c_int(0)
    assert capi.load().xnor_nn_hip_device_info(C.byref(cus), C.byref(khz)) == 0
    assert 32 <= cus.value <= 512 and 1_000_000 <= khz.value <= 3_000_000, (cus.value, khz.value)


def test_binarize_weights_float(oracle, gpu):
    """xnor_nn_binarize_weights_float on host and on device buffers: the signs follow
    w >= 0 exactly (a negative zero counts as positive), every magnitude is the same float,
    and that float is the mean of the weights.  The reference's own sum is only defined on one
    thread (a data race otherwise, reference src/binarize_weights_float.cpp:17-19) and is
    sequential there; the device sums 256 slices, so the mean is compared to 1e-6 of the mean
    magnitude instead of bit for bit."""
    import torch
    d, _, w = synth.make_workload("alexnet_conv4_mb256", 1)
    w = w.copy()
    w.ravel()[::97] = -0.0
    want = oracle.binarize_weights_float(oracle_shape(oracle, d), w)
    conv = make(d, w)
    host = np.empty_like(w)
    conv.binarizeWeightsFloat(w, host)
    dev = torch.empty(w.shape, dtype=torch.float32, device=gpu)
    conv.binarizeWeightsFloat(torch.from_numpy(w).to(gpu), dev)
    conv.close()
    scale = float(np.mean(np.abs(w.astype(np.float64))))
    for got in (host, dev.cpu().numpy()):
        assert np.array_equal(np.signbit(got), np.signbit(want))
        m = got[w >= 0][0]
        assert np.all(got[w >= 0] == m) and np.all(got[w < 0] == -m)
        assert abs(float(m) - float(want[w >= 0][0])) <= 1e-6 * scale
        assert abs(float(m) - float(np.mean(w.astype(np.float64)))) <= 1e-6 * scale


def test_pytorch_layer(oracle, gpu):
    """xnor_nn_amd.torch_layer.XnorConv2d, the forward pass of the reference's Caffe layer for
    PyTorch tensors: bit-identical to the oracle, rebuilt for a new batch size, new weights
    only after weights_changed()."""
    import torch
    from xnor_nn_amd.torch_layer import XnorConv2d
    d, x, w = synth.make_workload("alexnet_conv4_mb256", 3)
    s = oracle_shape(oracle, d)
    layer = XnorConv2d(d["ic"], d["oc"], (d["kh"], d["kw"]), stride=(d["sh"], d["sw"]),
                       padding=(d["ph"], d["pw"]), weight=torch.from_numpy(w)).to(gpu)
    xt = torch.from_numpy(x).to(gpu)
    y = layer(xt)
    assert np.array_equal(y.cpu().numpy().view(np.uint32),
                          oracle.forward(s, x, w)["dst"].view(np.uint32))
    # another batch size builds another descriptor
    d2 = dict(d, mb=2)
    y2 = layer(xt[:2])
    assert np.array_equal(y2.cpu().numpy().view(np.uint32),
                          oracle.forward(oracle_shape(oracle, d2), x[:2], w)["dst"].view(np.uint32))
    # new weights take effect once the layer is told
    w2 = np.ascontiguousarray(w[::-1])
    with torch.no_grad():
        layer.weight.copy_(torch.from_numpy(w2))
    assert torch.equal(layer(xt[:2]), y2)
    layer.weights_changed()
    y3 = layer(xt[:2])
    assert np.array_equal(y3.cpu().numpy().view(np.uint32),
                          oracle.forward(oracle_shape(oracle, d2), x[:2], w2)["dst"].view(np.uint32))
    bw = layer.binarized_weights().cpu().numpy()
    assert np.array_equal(np.signbit(bw), np.signbit(
        oracle.binarize_weights_float(oracle_shape(oracle, d2), w2)))
    # a stream other than the default one
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y4 = layer(xt[:2])
    side.synchronize()
    assert torch.equal(y4, y3)
    # first call and a weight change both inside a side stream: the weight stage has to run on
    # that stream too, behind the copy into `weight` and ahead of the forward pass
    layer2 = XnorConv2d(d["ic"], d["oc"], (d["kh"], d["kw"]), stride=(d["sh"], d["sw"]),
                        padding=(d["ph"], d["pw"]), weight=torch.from_numpy(w)).to(gpu)
    w2t = torch.from_numpy(w2).to(gpu)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        ya = layer2(xt[:2])
        layer2.weight.data.copy_(w2t, non_blocking=True)
        layer2.weights_changed()
        yb = layer2(xt[:2])
        bw2 = layer2.binarized_weights()
    side.synchronize()
    assert torch.equal(ya, y2) and torch.equal(yb, y3)
    assert np.array_equal(bw2.cpu().numpy(), bw)


def test_deferred_box_filter_keeps_stage_semantics(oracle, gpu, monkeypatch):
    """With the matrix-core kernel, calculate_k leaves the box filter to the convolution.
    The K plane must still be what calculate_k saw: (1) read back before any forward, (2)
    after the input and mean|x| were overwritten by a later binarize_data, (3) after a
    forward, where the convolution kernel itself wrote it, and (4) with the deferral
    switched off."""
    import torch
    d, x1, w = synth.make_workload("alexnet_conv4_mb256", 6)
    x2 = (x1[::-1] * np.float32(1.5)).copy()
    s = oracle_shape(oracle, d)
    want1 = oracle.forward(s, x1, w)
    want2 = oracle.forward(s, x2, w)
    x1t, x2t = torch.from_numpy(x1).to(gpu), torch.from_numpy(x2).to(gpu)
    dt = torch.empty(want1["dst"].shape, dtype=torch.float32, device=gpu)
    conv = make(d, torch.from_numpy(w).to(gpu))
    # (1)
    conv.stage("binarize_data", src=x1t, dst=dt)
    conv.stage("calculate_k")
    assert np.array_equal(conv.export_floats(capi.RES_K), want1["k"])
    # (2) K of x1 is owed when x2 is binarized; forward must then use K(x1) with bits(x2)
    conv.stage("binarize_data", src=x1t)
    conv.stage("calculate_k")
    conv.stage("binarize_data", src=x2t)
    assert np.array_equal(conv.export_floats(capi.RES_K), want1["k"])
    assert np.array_equal(conv.export_floats(capi.RES_A), want2["a"])
    # (3)
    conv.stage("calculate_k")
    conv.stage("forward")
    conv.synchronize()
    assert np.array_equal(dt.cpu().numpy().view(np.uint32), want2["dst"].view(np.uint32))
    assert np.array_equal(conv.export_floats(capi.RES_K), want2["k"])
    conv.close()
    # (4) the switch is read when a descriptor is initialised: the K plane is then complete,
    # in device memory, when calculate_k returns (read raw here, not through the export
    # helper, which would settle a deferred filter)
    monkeypatch.setenv("XNOR_NN_HIP_SEPARATE_K", "1")
    conv = make(d, torch.from_numpy(w).to(gpu))
    dt.zero_()
    kt = torch.zeros(want1["k"].shape, dtype=torch.float32, device=gpu)  # a K plane of ours
    own_k = conv.res[capi.RES_K]
    conv.res[capi.RES_K] = kt.data_ptr()
    conv.stage("binarize_data", src=x1t, dst=dt)
    conv.stage("calculate_k")
    conv.synchronize()
    assert np.array_equal(kt.cpu().numpy(), want1["k"])
    conv.stage("forward")
    conv.synchronize()
    assert np.array_equal(dt.cpu().numpy().view(np.uint32), want1["dst"].view(np.uint32))
    conv.res[capi.RES_K] = own_k
    conv.close()


def test_linearity_of_scaling_at_full_size(gpu):
    """Size-independent property at benchmark size: scaling the input by 2 leaves the
    packed bits and popcounts unchanged and doubles dst exactly (k is linear in |x| and
    powers of two commute with rounding)."""
    import torch
    d, x, w = synth.make_workload("alexnet_conv4_mb256")
    xt = torch.from_numpy(x).to(gpu)
    wt = torch.from_numpy(w).to(gpu)
    shape = (d["mb"], d["oc"], d["ih"], d["iw"])
    y1 = torch.empty(shape, dtype=torch.float32, device=gpu)
    y2 = torch.empty(shape, dtype=torch.float32, device=gpu)
    conv = make(d, wt)
    conv.forward(xt, y1)
    b1 = conv.export_bin_src()
    conv.forward(xt * 2, y2)
    conv.synchronize()
    assert np.array_equal(conv.export_bin_src(), b1)
    assert torch.equal(y2, y1 * 2)
    conv.close()


def test_random_problems_until_the_time_is_up(oracle, monkeypatch):
    """Fifteen seconds of seeded random problems larger than the ones above (channel counts
    around the 32/64/1024 boundaries up to 2048, kernels 1..9, strides 1..4, paddings 0..4,
    images up to 43 x 43, every layout combination, inputs with exact zeros of both signs;
    every third problem with a two-tile-size launch forced on (four and two, four and three),
    every third with persistent workgroups forced on (one to three per XCD, so that each walks
    over many tiles), every sixth with the small-problem kernel forced on wherever it can run,
    every fourth with streaming output stores): dst and the raw popcounts against the oracle,
    bit for bit, stopping at the first mismatch.  XNOR_NN_TEST_RANDOM_SECONDS and
    XNOR_NN_TEST_RANDOM_SEED lengthen the run and move it to other problems."""
    import time
    rng = np.random.default_rng(int(os.environ.get("XNOR_NN_TEST_RANDOM_SEED", "20251")))
    t_end = time.time() + float(os.environ.get("XNOR_NN_TEST_RANDOM_SECONDS", "15"))
    n = 0
    while time.time() < t_end:
        kh, kw = int(rng.integers(1, 10)), int(rng.integers(1, 10))
        ph, pw = int(rng.integers(0, 5)), int(rng.integers(0, 5))
        sh, sw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        ih = int(rng.integers(max(1, kh - 2 * pw), 44))
        iw = int(rng.integers(max(1, kw - 2 * pw), 44))
        ic = int(rng.choice([1, 3, 4, 31, 32, 33, 64, 65, 96, 100, 128, 160, 200, 256, 257, 320,
                             384, 448, 512, 513, 640, 700, 1000, 1024, 1028, 1500, 2048]))
        oc = int(rng.choice([1, 7, 16, 31, 32, 33, 64, 65, 100, 128, 130, 256, 260, 384, 512,
                             600]))
        mb = int(rng.integers(1, 7))
        oh, ow = (ih + 2 * pw - kh) // sh + 1, (iw + 2 * pw - kw) // sw + 1
        if oh < 1 or ow < 1 or ih + 2 * ph < kh:
            continue
        if max(mb * ic * ih * iw, mb * oc * oh * ow, oc * ic * kh * kw) > 6e6:
            continue
        if mb * oc * oh * ow * ic * kh * kw > 4e10:
            continue
        fmts = (int(rng.choice([capi.FMT_NCHW, capi.FMT_NHWC])),
                int(rng.choice([capi.FMT_OIHW, capi.FMT_HWIO])),
                int(rng.choice([capi.FMT_NCHW, capi.FMT_NHWC])))
        d = dict(mb=mb, ic=ic, oc=oc, ih=ih, iw=iw, kh=kh, kw=kw, sh=sh, sw=sw, ph=ph, pw=pw)
        x = synth.normal(1000 + n, mb * ic * ih * iw).reshape(mb, ic, ih, iw)
        x.ravel()[::7] = 0.0
        x.ravel()[3::11] = -0.0
        w = synth.normal(5000 + n, oc * ic * kh * kw, 0.05).reshape(oc, ic, kh, kw)
        xs = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if fmts[0] == capi.FMT_NHWC else x
        ws = np.ascontiguousarray(w.transpose(2, 3, 1, 0)) if fmts[1] == capi.FMT_HWIO else w
        want = oracle.forward(oracle_shape(oracle, d, fmts), xs, ws)
        # launch options that the library otherwise picks by problem size
        forced = {"XNOR_NN_HIP_MFMA_MIX": "1" if n % 6 == 2 else "3" if n % 6 == 5 else None,
                  "XNOR_NN_HIP_MFMA_PERSIST": str(1 + n % 3) if n % 6 in (0, 3) else None,
                  "XNOR_NN_HIP_MFMA_SMALL": "1" if n % 6 == 1 else None,
                  "XNOR_NN_HIP_STREAM_DST": "1" if n % 4 == 3 else None}
        for key, value in forced.items():
            if value is None:
                monkeypatch.delenv(key, raising=False)
            else:
                monkeypatch.setenv(key, value)
        print("case", n, d, fmts, {k: v for k, v in forced.items() if v}, flush=True)
        conv = make(d, ws, fmts)
        dst = np.empty(want["dst"].shape, np.float32)
        conv.forward(xs, dst)
        ok = np.array_equal(dst.view(np.uint32), want["dst"].view(np.uint32)) \
            and np.array_equal(conv.forward_popcount(), want["popc"])
        name = conv.kernel_name(0)
        conv.close()
        assert ok, "case %d %s formats %s (%s)" % (n, d, fmts, name)
        n += 1
    assert n >= 5


@pytest.mark.parametrize("fmts", [NCHW, (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC)],
                         ids=["nchw", "nhwc_out"])
def test_streaming_output_stores(oracle, gpu, monkeypatch, fmts):
    """The matrix-core kernel stores large outputs with the streaming cache policy (chosen
    from the footprint at init; the full-size ResNet workload above takes it).  Forced on
    here for small and ragged shapes: same bits, whatever the policy."""
    monkeypatch.setenv("XNOR_NN_HIP_STREAM_DST", "1")
    for name, mb in (("alexnet_conv4_mb256", 5), ("resnet_3x3_mb64", 1), ("vgg_512_mb32", 1)):
        d, x, w = synth.make_workload(name, mb)
        run_and_compare(oracle, d, x, w, fmts, device_tensors=True, gpu=gpu)
    d = shapes.as_dims((2, 70, 100, 9, 7, 3, 3, 1, 1, 1, 1))  # ragged filters and planes
    x = synth.normal(141, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.normal(142, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    run_and_compare(oracle, d, x, w, fmts)


@pytest.mark.parametrize("t,fmts", [
    ((40, 384, 256, 13, 13, 3, 3, 1, 1, 1, 1), NCHW),                    # conv4: 212 blocks, 27 per XCD
    ((7, 384, 256, 13, 13, 3, 3, 1, 1, 1, 1), NCHW),                     # fewer blocks than XCDs x 4
    ((3, 96, 130, 27, 27, 5, 5, 1, 1, 2, 2), NCHW),                      # paired taps, ragged filters
    ((5, 64, 64, 28, 28, 3, 3, 2, 2, 1, 1), (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC)),
    ((2, 512, 200, 14, 14, 3, 3, 1, 1, 1, 1), NCHW),                     # 8 steps per tap
    ((1, 33, 32, 5, 5, 3, 3, 1, 1, 1, 1), NCHW),                         # a single pixel block
    ((3, 512, 512, 14, 14, 3, 3, 1, 1, 1, 1), NCHW),                     # two filter chunks
    ((6, 64, 600, 11, 9, 3, 3, 1, 1, 1, 1), (capi.FMT_NCHW, capi.FMT_HWIO, capi.FMT_NHWC)),
], ids=lambda v: shapes.shape_id(v) if len(v) == 11 else "fmt%d%d%d" % v)
@pytest.mark.parametrize("small", [2, 3])
def test_two_tile_sizes_in_one_launch(oracle, monkeypatch, t, fmts, small):
    """The matrix-core kernel with four-block tiles for the first workgroups of an XCD and
    two- or three-block tiles for the rest (chosen by size at init; the full-size conv4 and
    VGG workloads above take one each), forced on for problems whose XCD ranges end raggedly,
    hold no big tile, or have several filter chunks."""
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_MIX", "1" if small == 2 else "3")
    d = shapes.as_dims(t)
    x = synth.normal(151, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::6] = 0.0
    w = synth.normal(152, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    name = make(d, w, fmts).kernel_name(0)
    assert "PS=4+%d" % small in name, name
    run_and_compare(oracle, d, x, w, fmts)


@pytest.mark.parametrize("t,fmts", [
    ((40, 384, 256, 13, 13, 3, 3, 1, 1, 1, 1), NCHW),                    # conv4: 212 blocks, 27 per XCD
    ((7, 384, 256, 13, 13, 3, 3, 1, 1, 1, 1), NCHW),                     # fewer blocks than XCDs x 4
    ((3, 96, 130, 27, 27, 5, 5, 1, 1, 2, 2), NCHW),                      # paired taps, ragged filters
    ((5, 64, 64, 28, 28, 3, 3, 2, 2, 1, 1), (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC)),
    ((2, 512, 200, 14, 14, 3, 3, 1, 1, 1, 1), NCHW),                     # 8 steps per tap
    ((1, 33, 32, 5, 5, 3, 3, 1, 1, 1, 1), NCHW),                         # a single pixel block
    ((3, 512, 512, 14, 14, 3, 3, 1, 1, 1, 1), NCHW),                     # two filter chunks
    ((6, 64, 600, 11, 9, 3, 3, 1, 1, 1, 1), (capi.FMT_NCHW, capi.FMT_HWIO, capi.FMT_NHWC)),
    ((4, 256, 40, 56, 56, 3, 3, 1, 1, 1, 1), NCHW),                      # ResNet rows, one wave with filters
    ((9, 100, 70, 17, 23, 5, 3, 2, 1, 2, 1), NCHW),                      # strides, ragged everything
], ids=lambda v: shapes.shape_id(v) if len(v) == 11 else "fmt%d%d%d" % v)
@pytest.mark.parametrize("wgs", [1, 2, 3, 64])
def test_persistent_workgroups(oracle, monkeypatch, t, fmts, wgs):
    """The matrix-core kernel with workgroups that stay and walk over their tiles (chosen by
    size at init when a workgroup slot gets six pixel blocks or more; the full-size ResNet and
    conv2-shape workloads above take it), forced on here with `wgs` workgroups per XCD: with
    one to three of them every workgroup walks over many tiles of both sizes, copies the next
    tile's packed words into LDS while it multiplies, and meets XCD ranges that end raggedly;
    with 64 most workgroups get one tile or none."""
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_PERSIST", str(wgs))
    d = shapes.as_dims(t)
    x = synth.normal(161, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::6] = 0.0
    w = synth.normal(162, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    xs = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if fmts[0] == capi.FMT_NHWC else x
    ws = np.ascontiguousarray(w.transpose(2, 3, 1, 0)) if fmts[1] == capi.FMT_HWIO else w
    name = make(d, ws, fmts).kernel_name(0)
    chunks = (d["oc"] + 255) // 256
    if wgs >= chunks:
        assert name.startswith("conv_mfma_fp4_persistent_kernel"), name
    run_and_compare(oracle, d, xs, ws, fmts)


@pytest.mark.parametrize("separate_k", [False, True], ids=["fused_k", "k_plane"])
@pytest.mark.parametrize("t,fmts", [
    ((1, 256, 384, 13, 13, 3, 3, 1, 1, 1, 1), NCHW),                     # conv4, minibatch 1
    ((3, 100, 70, 9, 7, 3, 3, 1, 1, 1, 1), NCHW),                        # ragged filters, channels, pixels
    ((2, 64, 64, 28, 28, 3, 3, 2, 2, 1, 1), (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC)),
    ((1, 512, 33, 14, 14, 1, 1, 1, 1, 0, 0), NCHW),                      # one tap, eight steps
    ((2, 40, 128, 6, 5, 5, 5, 1, 1, 2, 2), (capi.FMT_NHWC, capi.FMT_HWIO, capi.FMT_NCHW)),
    ((1, 1000, 16, 4, 4, 3, 3, 1, 1, 1, 1), NCHW),                       # sixteen steps per tap
    ((1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0), NCHW),                           # the smallest problem
    ((5, 600, 64, 3, 3, 7, 7, 4, 4, 3, 3), NCHW),                        # kernel wider than the image
], ids=lambda v: shapes.shape_id(v) if len(v) == 11 else "fmt%d%d%d" % v)
def test_small_problem_kernel(oracle, monkeypatch, t, fmts, separate_k):
    """The matrix-core kernel for launches of few tiles (a workgroup per 32 pixels x 32 filters,
    the four waves splitting the taps and adding their exact partial sums through LDS; chosen
    by size at init, conv4 at minibatch 1 takes it), forced on here for ragged and odd shapes,
    with K summed in the kernel and with K read from the plane."""
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_SMALL", "1")
    if separate_k:
        monkeypatch.setenv("XNOR_NN_HIP_SEPARATE_K", "1")
    d = shapes.as_dims(t)
    x = synth.normal(171, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::5] = 0.0
    w = synth.normal(172, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    xs = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if fmts[0] == capi.FMT_NHWC else x
    ws = np.ascontiguousarray(w.transpose(2, 3, 1, 0)) if fmts[1] == capi.FMT_HWIO else w
    name = make(d, ws, fmts).kernel_name(0)
    assert name.startswith("conv_mfma_fp4_small_kernel"), name
    run_and_compare(oracle, d, xs, ws, fmts)


@pytest.mark.parametrize("separate_k", [False, True], ids=["fused_k", "k_plane"])
@pytest.mark.parametrize("ps", ["1", "2", "3", "4"])
@pytest.mark.parametrize("t,fmts,groups", [
    ((3, 64, 64, 20, 20, 3, 3, 1, 1, 1, 1), NCHW, 4),                    # one wave's filters
    ((2, 100, 33, 17, 13, 3, 3, 1, 1, 1, 1), NCHW, 4),                   # ragged everything
    ((2, 96, 128, 15, 15, 5, 5, 1, 1, 2, 2), NCHW, 2),                   # tap pairs, two waves' filters
    ((3, 128, 100, 14, 14, 3, 3, 2, 2, 1, 1), (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC), 2),
    ((2, 40, 64, 12, 11, 3, 3, 1, 1, 1, 1), (capi.FMT_NHWC, capi.FMT_HWIO, capi.FMT_NHWC), 4),
    ((1, 256, 7, 23, 9, 1, 1, 1, 1, 0, 0), NCHW, 4),                     # 1x1, seven filters
    ((5, 32, 65, 9, 9, 3, 3, 1, 1, 1, 1), NCHW, 2),                      # one filter in the second wave
    ((1, 64, 16, 5, 5, 3, 3, 1, 1, 1, 1), NCHW, 4),                      # one block: three groups past the end
], ids=lambda v: shapes.shape_id(v) if isinstance(v, tuple) and len(v) == 11
   else "fmt%d%d%d" % v if isinstance(v, tuple) else "groups%d" % v)
def test_pixel_groups_for_few_filters(oracle, monkeypatch, t, fmts, groups, ps, separate_k):
    """With 128 filters or fewer the waves of a workgroup that would have no filters take the
    same filters on further pixel blocks (two or four pixel groups per tile): every tile size,
    ragged filter counts, both output layouts, strides, tap pairs, K summed in the kernel and
    read from its plane, tiles whose later groups lie past the last pixel; and the same
    problems with the groups switched off."""
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_SMALL", "0")
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_PS", ps)
    if separate_k:
        monkeypatch.setenv("XNOR_NN_HIP_SEPARATE_K", "1")
    d = shapes.as_dims(t)
    x = synth.normal(271, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::5] = 0.0
    w = synth.normal(272, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    xs = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if fmts[0] == capi.FMT_NHWC else x
    ws = np.ascontiguousarray(w.transpose(2, 3, 1, 0)) if fmts[1] == capi.FMT_HWIO else w
    name = make(d, ws, fmts).kernel_name(0)
    assert name.endswith("PS=%s%s,GROUPS=%d>" % (ps, ",PAIR" if "PAIR" in name else "", groups)), name
    run_and_compare(oracle, d, xs, ws, fmts)
    if not separate_k and ps == "2":
        monkeypatch.setenv("XNOR_NN_HIP_MFMA_GROUPS", "1")
        assert "GROUPS" not in make(d, ws, fmts).kernel_name(0)
        run_and_compare(oracle, d, xs, ws, fmts)
