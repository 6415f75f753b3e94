"""Pins the CPU oracle (oracle/xnor_oracle.c) without needing the upstream library:
the upstream tests' known-answer vectors, closed forms, brute force on small inputs, and
the committed digests of the upstream library's outputs (tests/golden/golden.json)."""
import os

import numpy as np
import pytest

import shapes
from util import brute_force_dot, oracle_shape, sha256
from xnor_nn_amd import capi, synth

P, N = 1.0, -1.0
# reference test/gtest/test_convolution_reference_forward.cpp:20-52
KA_SRC = np.array([P, P, P, N, P, N, N, N, N,
                   N, N, N, N, N, N, P, P, P], dtype=np.float32).reshape(1, 2, 3, 3)
KA_W = np.array([P, P, P, N, N, P, P, N, N,
                 P, P, P, P, P, P, P, P, P,
                 N, N, N, N, N, N, N, N, N,
                 P, P, P, N, N, P, P, N, N], dtype=np.float32).reshape(2, 2, 3, 3)
# reference test/gtest/test_convolution_reference_forward.cpp:58-73 (times 1/9)
KA_DST = np.array([-16, -48, -16, 24, 0, 0, 0, 0, 8,
                   0, 0, 0, -24, -18, 0, 0, 0, -8], dtype=np.float32).reshape(1, 2, 3, 3) / 9
KA_DIMS = dict(mb=1, ic=2, oc=2, ih=3, iw=3, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1)


def test_known_answer_a_and_k(oracle):
    """a == 1 and k = {4,6,4,6,9,6,4,6,4}/9
    (reference test/gtest/test_data_bin_reference.cpp:43-53), tolerance 1e-5 as there."""
    s = oracle_shape(oracle, KA_DIMS)
    a, k = oracle.calculate_k(s, KA_SRC)
    assert np.array_equal(a, np.ones((1, 3, 3), np.float32))
    want = np.array([4, 6, 4, 6, 9, 6, 4, 6, 4], np.float32).reshape(1, 3, 3) / 9
    assert np.allclose(k, want, atol=1e-5, rtol=0)


def test_known_answer_alpha(oracle):
    """alpha = {1, 1} (reference test/gtest/test_weights_bin_reference.cpp:50)."""
    s = oracle_shape(oracle, KA_DIMS)
    _, alpha, _ = oracle.binarize_weights(s, KA_W, oci=2)
    assert np.allclose(alpha, [1, 1], atol=1e-5, rtol=0)


@pytest.mark.parametrize("src_fmt,w_fmt,dst_fmt", [
    (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW),
    (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NHWC),
    (capi.FMT_NHWC, capi.FMT_HWIO, capi.FMT_NCHW),
    (capi.FMT_NHWC, capi.FMT_HWIO, capi.FMT_NHWC),
])
def test_known_answer_forward(oracle, src_fmt, w_fmt, dst_fmt):
    """The 18 precomputed outputs, in all four layout combinations, absolute tolerance
    1e-3 as in reference test/gtest/common.hpp:146-161."""
    s = oracle_shape(oracle, KA_DIMS, (src_fmt, w_fmt, dst_fmt))
    x = KA_SRC if src_fmt == capi.FMT_NCHW else KA_SRC.transpose(0, 2, 3, 1)
    w = KA_W if w_fmt == capi.FMT_OIHW else KA_W.transpose(2, 3, 1, 0)
    want = KA_DST if dst_fmt == capi.FMT_NCHW else KA_DST.transpose(0, 2, 3, 1)
    out = oracle.forward(s, np.ascontiguousarray(x), np.ascontiguousarray(w), oci=2)
    assert np.allclose(out["dst"], want, atol=1e-3, rtol=0)


def test_sign_convention_zero_and_nan(oracle):
    """bit = IEEE sign bit clear: +0 -> 1, -0 -> 0, NaN by its sign
    (reference src/bcast_binarize_data.cpp:61)."""
    vals = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 1e-45, -1e-45], np.float32)
    x = np.zeros((1, 8, 1, 1), np.float32)
    x[0, :, 0, 0] = vals
    d = dict(mb=1, ic=8, oc=16, ih=1, iw=1, kh=1, kw=1, sh=1, sw=1, ph=0, pw=0)
    s = oracle_shape(oracle, d)
    assert oracle.binarize_data(s, x)[0] == 0b10101010
    x.view(np.uint32)[0, 0, 0, 0] = 0x7FC00000  # +NaN
    x.view(np.uint32)[0, 1, 0, 0] = 0xFFC00000  # -NaN
    assert oracle.binarize_data(s, x)[0] == 0b10101010


@pytest.mark.parametrize("ic", [1, 3, 7, 8, 9, 15, 16, 17, 31, 33, 96])
def test_data_bits_closed_form_and_padding(oracle, ic):
    """Every real bit under the index formula of the reference's checker
    (reference test/gtest/common.hpp:68-98); tail bits and pad bytes are zero
    (reference src/bcast_binarize_data.cpp:65-72)."""
    d = dict(mb=2, ic=ic, oc=16, ih=3, iw=5, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1)
    s = oracle_shape(oracle, d)
    x = synth.normal(11 + ic, 2 * ic * 15).reshape(2, ic, 3, 5)
    packed = oracle.binarize_data(s, x)
    bici = 2
    abic = ((ic + 7) // 8 + bici - 1) // bici * bici
    packed = packed.reshape(2, 3, 5, abic)
    bits = np.unpackbits(packed, axis=-1)  # MSB first, like the reference
    want = (~np.signbit(x)).transpose(0, 2, 3, 1).astype(np.uint8)
    assert np.array_equal(bits[..., :ic], want)
    assert not bits[..., ic:].any()


@pytest.mark.parametrize("ic,oc", [(3, 16), (20, 32), (33, 16)])
def test_weight_bits_closed_form_and_ones_tail(oracle, ic, oc):
    """Index formula of reference test/gtest/common.hpp:101-144; bits of channels >= IC
    are ones (reference src/bcast_binarize_weights.cpp:80-88)."""
    d = dict(mb=1, ic=ic, oc=oc, ih=5, iw=5, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1)
    s = oracle_shape(oracle, d)
    w = synth.normal(5, oc * ic * 9, 0.05).reshape(oc, ic, 3, 3)
    packed, alpha, opc = oracle.binarize_weights(s, w)
    bici, oci = 2, 16
    ico = ((ic + bici - 1) // bici + 7) // 8
    packed = packed.reshape(oc // oci, 3, 3, ico, oci, bici)
    bits = np.unpackbits(packed, axis=-1).reshape(oc // oci, 3, 3, ico, oci, bici * 8)
    # channel c lives in word c // 16 at bit c % 16 of that word's MSB-first bit string
    got = bits.transpose(0, 4, 3, 5, 1, 2).reshape(oc, ico * bici * 8, 3, 3)
    assert np.array_equal(got[:, :ic], (~np.signbit(w)).astype(np.uint8))
    assert got[:, ic:].all()
    # alpha is the mean of |w| (float64 check, loose) and opc = IC * valid taps
    assert np.allclose(alpha, np.abs(w.astype(np.float64)).mean(axis=(1, 2, 3)), rtol=1e-5)
    vh = np.array([3 - (h == 0) - (h == 4) for h in range(5)])
    assert np.array_equal(opc, ic * np.outer(vh, vh))


@pytest.mark.parametrize("t", [
    (2, 5, 16, 6, 7, 3, 3, 1, 1, 1, 1),
    (1, 40, 32, 9, 9, 5, 5, 1, 1, 2, 2),
    (2, 3, 16, 23, 23, 11, 11, 4, 4, 0, 0),
    (1, 17, 16, 8, 6, 3, 3, 2, 2, 1, 1),
], ids=shapes.shape_id)
def test_convolution_brute_force(oracle, t):
    """2*popc - n equals the +-1 dot product over in-bounds taps computed from the raw
    floats; n = IC * in-bounds taps; dst = (2*popc - n) * alpha * k rounded per product."""
    d = shapes.as_dims(t)
    s = oracle_shape(oracle, d)
    x = synth.normal(21, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::7] = 0.0
    x.ravel()[3::11] = -0.0
    w = synth.normal(22, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    out = oracle.forward(s, x, w)
    dot, n = brute_force_dot(x, w, d)
    assert np.array_equal(out["opc"], n)
    assert np.array_equal(2 * out["popc"].astype(np.int64) - n[None, None], dot)
    want = ((dot.astype(np.float32) * out["alpha"][None, :, None, None]).astype(np.float32)
            * out["k"][:, None]).astype(np.float32)
    assert np.array_equal(out["dst"], want)


def test_all_ones_input_invariants(oracle):
    """x == 1 everywhere: a == IC * fl(1/IC) summed in order, k = taps/(KH*KW) up to
    rounding, and every in-bounds product is sgn(w)."""
    d = dict(mb=1, ic=8, oc=16, ih=6, iw=6, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1)
    s = oracle_shape(oracle, d)
    x = np.ones((1, 8, 6, 6), np.float32)
    a, k = oracle.calculate_k(s, x)
    assert np.array_equal(a, np.ones_like(a))  # 8 * 0.125 is exact
    vh = np.array([3 - (h == 0) - (h == 5) for h in range(6)], np.float64)
    assert np.allclose(k[0], np.outer(vh, vh) / 9, rtol=1e-6)


def test_golden_tiny_case_in_full(oracle, golden):
    """Inputs and every output of the upstream library on a tiny case, stored as numbers."""
    g = golden["tiny_full"]
    d = g["dims"]
    x = np.array(g["src_bits"], np.uint32).view(np.float32).reshape(d["mb"], d["ic"], d["ih"], d["iw"])
    w = np.array(g["weights_bits"], np.uint32).view(np.float32).reshape(d["oc"], d["ic"], d["kh"], d["kw"])
    out = oracle.forward(oracle_shape(oracle, d), x, w)
    assert out["bin_src"].tolist() == g["bin_src"]
    assert out["bin_weights"].tolist() == g["bin_weights"]
    assert out["a"].view(np.uint32).ravel().tolist() == g["a_bits"]
    assert out["k"].view(np.uint32).ravel().tolist() == g["k_bits"]
    assert out["alpha"].view(np.uint32).ravel().tolist() == g["alpha_bits"]
    assert out["opc"].ravel().tolist() == g["opc"]
    assert out["dst"].view(np.uint32).ravel().tolist() == g["dst_bits"]


@pytest.mark.parametrize("t", shapes.COMPARE_WITH_REFERENCE, ids=shapes.shape_id)
def test_golden_reference_test_shapes(oracle, golden, t):
    """Oracle output digests == digests of the upstream library's output on the shapes and
    closed-form inputs of its own differential test."""
    g = golden["reference_test_shapes"][shapes.shape_id(t)]
    d = shapes.as_dims(t)
    x = synth.reference_test_src(d["mb"], d["ic"], d["ih"], d["iw"])
    w = synth.reference_test_weights(d["oc"], d["ic"], d["kh"], d["kw"])
    out = oracle.forward(oracle_shape(oracle, d), x, w)
    for key, want in g["sha256"].items():
        assert sha256(out[key]) == want, key


@pytest.mark.parametrize("name", ["alexnet_conv4_mb1", "alexnet_conv4_mb256"])
def test_golden_workloads(oracle, golden, name):
    """Same at benchmark size for the two AlexNet conv4 workloads (the larger ones are
    covered by the GPU suite, which also checks the oracle against these digests)."""
    g = golden["workloads"][name]
    d, x, w = synth.make_workload(name)
    out = oracle.forward(oracle_shape(oracle, d), x, w)
    for key, want in g["sha256"].items():
        assert sha256(out[key]) == want, key


def test_binarize_weights_float_closed_forms(oracle):
    """sign(w) * mean(w) (reference src/binarize_weights_float.cpp:3-25): the mean is of the
    weights themselves, not of their magnitudes; -0.0 counts as >= 0; the sum runs in index
    order in float."""
    s = oracle.shape(1, 4, 3, 5, 5, 3, 3, 1, 1, 1, 1)
    n = 4 * 3 * 3 * 3
    ones = np.ones(n, np.float32)
    assert np.array_equal(oracle.binarize_weights_float(s, ones), ones)
    # alternating +-c sums to exactly zero (n is even): the outputs are zeros whose sign is
    # that of the weight
    alt = np.where(np.arange(n) % 2 == 0, np.float32(0.75), np.float32(-0.75))
    out = oracle.binarize_weights_float(s, alt)
    assert np.all(out == 0) and np.array_equal(np.signbit(out), alt < 0)
    # a negative zero is "not negative"
    w = np.full(n, 2.0, np.float32)
    w[5] = -0.0
    w[6] = -1.0
    out = oracle.binarize_weights_float(s, w)
    mean = np.float32(np.float32((n - 2) * 2.0 - 1.0) * np.float32(1.0 / n))
    want = np.full(n, mean, np.float32)
    want[6] = -mean
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    # sequential float sum, then one multiply by 1.f/n: restated with numpy scalars
    w = synth.normal(5, n, 0.05)
    acc = np.float32(0)
    for v in w:
        acc = np.float32(acc + v)
    mean = np.float32(acc * np.float32(1.0 / n))
    want = np.where(w >= 0, mean, -mean).astype(np.float32)
    assert np.array_equal(oracle.binarize_weights_float(s, w).view(np.uint32),
                          want.view(np.uint32))
    assert abs(float(mean) - float(np.mean(w.astype(np.float64)))) < 1e-7


def test_oracle_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    """tests/oracle_sanitize.c compiles the oracle's source into a host program with
    -fsanitize=address,undefined and runs every stage over small and ragged shapes in all
    eight layout combinations on exactly sized heap buffers: an index outside a tensor or
    undefined arithmetic in the restatement ends it with a report."""
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    exe = tmp_path / "oracle_sanitize"
    subprocess.check_call(["gcc", "-std=c11", "-O1", "-g", "-fopenmp", "-ffp-contract=off",
                           "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                           "-static-libasan", os.path.join(here, "oracle_sanitize.c"), "-lm",
                           "-o", str(exe)])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, (out.stdout[-1000:], out.stderr[-3000:])
    assert out.stdout.strip().endswith("0 bad")
