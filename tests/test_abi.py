"""The C-ABI boundary without a GPU: the library loads, exports every function that
include/*.h declares, the descriptor has the layout a C compiler gives it, and the host-only
entry points behave like the reference's."""
import ctypes as C
import os
import re
import subprocess

import pytest

from xnor_nn_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


def declared_functions():
    names = set()
    for header in ("xnor_nn.h", "xnor_nn_hip.h"):
        text = open(os.path.join(INCLUDE, header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(xnor_nn_\w+)\s*\(", text))
    return sorted(names)


def test_every_declared_symbol_is_exported():
    lib = C.CDLL(capi.library_path())
    names = declared_functions()
    assert len(names) >= 16
    for name in names:
        assert hasattr(lib, name), name
    # and the ctypes tables cover exactly the declared set
    assert set(names) == set(capi.CORE_SYMBOLS) | set(capi.HIP_SYMBOLS)


def test_descriptor_layout_matches_a_c_compiler(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "xnor_nn.h"
#include "xnor_nn_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(xnor_nn_convolution_t),
        offsetof(xnor_nn_convolution_t, mb), offsetof(xnor_nn_convolution_t, src_format),
        offsetof(xnor_nn_convolution_t, resource_size),
        offsetof(xnor_nn_convolution_t, binarize_weights),
        offsetof(xnor_nn_convolution_t, forward), offsetof(xnor_nn_convolution_t, state),
        sizeof(xnor_nn_resources_t));
    printf("%d %d %d %d %d %d\n", xnor_nn_unimplemented, xnor_nn_algorithm_bcast,
        xnor_nn_resource_operations_count, xnor_nn_resource_number,
        xnor_nn_weights_format_hwio, xnor_nn_operation_calculate_k);
    return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-I", INCLUDE,
                           str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)]).decode().split()
    D = capi.ConvolutionDesc
    want = [C.sizeof(D), D.mb.offset, D.src_format.offset, D.resource_size.offset,
            D.binarize_weights.offset, D.forward.offset, D.state.offset,
            C.sizeof(capi.Resources)]
    assert [int(v) for v in out[:8]] == want
    assert [int(v) for v in out[8:]] == [3, 1, 8, 9, 3, 3]


def test_cpp_wrapper_header_compiles(tmp_path):
    src = tmp_path / "wrap.cpp"
    src.write_text('#include "xnor_nn.hpp"\n'
                   'int use(const void *w) { xnor_nn::Convolution c{xnor_nn_algorithm_bcast,'
                   ' xnor_nn_data_format_nchw, xnor_nn_weights_format_oihw,'
                   ' xnor_nn_data_format_nchw, 1, 16, 8, 5, 5, 3, 3, 1, 1, 1, 1, w};'
                   ' return 0; }\n')
    subprocess.check_call(["g++", "-std=c++14", "-Wall", "-Werror", "-fsyntax-only",
                           "-I", INCLUDE, str(src)])


def test_status_messages():
    """reference src/status.cpp:3-15"""
    lib = capi.load()
    assert [capi.status_message(lib, s) for s in range(4)] == [
        "success", "memory_error", "bad_input", "unimplemented"]


def test_init_fills_descriptor_like_the_reference():
    """reference src/common_convolution.cpp:9-63: every field set, oh AND ow from pw,
    always success; plus this library's device buffer sizes."""
    lib = capi.load()
    c = capi.ConvolutionDesc()
    st = lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW,
                                      capi.FMT_OIHW, capi.FMT_NCHW,
                                      4, 256, 96, 27, 27, 5, 5, 1, 1, 2, 2)
    assert st == capi.SUCCESS
    assert (c.mb, c.ic, c.ih, c.iw, c.oc, c.oh, c.ow) == (4, 96, 27, 27, 256, 27, 27)
    assert (c.kh, c.kw, c.sh, c.sw, c.ph, c.pw) == (5, 5, 1, 1, 2, 2)
    assert c.state and all((c.binarize_weights, c.binarize_data, c.calculate_k, c.forward))
    assert c.resource_size[capi.RES_BIN_SRC] == 4 * 27 * 27 * 3 * 4
    # packed sign words [OC/16][taps][words][16], then the same signs as FP4 matrix-core
    # fragments [OC/32][units][steps][64 lanes][16 bytes]; IC = 96 is three 32-channel words,
    # an odd number, so a unit is a pair of taps (13 for 25 taps) of 3 steps
    assert c.resource_size[capi.RES_BIN_WEIGHTS] == 16 * 25 * 3 * 16 * 4 + 8 * 13 * 3 * 64 * 16
    assert c.resource_size[capi.RES_A] == c.resource_size[capi.RES_K] == 4 * 27 * 27 * 4
    assert c.resource_size[capi.RES_ALPHA] == 256 * 4
    assert c.resource_size[capi.RES_OPERATIONS_COUNT] == 27 * 27 * 4
    # oh uses pw, not ph (reference src/common_convolution.cpp:16)
    lib.xnor_nn_destroy_convolution(C.byref(c))
    assert not c.state
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, 0, 2, 0,
                                 1, 16, 8, 10, 10, 3, 3, 1, 1, 0, 1)
    assert (c.oh, c.ow) == (10, 10)
    lib.xnor_nn_destroy_convolution(C.byref(c))
    lib.xnor_nn_destroy_convolution(C.byref(c))  # idempotent


def test_null_and_format_checks_of_the_executors():
    """Same status codes as the reference for missing slots
    (reference src/bcast_binarize_data.cpp:15-19, src/bcast_calculate_k.cpp:15-20,
    src/bcast_binarize_weights.cpp:15-21, src/default/bcast_convolution_default.cpp:25-33)
    and unknown formats (reference src/bcast_binarize_data.cpp:36-38).  No GPU needed: the
    checks come before any device work."""
    lib = capi.load()
    c = capi.ConvolutionDesc()
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW,
                                 capi.FMT_OIHW, capi.FMT_NCHW, 1, 16, 8, 5, 5, 3, 3, 1, 1, 1, 1)
    res = capi.Resources()
    for stage in ("binarize_data", "calculate_k", "binarize_weights", "forward"):
        assert getattr(c, stage)(C.byref(c), res) == capi.ERROR_INVALID_INPUT, stage
    lib.xnor_nn_free_resources(res)  # safe on a zeroed table
    lib.xnor_nn_destroy_convolution(C.byref(c))

    dummy = (C.c_float * 4)()
    for i in range(capi.RES_NUMBER):
        res[i] = C.addressof(dummy)
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, 7, 9, 11,
                                 1, 16, 8, 5, 5, 3, 3, 1, 1, 1, 1)
    for stage in ("binarize_data", "calculate_k", "binarize_weights", "forward"):
        assert getattr(c, stage)(C.byref(c), res) == capi.UNIMPLEMENTED, stage
    lib.xnor_nn_destroy_convolution(C.byref(c))


def test_reference_algorithm_has_no_gpu_path():
    lib = capi.load()
    c = capi.ConvolutionDesc()
    st = lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_REFERENCE, 0, 2, 0,
                                      1, 16, 8, 5, 5, 3, 3, 1, 1, 1, 1)
    assert st == capi.SUCCESS and not c.state
    res = capi.Resources()
    assert c.forward(C.byref(c), res) == capi.UNIMPLEMENTED
    lib.xnor_nn_destroy_convolution(C.byref(c))


def test_word_size_of_the_exported_layout():
    """The export helpers hand out the reference's CPU layout, whose packed words are 16 bits
    wide while IC*KH*KW < 32767 and 32 bits wide from there on (reference
    src/implementation.cpp:17-22, src/convolution_traits.hpp:29-56)."""
    lib = capi.load()
    for ic, want in ((384, 2), (3640, 2), (3641, 4), (4000, 4)):
        c = capi.ConvolutionDesc()
        lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, 0, 2, 0,
                                     1, 16, ic, 5, 5, 3, 3, 1, 1, 1, 1)
        assert lib.xnor_nn_hip_canonical_bici(C.byref(c)) == want, ic
        lib.xnor_nn_destroy_convolution(C.byref(c))


def test_package_does_not_touch_the_oracle():
    """The oracle is test infrastructure: nothing under xnor_nn_amd/ may name it."""
    pkg = os.path.join(ROOT, "xnor_nn_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text.lower(), os.path.join(base, f)


@pytest.mark.skipif(not os.path.isdir("/root/reference/example"),
                    reason="upstream sources not mounted")
@pytest.mark.parametrize("name,cc", [("simple_convolution.c", "gcc"),
                                     ("simple_convolution.cpp", "g++")])
def test_upstream_examples_compile_and_link_unchanged(tmp_path, name, cc):
    """The reference's own example programs (reference example/simple_convolution.c,
    .cpp) build against include/ and link to libxnor_nn.so without edits."""
    exe = tmp_path / "example"
    libdir = os.path.dirname(capi.library_path())
    subprocess.check_call([cc, "-I", INCLUDE, os.path.join("/root/reference/example", name),
                           "-L", libdir, "-lxnor_nn", "-Wl,-rpath," + libdir,
                           "-Wl,-rpath-link,/opt/rocm/lib", "-o", str(exe)])


def test_forward_popcount_needs_only_the_two_packed_tensors():
    """xnor_nn_hip_forward_popcount checks exactly the slots its header names: bin_src,
    bin_weights and the output pointer (host-only: the checks come before device work)."""
    lib = capi.load()
    c = capi.ConvolutionDesc()
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW,
                                 capi.FMT_OIHW, capi.FMT_NCHW, 1, 16, 8, 5, 5, 3, 3, 1, 1, 1, 1)
    res = capi.Resources()
    out = (C.c_int32 * (16 * 25))()
    assert lib.xnor_nn_hip_forward_popcount(C.byref(c), res, out) == capi.ERROR_INVALID_INPUT
    dummy = (C.c_float * 4)()
    res[capi.RES_BIN_SRC] = C.addressof(dummy)
    assert lib.xnor_nn_hip_forward_popcount(C.byref(c), res, out) == capi.ERROR_INVALID_INPUT
    res[capi.RES_BIN_WEIGHTS] = C.addressof(dummy)
    assert lib.xnor_nn_hip_forward_popcount(C.byref(c), res, None) == capi.ERROR_INVALID_INPUT
    lib.xnor_nn_destroy_convolution(C.byref(c))
    # a descriptor without the bcast state has no popcount path
    assert lib.xnor_nn_hip_forward_popcount(C.byref(c), res, out) == capi.ERROR_INVALID_INPUT
    assert lib.xnor_nn_hip_set_stage_fusion(C.byref(c), 0) == capi.ERROR_INVALID_INPUT


def test_stage_fusion_switch_and_table_bookkeeping_without_a_gpu():
    """The switch is per descriptor; freeing a zeroed or hand-filled table and destroying a
    descriptor that never ran are safe (the hand-over bookkeeping is keyed on buffers)."""
    lib = capi.load()
    c = capi.ConvolutionDesc()
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW,
                                 capi.FMT_OIHW, capi.FMT_NCHW, 1, 16, 8, 5, 5, 3, 3, 1, 1, 1, 1)
    assert lib.xnor_nn_hip_set_stage_fusion(C.byref(c), 0) == capi.SUCCESS
    assert lib.xnor_nn_hip_set_stage_fusion(C.byref(c), 1) == capi.SUCCESS
    res = capi.Resources()
    lib.xnor_nn_free_resources(res)
    lib.xnor_nn_destroy_convolution(C.byref(c))


def kernel_names(shape, fmts=(capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW)):
    """(binarize kernel, convolution kernel) the library plans for a shape
    (mb, oc, ic, ih, iw, kh, kw, sh, sw, ph, pw); planning needs no GPU (256 CUs assumed)."""
    lib = capi.load()
    c = capi.ConvolutionDesc()
    assert lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, *fmts, *shape) \
        == capi.SUCCESS
    buf = C.create_string_buffer(96)
    out = []
    for stage in (capi.OP_BINARIZE_DATA, capi.OP_CONVOLUTION_FORWARD):
        lib.xnor_nn_hip_kernel_name(C.byref(c), stage, buf, len(buf))
        out.append(buf.value.decode())
    lib.xnor_nn_destroy_convolution(C.byref(c))
    return tuple(out)


def test_kernel_variants_planned_for_known_shapes(monkeypatch):
    """The counterpart of the reference's dispatcher (reference src/bcast_convolution.hpp:13-38,
    src/bcast_convolution.cpp:14-43: exact-match table of shapes -> unrolled kernel, else the
    runtime-shape kernel): which kernel variant each of the five benchmark workloads and the
    boundary shapes get, decided at init from the shape alone."""
    for key in ("XNOR_NN_HIP_CONV", "XNOR_NN_HIP_MFMA_PS", "XNOR_NN_HIP_MFMA_MIX",
                "XNOR_NN_HIP_MFMA_PAIR", "XNOR_NN_HIP_NHWC", "XNOR_NN_HIP_STREAM_DST",
                "XNOR_NN_HIP_MFMA_PERSIST", "XNOR_NN_HIP_MFMA_SMALL", "XNOR_NN_HIP_MFMA_GROUPS"):
        monkeypatch.delenv(key, raising=False)
    conv4 = (256, 384, 13, 13, 3, 3, 1, 1, 1, 1)
    # 6 pixel blocks x 8 filter blocks: fewer (block, block) pairs than compute units
    assert kernel_names((1,) + conv4) == ("binarize_nchw_kernel", "conv_mfma_fp4_small_kernel<KS=6>")
    assert kernel_names((8,) + conv4)[1] == "conv_mfma_fp4_small_kernel<KS=6>"
    # up to two pairs per compute unit when a wave would walk 48 steps or more (here 54)
    assert kernel_names((12,) + conv4)[1] == "conv_mfma_fp4_small_kernel<KS=6>"
    assert kernel_names((16,) + conv4)[1] == "conv_mfma_fp4_kernel<KS=6,PS=1>"
    # 36 steps: the large-launch kernel from 1.5 pairs per compute unit
    assert kernel_names((8, 256, 256, 14, 14, 3, 3, 1, 1, 1, 1))[1] == "conv_mfma_fp4_kernel<KS=4,PS=1>"
    # 5.3 pixel blocks per compute unit: two tile sizes in one launch
    assert kernel_names((256,) + conv4)[1] == "conv_mfma_fp4_kernel<KS=6,PS=4+2>"
    assert kernel_names((1024,) + conv4)[1] == "conv_mfma_fp4_kernel<KS=6,PS=4>"
    # 96 channels = three words: two taps share three steps; several rounds of tiles with at
    # most four steps per tap: tiles of two blocks, three workgroups to a compute unit
    assert kernel_names((128, 256, 96, 27, 27, 5, 5, 1, 1, 2, 2))[1] \
        == "conv_mfma_fp4_kernel<KS=3,PS=2,PAIR>"
    assert kernel_names((64, 256, 256, 56, 56, 3, 3, 1, 1, 1, 1))[1] \
        == "conv_mfma_fp4_kernel<KS=4,PS=2>"
    # 64 filters are one wave's worth: the other three waves take further pixel blocks; 128
    # filters: two pixel groups
    assert kernel_names((64, 64, 64, 56, 56, 3, 3, 1, 1, 1, 1))[1] \
        == "conv_mfma_fp4_kernel<KS=1,PS=2,GROUPS=4>"
    assert kernel_names((64, 128, 128, 56, 56, 3, 3, 1, 1, 1, 1))[1] \
        == "conv_mfma_fp4_kernel<KS=2,PS=2,GROUPS=2>"
    # 98 blocks for 32 slots per XCD and filter chunk: 2 tiles of four, 30 of three
    assert kernel_names((32, 512, 512, 28, 28, 3, 3, 1, 1, 1, 1))[1] \
        == "conv_mfma_fp4_kernel<KS=8,PS=4+3>"
    # more than 1024 channels: channel parts; more than 4096: no matrix cores
    assert re.fullmatch(r"conv_mfma_fp4_kernel<KS=1[26],PS=\d,PARTS=\d>",
                        kernel_names((2, 64, 2048, 8, 8, 3, 3, 1, 1, 1, 1))[1])
    deep = kernel_names((1, 32, 8200, 4, 4, 1, 1, 1, 1, 0, 0))
    assert deep[0] == "binarize_generic_kernel" and deep[1] == "conv_xnor_popc_kernel<XW=0,Q=16>"  # XW=0: word count at run time
    # kernels wider than 32 taps keep their tap masks in 32 bits: XNOR/popcount kernel
    assert kernel_names((1, 16, 32, 40, 40, 33, 33, 1, 1, 0, 0))[1].startswith("conv_xnor_popc")
    # input layouts
    nhwc = (capi.FMT_NHWC, capi.FMT_OIHW, capi.FMT_NCHW)
    assert kernel_names((4,) + conv4, nhwc)[0] == "binarize_nhwc_tiled_kernel"
    assert kernel_names((1, 32, 2048, 6, 6, 3, 3, 1, 1, 1, 1), nhwc)[0] == "binarize_nhwc_kernel"
    assert kernel_names((1, 32, 30, 6, 6, 3, 3, 1, 1, 1, 1), nhwc)[0] == "binarize_generic_kernel"
    # the switch that forces the XNOR/popcount kernel (used to profile the two side by side)
    monkeypatch.setenv("XNOR_NN_HIP_CONV", "valu")
    assert kernel_names((256,) + conv4)[1] == "conv_xnor_popc_kernel<XW=12,Q=16>"


def test_inputs_that_reach_the_dropped_offset_take_the_generic_kernel():
    """The tiled binarize kernels read a channel past the end of a ragged slice through the
    byte offset 0xFFFFFFF0, which the hardware drops only while it lies outside the buffer.
    An input that ends at or beyond that offset (but below 4 GiB) must not run them."""
    # 1 x 3 x 21 x 17043521 floats = 0xFFFFFFFC bytes: inside the gap
    assert kernel_names((1, 4, 3, 21, 17043521, 1, 1, 1, 1, 0, 0))[0] == "binarize_generic_kernel"
    nhwc = (capi.FMT_NHWC, capi.FMT_OIHW, capi.FMT_NCHW)
    # 1 x 4 x 1 x 268435455 floats = 0xFFFFFFF0 bytes, channels a multiple of four
    assert kernel_names((1, 4, 4, 1, 268435455, 1, 1, 1, 1, 0, 0), nhwc)[0] \
        == "binarize_generic_kernel"
    # just below: 0xFFFFFFEC bytes
    assert kernel_names((1, 4, 1, 1, 1073741819, 1, 1, 1, 1, 0, 0))[0] == "binarize_nchw_kernel"
    assert kernel_names((1, 4, 4, 1, 268435454, 1, 1, 1, 1, 0, 0), nhwc)[0] \
        == "binarize_nhwc_tiled_kernel"


def test_persistent_workgroups_are_planned_on_request_only(monkeypatch):
    """XNOR_NN_HIP_MFMA_PERSIST=N: N workgroups per XCD that walk over the tiles; without it a
    workgroup per tile, whatever the size (measured faster)."""
    resnet = (64, 256, 256, 56, 56, 3, 3, 1, 1, 1, 1)
    monkeypatch.delenv("XNOR_NN_HIP_MFMA_PERSIST", raising=False)
    assert kernel_names(resnet)[1] == "conv_mfma_fp4_kernel<KS=4,PS=2>"
    monkeypatch.setenv("XNOR_NN_HIP_MFMA_PERSIST", "64")
    assert kernel_names(resnet)[1] == "conv_mfma_fp4_persistent_kernel<KS=4,PS=4+3>"
    # sixteen steps per tap have no four-block tile: never persistent
    assert kernel_names((8, 256, 1024, 14, 14, 3, 3, 1, 1, 1, 1))[1].startswith(
        "conv_mfma_fp4_kernel<KS=16")
