"""The C-ABI boundary on the GPU: resource tables, call orders the reference allows because
its stages are independent, host threads sharing a descriptor, failure paths and the verbose
lines.  Everything goes through libxnor_nn.so; results are compared with the CPU oracle bit
for bit."""
import ctypes as C
import os
import subprocess
import sys
import threading

import numpy as np
import pytest

import shapes
from util import oracle_shape
from xnor_nn_amd import Convolution, capi, synth

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NCHW = (capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW)


def make(d, w, fmts=NCHW):
    return Convolution(capi.ALGORITHM_BCAST, fmts[0], fmts[1], fmts[2],
                       d["mb"], d["oc"], d["ic"], d["ih"], d["iw"], d["kh"], d["kw"],
                       d["sh"], d["sw"], d["ph"], d["pw"], w)


def same_bits(got, want):
    return np.array_equal(np.asarray(got).view(np.uint32), np.asarray(want).view(np.uint32))


def second_table(conv, wt):
    """Another resource table for conv's descriptor, with its own buffers and its own
    binarized weights."""
    res = capi.Resources()
    assert conv.lib.xnor_nn_allocate_resources(C.byref(conv.desc), res) == capi.SUCCESS
    res[capi.RES_USER_WEIGHTS] = capi.as_pointer(wt)
    assert conv.desc.binarize_weights(C.byref(conv.desc), res) == capi.SUCCESS
    return res


def run(conv, res, stage, src=None, dst=None):
    if src is not None:
        res[capi.RES_USER_SRC] = capi.as_pointer(src)
    if dst is not None:
        res[capi.RES_USER_DST] = capi.as_pointer(dst)
    assert getattr(conv.desc, stage)(C.byref(conv.desc), res) == capi.SUCCESS, stage


@pytest.mark.parametrize("conv_kind", ["mfma", "valu"])
def test_calculate_k_before_binarize_data_on_a_reused_buffer(oracle, gpu, monkeypatch, conv_kind):
    """calculate_k -> binarize_data -> forward per iteration, the input buffer rewritten in
    place between iterations: the mean|x| that binarize_data leaves behind must not be taken
    for the next iteration's (reference stages are independent:
    src/bcast_calculate_k.cpp:42-85 reads user_src on every call)."""
    import torch
    if conv_kind == "valu":
        monkeypatch.setenv("XNOR_NN_HIP_CONV", "valu")
    d, x1, w = synth.make_workload("alexnet_conv4_mb256", 5)
    x2 = (x1[::-1] * np.float32(0.75)).copy()
    s = oracle_shape(oracle, d)
    wants = [oracle.forward(s, x, w) for x in (x1, x2)]
    buf = torch.empty(x1.shape, dtype=torch.float32, device=gpu)
    dt = torch.empty(wants[0]["dst"].shape, dtype=torch.float32, device=gpu)
    conv = make(d, torch.from_numpy(w).to(gpu))
    for x, want in zip((x1, x2, x1), (wants[0], wants[1], wants[0])):
        buf.copy_(torch.from_numpy(x))
        torch.cuda.synchronize()
        conv.stage("calculate_k", src=buf, dst=dt)
        conv.stage("binarize_data")
        conv.stage("forward")
        conv.synchronize()
        assert same_bits(dt.cpu().numpy(), want["dst"])
        assert same_bits(conv.export_floats(capi.RES_K), want["k"])
        assert same_bits(conv.export_floats(capi.RES_A), want["a"])
    # and the usual order on the same reused buffer
    for x, want in zip((x2, x1), (wants[1], wants[0])):
        buf.copy_(torch.from_numpy(x))
        torch.cuda.synchronize()
        conv.forward(buf, dt)
        conv.synchronize()
        assert same_bits(dt.cpu().numpy(), want["dst"])
    conv.close()


def test_two_resource_tables_on_one_descriptor(oracle, gpu):
    """One descriptor, two resource tables used in turn and interleaved stage by stage: what
    one table's stages hand to each other must not leak into the other table (reference
    executors read and write only through res[], src/bcast_convolution.hpp:77-93)."""
    import torch
    d, x1, w = synth.make_workload("alexnet_conv4_mb256", 4)
    x2 = (x1[::-1] * np.float32(1.25)).copy()
    s = oracle_shape(oracle, d)
    want1, want2 = oracle.forward(s, x1, w), oracle.forward(s, x2, w)
    wt = torch.from_numpy(w).to(gpu)
    x1t, x2t = torch.from_numpy(x1).to(gpu), torch.from_numpy(x2).to(gpu)
    y1 = torch.empty(want1["dst"].shape, dtype=torch.float32, device=gpu)
    y2 = torch.empty_like(y1)
    conv = make(d, wt)
    res2 = second_table(conv, wt)
    r1 = conv.res
    # interleaved: every stage of table 1 is followed by the same stage of table 2
    run(conv, r1, "binarize_data", x1t, y1)
    run(conv, res2, "binarize_data", x2t, y2)
    run(conv, r1, "calculate_k")
    run(conv, res2, "calculate_k")
    run(conv, r1, "forward")
    run(conv, res2, "forward")
    conv.synchronize()
    assert same_bits(y1.cpu().numpy(), want1["dst"])
    assert same_bits(y2.cpu().numpy(), want2["dst"])
    # table 2 computes K, then table 1 runs a whole pass, then table 2 convolves
    y1.zero_(); y2.zero_()
    run(conv, res2, "binarize_data", x1t, y2)
    run(conv, res2, "calculate_k")
    run(conv, r1, "binarize_data", x2t, y1)
    run(conv, r1, "calculate_k")
    run(conv, r1, "forward")
    run(conv, res2, "forward")
    conv.synchronize()
    assert same_bits(y1.cpu().numpy(), want2["dst"])
    assert same_bits(y2.cpu().numpy(), want1["dst"])
    # a forward on table 1 with table 2's K plane (hand-made table): K of x1, bits of x2
    mixed = capi.Resources()
    for i in range(capi.RES_NUMBER):
        mixed[i] = r1[i]
    mixed[capi.RES_K] = res2[capi.RES_K]
    run(conv, res2, "binarize_data", x1t)
    run(conv, res2, "calculate_k")       # K(x1) owed to table 2's K plane
    run(conv, mixed, "forward", dst=y1)  # bits(x2) from table 1, K(x1) from table 2
    conv.synchronize()
    k1 = want1["k"][:, None, :, :]
    k2 = want2["k"][:, None, :, :]
    base = want2  # dst = fl(fl(n * alpha) * k): the K factor of want2 swapped for want1's
    n_alpha = (2 * base["popc"].astype(np.int64) - base["opc"][None, None]).astype(np.float32) \
        * base["alpha"][None, :, None, None]
    assert same_bits(y1.cpu().numpy(), (n_alpha * k1).astype(np.float32))
    assert not same_bits(y1.cpu().numpy(), (n_alpha * k2).astype(np.float32))
    conv.lib.xnor_nn_free_resources(res2)
    conv.close()


def test_two_descriptors_on_two_streams_share_a_mean_plane(oracle, gpu):
    """Descriptor A (stream sa) leaves its box filter owed to its K plane; descriptor B
    (stream sb, a table that names A's mean|x| plane as its own) then binarizes other data
    and so overwrites that plane.  The filter owed by A has to run first, where A's mean|x|
    was written (on sa, behind A's binarize kernel), and B's kernel has to wait for it: the
    two streams are ordered with events.  A large batch keeps A's binarize kernel busy when
    B is called.  Then the other way round: B's K owed, read back through A."""
    import torch
    d, x1, w = synth.make_workload("alexnet_conv4_mb256", 96)
    x2 = (x1[::-1] * np.float32(0.75)).copy()
    s = oracle_shape(oracle, d)
    want1, want2 = oracle.forward(s, x1, w), oracle.forward(s, x2, w)
    wt = torch.from_numpy(w).to(gpu)
    x1t, x2t = torch.from_numpy(x1).to(gpu), torch.from_numpy(x2).to(gpu)
    ya = torch.empty(want1["dst"].shape, dtype=torch.float32, device=gpu)
    yb = torch.empty_like(ya)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    A, B = make(d, wt), make(d, wt)
    A.set_stream(sa)
    B.set_stream(sb)
    own_a = B.res[capi.RES_A]
    B.res[capi.RES_A] = A.res[capi.RES_A]  # one mean|x| plane for both tables
    torch.cuda.synchronize()
    for rep in range(3):
        run(A, A.res, "binarize_data", x1t, ya)
        run(A, A.res, "calculate_k")          # K(x1) owed to A's K plane, mean|x| written on sa
        run(B, B.res, "binarize_data", x2t, yb)  # overwrites the plane: A's filter runs first
        run(B, B.res, "calculate_k")
        run(B, B.res, "forward")
        run(A, A.res, "forward")              # bits(x1), K(x1) from the finished K plane
        torch.cuda.synchronize()
        assert same_bits(A.export_floats(capi.RES_K), want1["k"]), rep
        assert same_bits(ya.cpu().numpy(), want1["dst"]), rep
        assert same_bits(yb.cpu().numpy(), want2["dst"]), rep
        # B's K owed (on sb); A asks for a forward with B's K plane in its table
        run(B, B.res, "binarize_data", x2t, yb)
        run(B, B.res, "calculate_k")
        mixed = capi.Resources()
        for i in range(capi.RES_NUMBER):
            mixed[i] = A.res[i]
        mixed[capi.RES_K] = B.res[capi.RES_K]
        run(A, mixed, "forward", dst=ya)      # bits(x1) of A's table, K(x2) owed by B
        torch.cuda.synchronize()
        n_alpha = (2 * want1["popc"].astype(np.int64) - want1["opc"][None, None]).astype(
            np.float32) * want1["alpha"][None, :, None, None]
        assert same_bits(ya.cpu().numpy(), (n_alpha * want2["k"][:, None]).astype(np.float32)), rep
    B.res[capi.RES_A] = own_a
    A.close()
    B.close()


def test_free_and_allocate_between_calculate_k_and_forward(oracle, gpu):
    """calculate_k leaves its box filter to forward; when the table is freed in between,
    nothing may run later on the freed buffers, and a fresh table on the same descriptor
    gives the right result."""
    import torch
    d, x, w = synth.make_workload("alexnet_conv4_mb256", 3)
    s = oracle_shape(oracle, d)
    want = oracle.forward(s, x, w)
    xt, wt = torch.from_numpy(x).to(gpu), torch.from_numpy(w).to(gpu)
    yt = torch.empty(want["dst"].shape, dtype=torch.float32, device=gpu)
    conv = make(d, wt)
    conv.stage("binarize_data", src=xt, dst=yt)
    conv.stage("calculate_k")
    conv.synchronize()
    conv.lib.xnor_nn_free_resources(conv.res)
    assert all(conv.res[i] is None for i in range(capi.RES_INTERNAL, capi.RES_NUMBER))
    assert conv.lib.xnor_nn_allocate_resources(C.byref(conv.desc), conv.res) == capi.SUCCESS
    conv.change_weights(wt)
    # stale hand-overs would show here: calculate_k without a binarize_data before it, then a
    # K export, on buffers that may sit where the freed ones were
    conv.stage("calculate_k", src=xt)
    assert same_bits(conv.export_floats(capi.RES_K), want["k"])
    conv.forward(xt, yt)
    conv.synchronize()
    assert same_bits(yt.cpu().numpy(), want["dst"])
    conv.close()


def test_two_host_threads_share_one_descriptor(oracle, gpu):
    """Two host threads drive one descriptor, each with its own resource table and its own
    input, thirty forward passes each, device pointers on one and host pointers on the other
    (reference: executors are re-entrant on distinct res, src/bcast_convolution.hpp:77-93)."""
    import torch
    d, x1, w = synth.make_workload("alexnet_conv4_mb256", 4)
    x2 = (x1[::-1] * np.float32(2.0)).copy()
    s = oracle_shape(oracle, d)
    want = [oracle.forward(s, x1, w)["dst"], oracle.forward(s, x2, w)["dst"]]
    wt = torch.from_numpy(w).to(gpu)
    conv = make(d, wt)
    tables = [conv.res, second_table(conv, wt)]
    x1t = torch.from_numpy(x1).to(gpu)
    y1t = torch.empty(want[0].shape, dtype=torch.float32, device=gpu)
    y2 = np.empty(want[1].shape, np.float32)
    torch.cuda.synchronize()
    errors = []

    def worker(i):
        try:
            res = tables[i]
            for it in range(30):
                if i == 0:
                    y1t.zero_()
                    torch.cuda.synchronize()
                    run(conv, res, "binarize_data", x1t, y1t)
                    run(conv, res, "calculate_k")
                    run(conv, res, "forward")
                    conv.synchronize()
                    got = y1t.cpu().numpy()
                else:
                    y2.fill(0)
                    run(conv, res, "binarize_data", x2, y2)
                    run(conv, res, "calculate_k")
                    run(conv, res, "forward")
                    got = y2
                if not same_bits(got, want[i]):
                    errors.append("thread %d, pass %d: wrong dst" % (i, it))
                    return
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (i, e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    conv.lib.xnor_nn_free_resources(tables[1])
    conv.close()


def test_stage_fusion_switched_off_by_the_api(oracle, gpu):
    """xnor_nn_hip_set_stage_fusion(c, 0): calculate_k reads the input itself and finishes
    the K plane, so the input may change between binarize_data and calculate_k."""
    import torch
    d, x1, w = synth.make_workload("alexnet_conv4_mb256", 3)
    x2 = (x1[::-1] * np.float32(0.5)).copy()
    s = oracle_shape(oracle, d)
    want1, want2 = oracle.forward(s, x1, w), oracle.forward(s, x2, w)
    buf = torch.from_numpy(x1).to(gpu)
    yt = torch.empty(want1["dst"].shape, dtype=torch.float32, device=gpu)
    conv = make(d, torch.from_numpy(w).to(gpu))
    conv.set_stage_fusion(False)
    # the K plane is a buffer of the caller's here, so that it can be read directly
    kt = torch.zeros(want1["k"].shape, dtype=torch.float32, device=gpu)
    own_k = conv.res[capi.RES_K]
    conv.res[capi.RES_K] = kt.data_ptr()
    conv.stage("binarize_data", src=buf, dst=yt)
    buf.copy_(torch.from_numpy(x2))
    torch.cuda.synchronize()
    conv.stage("calculate_k")
    conv.synchronize()
    assert same_bits(kt.cpu().numpy(), want2["k"])  # complete in res[k] without any helper
    conv.stage("forward")
    conv.synchronize()
    # bits of x1 with K of x2
    n_alpha = (2 * want1["popc"].astype(np.int64) - want1["opc"][None, None]).astype(np.float32) \
        * want1["alpha"][None, :, None, None]
    assert same_bits(yt.cpu().numpy(), (n_alpha * want2["k"][:, None]).astype(np.float32))
    conv.res[capi.RES_K] = own_k
    conv.close()


def test_popcount_accumulators_without_an_operations_count(oracle, gpu):
    """xnor_nn_hip_forward_popcount with only bin_src and bin_weights in the table, as its
    header promises (the matrix-core kernel derives the operation count itself)."""
    import torch
    for t in ((3, 384, 256, 13, 13, 3, 3, 1, 1, 1, 1), (2, 96, 70, 11, 9, 5, 5, 2, 2, 2, 2),
              (1, 40, 33, 9, 9, 7, 7, 1, 1, 3, 3)):
        d = shapes.as_dims(t)
        x = synth.normal(11, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
            d["mb"], d["ic"], d["ih"], d["iw"])
        w = synth.normal(12, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
            d["oc"], d["ic"], d["kh"], d["kw"])
        want = oracle.forward(oracle_shape(oracle, d), x, w)
        conv = make(d, w)
        dst = np.empty(want["dst"].shape, np.float32)
        conv.forward(x, dst)
        bare = capi.Resources()
        bare[capi.RES_BIN_SRC] = conv.res[capi.RES_BIN_SRC]
        bare[capi.RES_BIN_WEIGHTS] = conv.res[capi.RES_BIN_WEIGHTS]
        popc = np.empty(want["popc"].shape, np.int32)
        assert conv.lib.xnor_nn_hip_forward_popcount(
            C.byref(conv.desc), bare, popc.ctypes.data) == capi.SUCCESS
        assert np.array_equal(popc, want["popc"])
        conv.close()


def test_more_channels_than_the_tiled_binarize_kernel_stages(oracle, gpu):
    """NCHW input with 8200 channels: the packed words of a 64-pixel tile no longer fit 64 KB
    of LDS, so the generic kernel takes it (the reference takes any channel count,
    src/convolution_traits.hpp:29-56)."""
    d = shapes.as_dims((1, 8200, 16, 5, 4, 3, 3, 1, 1, 1, 1))
    x = synth.normal(21, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
        d["mb"], d["ic"], d["ih"], d["iw"])
    x.ravel()[::5] = 0.0
    x.ravel()[2::9] = -0.0
    w = synth.normal(22, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
        d["oc"], d["ic"], d["kh"], d["kw"])
    want = oracle.forward(oracle_shape(oracle, d), x, w)
    conv = make(d, w)
    assert conv.kernel_name(2) == "binarize_generic_kernel"
    dst = np.empty(want["dst"].shape, np.float32)
    conv.forward(x, dst)
    assert np.array_equal(conv.export_bin_src(), want["bin_src"])
    assert same_bits(conv.export_floats(capi.RES_A), want["a"])
    assert same_bits(conv.export_floats(capi.RES_K), want["k"])
    assert np.array_equal(conv.forward_popcount(), want["popc"])
    assert same_bits(dst, want["dst"])
    conv.close()


def test_allocation_failure_rolls_back(gpu):
    """A descriptor whose packed input alone is larger than the GPU's memory:
    xnor_nn_allocate_resources reports memory_error and leaves every slot null, the slots it
    had already filled included (reference src/memory.cpp:23-33); the next, ordinary
    allocation works."""
    lib = capi.load()
    c = capi.ConvolutionDesc()
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW,
                                 capi.FMT_NCHW, 4096, 64, 4096, 512, 512, 3, 3, 1, 1, 1, 1)
    assert c.resource_size[capi.RES_BIN_SRC] == 4096 * 512 * 512 * 128 * 4  # 512 GiB
    res = capi.Resources()
    assert lib.xnor_nn_allocate_resources(C.byref(c), res) == capi.ERROR_MEMORY
    assert all(res[i] is None for i in range(capi.RES_NUMBER))
    lib.xnor_nn_destroy_convolution(C.byref(c))
    lib.xnor_nn_init_convolution(C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW,
                                 capi.FMT_NCHW, 2, 64, 64, 8, 8, 3, 3, 1, 1, 1, 1)
    assert lib.xnor_nn_allocate_resources(C.byref(c), res) == capi.SUCCESS
    assert all(res[i] is not None for i in range(capi.RES_INTERNAL, capi.RES_NUMBER))
    lib.xnor_nn_free_resources(res)
    lib.xnor_nn_destroy_convolution(C.byref(c))


VERBOSE_CHILD = r"""
import sys
sys.path.insert(0, %(root)r)
import numpy as np
from xnor_nn_amd import Convolution, capi, synth
d, x, w = synth.make_workload("alexnet_conv4_mb256", 2)
conv = Convolution(capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW,
                   d["mb"], d["oc"], d["ic"], d["ih"], d["iw"], d["kh"], d["kw"],
                   d["sh"], d["sw"], d["ph"], d["pw"], w)
dst = np.empty((d["mb"], d["oc"], d["ih"], d["iw"]), np.float32)
conv.forward(x, dst)
sys.stdout.flush()
print("NAMES %%s|%%s" %% (conv.kernel_name(0), conv.kernel_name(2)))
conv.close()
"""


@pytest.mark.parametrize("conv_kind", ["mfma", "valu"])
def test_verbose_lines_name_the_kernels(gpu, conv_kind):
    """XNOR_NN_VERBOSE=1 prints one line for init and one per executor call, naming the kernel
    variant that runs, the counterpart of the reference's logger (reference
    src/utils/convolution_logger.hpp:99-152).  Run in a child process so that the lines,
    printed by the C library, can be read back."""
    env = dict(os.environ, XNOR_NN_VERBOSE="1")
    if conv_kind == "valu":
        env["XNOR_NN_HIP_CONV"] = "valu"
    out = subprocess.run([sys.executable, "-c", VERBOSE_CHILD % {"root": ROOT}], env=env,
                         capture_output=True, text=True, timeout=170)
    assert out.returncode == 0, (out.stdout[-2000:], out.stderr[-2000:])
    lines = [l for l in out.stdout.splitlines() if l.startswith("xnor_nn ")]
    names = [l for l in out.stdout.splitlines() if l.startswith("NAMES ")][0][6:].split("|")
    conv_name, bin_name = names
    assert conv_name.startswith("conv_mfma_fp4" if conv_kind == "mfma" else "conv_xnor_popc")
    init = [l for l in lines if l.startswith("xnor_nn init:")]
    assert len(init) == 1 and "mb=2 ic=384 13x13 oc=256" in init[0] and conv_name in init[0]
    execs = [l for l in lines if l.startswith("xnor_nn exec")]
    assert execs[0].startswith("xnor_nn exec binarize_weights:")
    assert execs[1] == "xnor_nn exec binarize_data: " + bin_name
    assert execs[2].startswith("xnor_nn exec calculate_k:")
    if conv_kind == "mfma":
        assert "deferred to the convolution" in execs[2]
        assert execs[3] == "xnor_nn exec forward: %s (with the box filter of calculate_k)" \
            % conv_name
    else:
        assert "box_filter_kernel" in execs[2]
        assert execs[3] == "xnor_nn exec forward: " + conv_name
    assert len(execs) == 4


def test_plain_read_calibration_kernel(gpu):
    """xnor_nn_hip_plain_read: runs on device memory of any size from one 16-byte piece up
    (ragged ends included) and refuses what it cannot read."""
    import torch
    lib = capi.load()
    for n in (4, 1000, 1 << 20, (1 << 22) + 5):
        t = torch.ones(n, dtype=torch.float32, device=gpu)
        assert lib.xnor_nn_hip_plain_read(t.data_ptr(), n * 4, None) == capi.SUCCESS
    torch.cuda.synchronize()
    host = np.ones(64, np.float32)
    assert lib.xnor_nn_hip_plain_read(host.ctypes.data, host.nbytes, None) == capi.ERROR_INVALID_INPUT
    assert lib.xnor_nn_hip_plain_read(None, 64, None) == capi.ERROR_INVALID_INPUT
    assert lib.xnor_nn_hip_plain_read(t.data_ptr(), 8, None) == capi.ERROR_INVALID_INPUT
    assert lib.xnor_nn_hip_plain_read(t.data_ptr() + 4, 64, None) == capi.ERROR_INVALID_INPUT


def test_matrix_instruction_calibration_kernel(gpu):
    """xnor_nn_hip_mfma_only runs (it touches no memory) and checks its two counts."""
    import torch
    lib = capi.load()
    assert lib.xnor_nn_hip_mfma_only(8, 3, None) == capi.SUCCESS
    assert lib.xnor_nn_hip_mfma_only(512, 50, None) == capi.SUCCESS
    torch.cuda.synchronize()
    assert lib.xnor_nn_hip_mfma_only(0, 3, None) == capi.ERROR_INVALID_INPUT
    assert lib.xnor_nn_hip_mfma_only(8, 0, None) == capi.ERROR_INVALID_INPUT
