"""CPU checkers used by the tests: the C oracle (oracle/libxnor_oracle.so) and, when it
has been built, the real upstream library (oracle/_ref/libxnor_nn_ref.so).

Both are test infrastructure.  Nothing here is imported by the package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from xnor_nn_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libxnor_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libxnor_nn_ref.so")


class Shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "mb", "ic", "ih", "iw", "oc", "oh", "ow", "kh", "kw", "sh", "sw", "ph", "pw",
        "src_fmt", "w_fmt", "dst_fmt")]


def _fptr(a):
    return a.ctypes.data_as(C.c_void_p)


class Oracle:
    """ctypes front end of oracle/xnor_oracle.c."""

    def __init__(self):
        if not os.path.exists(ORACLE_SO):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "all"])
        lib = C.CDLL(ORACLE_SO)
        P = C.POINTER(Shape)
        lib.xo_shape_init.argtypes = [P] + [C.c_int] * 14
        for name in ("xo_bici", "xo_bic", "xo_abic", "xo_ico"):
            getattr(lib, name).argtypes = [P]
            getattr(lib, name).restype = C.c_int
        lib.xo_oco.argtypes = [P, C.c_int]
        lib.xo_bin_src_bytes.argtypes = [P]
        lib.xo_bin_src_bytes.restype = C.c_size_t
        lib.xo_bin_weights_bytes.argtypes = [P, C.c_int]
        lib.xo_bin_weights_bytes.restype = C.c_size_t
        lib.xo_binarize_data.argtypes = [P, C.c_void_p, C.c_void_p]
        lib.xo_calculate_k.argtypes = [P, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.xo_binarize_weights.argtypes = [P, C.c_int] + [C.c_void_p] * 4
        lib.xo_convolution.argtypes = [P, C.c_int] + [C.c_void_p] * 7
        lib.xo_binarize_weights_float.argtypes = [P, C.c_void_p, C.c_void_p]
        self.lib = lib

    def shape(self, mb, oc, ic, ih, iw, kh, kw, sh, sw, ph, pw,
              src_fmt=capi.FMT_NCHW, w_fmt=capi.FMT_OIHW, dst_fmt=capi.FMT_NCHW):
        s = Shape()
        self.lib.xo_shape_init(C.byref(s), src_fmt, w_fmt, dst_fmt,
                               mb, oc, ic, ih, iw, kh, kw, sh, sw, ph, pw)
        return s

    def default_oci(self, s):
        """Filters per packed block on a 256-bit CPU (reference
        src/bcast_convolution.hpp:56-58 with vlen = 256)."""
        return 256 // 8 // self.lib.xo_bici(C.byref(s))

    def binarize_data(self, s, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(self.lib.xo_bin_src_bytes(C.byref(s)), dtype=np.uint8)
        self.lib.xo_binarize_data(C.byref(s), _fptr(x), _fptr(out))
        return out

    def calculate_k(self, s, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        a = np.empty((s.mb, s.ih, s.iw), dtype=np.float32)
        k = np.empty((s.mb, s.oh, s.ow), dtype=np.float32)
        self.lib.xo_calculate_k(C.byref(s), _fptr(x), _fptr(a), _fptr(k))
        return a, k

    def binarize_weights(self, s, w, oci=None):
        oci = oci or self.default_oci(s)
        w = np.ascontiguousarray(w, dtype=np.float32)
        out = np.empty(self.lib.xo_bin_weights_bytes(C.byref(s), oci), dtype=np.uint8)
        alpha = np.empty(s.oc, dtype=np.float32)
        opc = np.empty((s.oh, s.ow), dtype=np.int32)
        self.lib.xo_binarize_weights(C.byref(s), oci, _fptr(w), _fptr(out), _fptr(alpha),
                                     _fptr(opc))
        return out, alpha, opc

    def convolution(self, s, bsrc, bw, alpha, k, opc, oci=None):
        oci = oci or self.default_oci(s)
        popc = np.empty((s.mb, s.oc, s.oh, s.ow), dtype=np.int32)
        dshape = (s.mb, s.oc, s.oh, s.ow) if s.dst_fmt == capi.FMT_NCHW \
            else (s.mb, s.oh, s.ow, s.oc)
        dst = np.empty(dshape, dtype=np.float32)
        self.lib.xo_convolution(C.byref(s), oci, _fptr(bsrc), _fptr(bw), _fptr(alpha),
                                _fptr(k), _fptr(opc), _fptr(popc), _fptr(dst))
        return popc, dst

    def binarize_weights_float(self, s, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        out = np.empty(w.shape, dtype=np.float32)
        self.lib.xo_binarize_weights_float(C.byref(s), _fptr(w), _fptr(out))
        return out

    def forward(self, s, x, w, oci=None):
        """Whole pipeline; returns a dict with every intermediate."""
        bsrc = self.binarize_data(s, x)
        a, k = self.calculate_k(s, x)
        bw, alpha, opc = self.binarize_weights(s, w, oci)
        popc, dst = self.convolution(s, bsrc, bw, alpha, k, opc, oci)
        return dict(bin_src=bsrc, bin_weights=bw, a=a, k=k, alpha=alpha, opc=opc,
                    popc=popc, dst=dst)


def have_ref():
    return os.path.exists(REF_SO)


class RefLib:
    """The real upstream library, driven through its public C API.

    XNOR_NN_ISA=2 pins its 256-bit AVX kernels: on hosts with AVX-512 the library sizes its
    weight blocks for 512-bit vectors but only has 256-bit kernels (reference
    src/utils/cpuid.hpp:19-29 against src/bcast_convolution.cpp:93-105), which corrupts
    the output unless the override (reference src/utils/cpuid.hpp:96-112) is set before
    the first call."""

    def __init__(self):
        os.environ["XNOR_NN_ISA"] = "2"
        self.lib = capi.bind(C.CDLL(REF_SO), capi.CORE_SYMBOLS)

    def binarize_weights_float(self, dims, w, threads=1):
        """xnor_nn_binarize_weights_float on `threads` OpenMP threads.  Only one thread gives
        a defined result: the loop adds into a shared variable without a reduction
        (reference src/binarize_weights_float.cpp:17-19)."""
        lib = self.lib
        omp = C.CDLL("libgomp.so.1")
        c = capi.ConvolutionDesc()
        assert lib.xnor_nn_init_convolution(
            C.byref(c), capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW,
            dims["mb"], dims["oc"], dims["ic"], dims["ih"], dims["iw"],
            dims["kh"], dims["kw"], dims["sh"], dims["sw"], dims["ph"], dims["pw"]) == 0
        w = np.ascontiguousarray(w, dtype=np.float32)
        out = np.empty(w.shape, dtype=np.float32)
        before = omp.omp_get_max_threads()
        omp.omp_set_num_threads(threads)
        try:
            lib.xnor_nn_binarize_weights_float(C.byref(c), w.ctypes.data, out.ctypes.data)
        finally:
            omp.omp_set_num_threads(before)
        lib.xnor_nn_destroy_convolution(C.byref(c))
        return out

    def forward(self, dims, x, w, algorithm=capi.ALGORITHM_BCAST,
                fmts=(capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW), reps=1, timer=None):
        lib = self.lib
        c = capi.ConvolutionDesc()
        res = capi.Resources()
        st = lib.xnor_nn_init_convolution(
            C.byref(c), algorithm, fmts[0], fmts[1], fmts[2],
            dims["mb"], dims["oc"], dims["ic"], dims["ih"], dims["iw"],
            dims["kh"], dims["kw"], dims["sh"], dims["sw"], dims["ph"], dims["pw"])
        assert st == 0
        assert lib.xnor_nn_allocate_resources(C.byref(c), res) == 0
        x = np.ascontiguousarray(x, dtype=np.float32)
        w = np.ascontiguousarray(w, dtype=np.float32)
        dshape = (c.mb, c.oc, c.oh, c.ow) if fmts[2] == capi.FMT_NCHW \
            else (c.mb, c.oh, c.ow, c.oc)
        dst = np.zeros(dshape, dtype=np.float32)
        res[capi.RES_USER_SRC] = x.ctypes.data
        res[capi.RES_USER_WEIGHTS] = w.ctypes.data
        res[capi.RES_USER_DST] = dst.ctypes.data
        assert c.binarize_weights(C.byref(c), res) == 0
        times = []
        for _ in range(reps):
            t = [timer()] if timer else None
            assert c.binarize_data(C.byref(c), res) == 0
            if timer: t.append(timer())
            assert c.calculate_k(C.byref(c), res) == 0
            if timer: t.append(timer())
            assert c.forward(C.byref(c), res) == 0
            if timer: t.append(timer()); times.append(t)

        def grab(slot, dtype, count):
            return np.ctypeslib.as_array(
                C.cast(res[slot], C.POINTER(C.c_uint8)),
                shape=(count * np.dtype(dtype).itemsize,)).view(dtype).copy()

        out = dict(dst=dst, times=times)
        if algorithm == capi.ALGORITHM_BCAST:
            bici = 2 if c.ic * c.kh * c.kw < 32767 else 4
            bic = (c.ic + 7) // 8
            abic = (bic + bici - 1) // bici * bici
            ico = abic // bici
            oci = 256 // 8 // bici
            oco = (c.oc + oci - 1) // oci
            out["bin_src"] = grab(capi.RES_BIN_SRC, np.uint8, c.mb * c.ih * c.iw * abic)
            out["bin_weights"] = grab(capi.RES_BIN_WEIGHTS, np.uint8,
                                      oco * c.kh * c.kw * ico * oci * bici)
            opc_t = np.int16 if bici == 2 else np.int32
            out["opc"] = grab(capi.RES_OPERATIONS_COUNT, opc_t, c.oh * c.ow) \
                .astype(np.int32).reshape(c.oh, c.ow)
            out["bcast_applicable"] = (c.oc % oci == 0)
        out["a"] = grab(capi.RES_A, np.float32, c.mb * c.ih * c.iw).reshape(c.mb, c.ih, c.iw)
        out["k"] = grab(capi.RES_K, np.float32, c.mb * c.oh * c.ow).reshape(c.mb, c.oh, c.ow)
        out["alpha"] = grab(capi.RES_ALPHA, np.float32, c.oc)
        lib.xnor_nn_free_resources(res)
        lib.xnor_nn_destroy_convolution(C.byref(c))
        return out
