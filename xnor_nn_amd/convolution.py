"""Python mirror of ``xnor_nn::Convolution`` (include/xnor_nn.hpp) over the C ABI.

Same construction arguments, same methods (``change_weights``, ``forward``,
``binarizeWeightsFloat``) and the same call order as the C++ wrapper of the reference
(reference include/xnor_nn.hpp:11-68); every call goes through libxnor_nn.so.  Tensors may
be numpy arrays (host memory, staged by the library) or torch tensors on the GPU (used in
place).  The extra methods expose the helpers of include/xnor_nn_hip.h.
"""
import ctypes as C

import numpy as np

from . import capi


class XnorNNError(RuntimeError):
    """Raised with the library's status text ("memory_error", "bad_input", ...)."""


class Convolution:
    def __init__(self, algorithm, src_fmt, weights_fmt, dst_fmt,
                 MB, OC, IC, IH, IW, KH, KW, SH, SW, PH, PW, weights, stream=None):
        self.lib = capi.load()
        self.desc = capi.ConvolutionDesc()
        self.res = capi.Resources()
        self._check(self.lib.xnor_nn_init_convolution(
            C.byref(self.desc), algorithm, src_fmt, weights_fmt, dst_fmt,
            MB, OC, IC, IH, IW, KH, KW, SH, SW, PH, PW))
        self._allocated = False
        self._check(self.lib.xnor_nn_allocate_resources(C.byref(self.desc), self.res))
        self._allocated = True
        if stream is not None:
            self.set_stream(stream)
        if weights is not None:
            self.change_weights(weights)

    # -- xnor_nn::Convolution ----------------------------------------------------------
    def change_weights(self, weights):
        self._weights = weights  # keep the tensor alive while the slot points at it
        self.res[capi.RES_USER_WEIGHTS] = capi.as_pointer(weights)
        self._check(self.desc.binarize_weights(C.byref(self.desc), self.res))

    def binarizeWeightsFloat(self, src, dst):
        self.lib.xnor_nn_binarize_weights_float(
            C.byref(self.desc), capi.as_pointer(src), capi.as_pointer(dst))

    def forward(self, src, dst):
        self.res[capi.RES_USER_SRC] = capi.as_pointer(src)
        self.res[capi.RES_USER_DST] = capi.as_pointer(dst)
        self._check(self.desc.binarize_data(C.byref(self.desc), self.res))
        self._check(self.desc.calculate_k(C.byref(self.desc), self.res))
        self._check(self.desc.forward(C.byref(self.desc), self.res))
        self.res[capi.RES_USER_SRC] = None
        self.res[capi.RES_USER_DST] = None

    # -- stage-level access (what C callers do through the descriptor) -----------------
    def stage(self, name, src=None, dst=None, check=True):
        """Run one executor ("binarize_data", "calculate_k", "forward",
        "binarize_weights") and return its status code."""
        if src is not None:
            self.res[capi.RES_USER_SRC] = capi.as_pointer(src)
        if dst is not None:
            self.res[capi.RES_USER_DST] = capi.as_pointer(dst)
        st = getattr(self.desc, name)(C.byref(self.desc), self.res)
        if check:
            self._check(st)
        return st

    # -- include/xnor_nn_hip.h ------------------------------------------------------------
    def set_stream(self, stream):
        handle = getattr(stream, "cuda_stream", stream)
        self._check(self.lib.xnor_nn_hip_set_stream(C.byref(self.desc), handle))

    def set_stage_fusion(self, on):
        self._check(self.lib.xnor_nn_hip_set_stage_fusion(C.byref(self.desc), int(bool(on))))

    def time_kernels(self, capacity):
        """Attach HIP events to the next launches of the binarize and convolution kernels
        (a ring of `capacity` launches per stage; 0 switches it off)."""
        self._check(self.lib.xnor_nn_hip_time_kernels(C.byref(self.desc), capacity))

    def kernel_times(self, stage, max_launches=65536):
        """Durations in milliseconds of the timed launches of one stage since the last call."""
        buf = (C.c_float * max_launches)()
        n = self.lib.xnor_nn_hip_kernel_times(C.byref(self.desc), stage, buf, max_launches)
        if n < 0:
            raise XnorNNError("kernel times are not available")
        return list(buf[:n])

    def synchronize(self):
        self._check(self.lib.xnor_nn_hip_synchronize(C.byref(self.desc)))

    def canonical_bici(self):
        return self.lib.xnor_nn_hip_canonical_bici(C.byref(self.desc))

    def export_bin_src(self):
        d = self.desc
        bici = self.canonical_bici()
        abic = ((d.ic + 7) // 8 + bici - 1) // bici * bici
        out = np.empty(d.mb * d.ih * d.iw * abic, dtype=np.uint8)
        self._check(self.lib.xnor_nn_hip_export_bin_src(
            C.byref(d), self.res, out.ctypes.data, out.nbytes))
        return out

    def export_bin_weights(self, oci=None):
        d = self.desc
        bici = self.canonical_bici()
        oci = oci or 256 // 8 // bici
        ico = ((d.ic + bici - 1) // bici + 7) // 8
        out = np.empty((d.oc // oci) * d.kh * d.kw * ico * oci * bici, dtype=np.uint8)
        self._check(self.lib.xnor_nn_hip_export_bin_weights(
            C.byref(d), self.res, oci, out.ctypes.data, out.nbytes))
        return out

    def export_floats(self, slot):
        d = self.desc
        shape = {capi.RES_ALPHA: (d.oc,), capi.RES_A: (d.mb, d.ih, d.iw),
                 capi.RES_K: (d.mb, d.oh, d.ow)}[slot]
        out = np.empty(shape, dtype=np.float32)
        self._check(self.lib.xnor_nn_hip_export_floats(
            C.byref(d), self.res, slot, out.ctypes.data, out.nbytes))
        return out

    def export_operations_count(self):
        d = self.desc
        out = np.empty((d.oh, d.ow), dtype=np.int32)
        self._check(self.lib.xnor_nn_hip_export_operations_count(
            C.byref(d), self.res, out.ctypes.data, out.nbytes))
        return out

    def forward_popcount(self, popc=None):
        d = self.desc
        if popc is None:
            popc = np.empty((d.mb, d.oc, d.oh, d.ow), dtype=np.int32)
        self._check(self.lib.xnor_nn_hip_forward_popcount(
            C.byref(d), self.res, capi.as_pointer(popc)))
        return popc

    def kernel_name(self, stage):
        buf = C.create_string_buffer(96)
        self.lib.xnor_nn_hip_kernel_name(C.byref(self.desc), stage, buf, len(buf))
        return buf.value.decode()

    # -- lifetime --------------------------------------------------------------------------
    def close(self):
        if getattr(self, "lib", None) is None:
            return
        if self._allocated:
            self.lib.xnor_nn_free_resources(self.res)
            self._allocated = False
        self.lib.xnor_nn_destroy_convolution(C.byref(self.desc))
        self.lib = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, status):
        if status != capi.SUCCESS:
            raise XnorNNError(capi.status_message(self.lib, status))
