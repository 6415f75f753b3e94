"""ctypes view of the xnor_nn C ABI (include/xnor_nn_types.h, include/xnor_nn.h).

The structure below mirrors ``struct xnor_nn_convolution_`` field for field, so the same
definitions bind both this repository's HIP library and any other library that exports the
xnor_nn ABI (the tests use that to drive a CPU build of the upstream library as a checker).
"""
import ctypes as C
import os

# xnor_nn_status_t
SUCCESS, ERROR_MEMORY, ERROR_INVALID_INPUT, UNIMPLEMENTED = range(4)
# xnor_nn_algorithm_t
ALGORITHM_REFERENCE, ALGORITHM_BCAST = 0, 1
ALGORITHM_BEST = 1
# xnor_nn_resource_type_t
(RES_USER_SRC, RES_USER_WEIGHTS, RES_USER_DST, RES_ALPHA, RES_BIN_SRC, RES_BIN_WEIGHTS,
 RES_A, RES_K, RES_OPERATIONS_COUNT, RES_NUMBER) = range(10)
RES_INTERNAL = 3
# xnor_nn_tensor_format_t
FMT_NCHW, FMT_NHWC, FMT_OIHW, FMT_HWIO = range(4)

# xnor_nn_operation_t
(OP_CONVOLUTION_FORWARD, OP_BINARIZE_WEIGHTS, OP_BINARIZE_DATA, OP_CALCULATE_K) = range(4)

Resources = C.c_void_p * RES_NUMBER


class ConvolutionDesc(C.Structure):
    pass


Executor = C.CFUNCTYPE(C.c_int, C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p))

ConvolutionDesc._fields_ = [
    ("algorithm", C.c_int),
    ("mb", C.c_int),
    ("ic", C.c_int), ("ih", C.c_int), ("iw", C.c_int),
    ("oc", C.c_int), ("oh", C.c_int), ("ow", C.c_int),
    ("sh", C.c_int), ("sw", C.c_int),
    ("kh", C.c_int), ("kw", C.c_int),
    ("ph", C.c_int), ("pw", C.c_int),
    ("src_format", C.c_int),
    ("weights_format", C.c_int),
    ("dst_format", C.c_int),
    ("resource_size", C.c_size_t * RES_NUMBER),
    ("binarize_weights", Executor),
    ("binarize_data", Executor),
    ("calculate_k", Executor),
    ("forward", Executor),
    ("state", C.c_void_p),
]

# Symbols of include/xnor_nn.h: name -> (restype, argtypes)
CORE_SYMBOLS = {
    "xnor_nn_get_status_message": (None, [C.c_char_p, C.c_int]),
    "xnor_nn_allocate_resources": (C.c_int, [C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p)]),
    "xnor_nn_free_resources": (None, [C.POINTER(C.c_void_p)]),
    "xnor_nn_binarize_weights_float": (None, [C.POINTER(ConvolutionDesc), C.c_void_p, C.c_void_p]),
    "xnor_nn_init_convolution": (C.c_int, [C.POINTER(ConvolutionDesc)] + [C.c_int] * 15),
    "xnor_nn_destroy_convolution": (None, [C.POINTER(ConvolutionDesc)]),
}

# Symbols of include/xnor_nn_hip.h
HIP_SYMBOLS = {
    "xnor_nn_hip_set_stream": (C.c_int, [C.POINTER(ConvolutionDesc), C.c_void_p]),
    "xnor_nn_hip_set_stage_fusion": (C.c_int, [C.POINTER(ConvolutionDesc), C.c_int]),
    "xnor_nn_hip_plain_read": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "xnor_nn_hip_mfma_only": (C.c_int, [C.c_int, C.c_int, C.c_void_p]),
    "xnor_nn_hip_synchronize": (C.c_int, [C.POINTER(ConvolutionDesc)]),
    "xnor_nn_hip_export_bin_src": (C.c_int, [C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p), C.c_void_p, C.c_size_t]),
    "xnor_nn_hip_export_bin_weights": (C.c_int, [C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_size_t]),
    "xnor_nn_hip_export_floats": (C.c_int, [C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_size_t]),
    "xnor_nn_hip_export_operations_count": (C.c_int, [C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p), C.c_void_p, C.c_size_t]),
    "xnor_nn_hip_forward_popcount": (C.c_int, [C.POINTER(ConvolutionDesc), C.POINTER(C.c_void_p), C.c_void_p]),
    "xnor_nn_hip_canonical_bici": (C.c_int, [C.POINTER(ConvolutionDesc)]),
    "xnor_nn_hip_device_info": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "xnor_nn_hip_binarize_weights_float_noalloc": (C.c_int, [C.POINTER(ConvolutionDesc), C.c_void_p, C.c_void_p]),
    "xnor_nn_hip_time_kernels": (C.c_int, [C.POINTER(ConvolutionDesc), C.c_int]),
    "xnor_nn_hip_kernel_times": (C.c_int, [C.POINTER(ConvolutionDesc), C.c_int, C.POINTER(C.c_float), C.c_int]),
    "xnor_nn_hip_kernel_name": (C.c_int, [C.POINTER(ConvolutionDesc), C.c_int, C.c_char_p, C.c_size_t]),
}


def bind(lib, symbols):
    """Attach restype/argtypes; raises AttributeError naming the first missing symbol."""
    for name, (restype, argtypes) in symbols.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def library_path():
    """In-tree location of the HIP library built by ``xnor_nn_amd.build``."""
    here = os.path.dirname(os.path.abspath(__file__))
    # XNOR_NN_AMD_LIBRARY names another build of the same library (measurements of variants)
    return os.environ.get("XNOR_NN_AMD_LIBRARY") or os.path.join(here, "lib", "libxnor_nn.so")


_LIB = None


def load():
    """Load the in-tree HIP library.  There is no CPU fallback: a missing or unloadable
    library is an error."""
    global _LIB
    if _LIB is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(
                "%s is missing: build it with `python -m xnor_nn_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no CPU fallback" % path)
        # A process must hold ONE HIP runtime.  PyTorch ships its own copy (same soname as
        # the system one): when torch is imported first, the dynamic loader resolves this
        # library's dependency to that copy; the other order would load a second runtime
        # and leave torch without a device.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = C.CDLL(path)
        bind(lib, CORE_SYMBOLS)
        bind(lib, HIP_SYMBOLS)
        _LIB = lib
    return _LIB


def status_message(lib, status):
    buf = C.create_string_buffer(16)
    lib.xnor_nn_get_status_message(buf, status)
    return buf.value.decode()


def as_pointer(obj):
    """Address of a torch tensor (``data_ptr``), a numpy array, a ctypes buffer or an int."""
    if obj is None:
        return None
    if isinstance(obj, int):
        return obj
    if hasattr(obj, "data_ptr"):
        return obj.data_ptr()
    if hasattr(obj, "ctypes"):
        return obj.ctypes.data
    return C.addressof(obj)
