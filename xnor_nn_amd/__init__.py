"""MI355X (gfx950) implementation of the XNOR-Net binary-convolution forward path behind
the xnor_nn C API.  The product is ``lib/libxnor_nn.so`` (HIP); this package holds its
sources (``csrc/``), its build script and a thin ctypes mirror of the C/C++ interface."""
from . import capi  # noqa: F401
from .convolution import Convolution, XnorNNError  # noqa: F401
