"""The caller one step above the path, for PyTorch-ROCm: the forward pass of the reference's
Caffe layer (reference external/caffe/src/caffe/layers/xnor_nn_conv_layer.cpp:25-67) on
device tensors.

Like that layer, the module builds its ``xnor_nn::Convolution`` on the first forward call
(the descriptor is fixed to one input shape; another shape builds another), re-binarizes the
weights only when told that they changed, and runs ``binarize_data -> calculate_k ->
forward`` per call.  Everything is computed by libxnor_nn.so on the current HIP stream;
torch only allocates the output.  Forward only: the reference's backward is a float GEMM
over ``binarized_weights()`` and lives in the framework, not in this library.
"""
import torch

from . import capi
from .convolution import Convolution


class XnorConv2d(torch.nn.Module):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 weight=None):
        super().__init__()
        pair = lambda v: (v, v) if isinstance(v, int) else tuple(v)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride, self.padding = pair(kernel_size), pair(stride), pair(padding)
        if weight is None:
            weight = torch.randn(out_channels, in_channels, *self.kernel_size) * 0.05
        assert tuple(weight.shape) == (out_channels, in_channels) + self.kernel_size
        self.weight = torch.nn.Parameter(weight.detach().to(torch.float32).contiguous(),
                                         requires_grad=False)
        self._conv = None
        self._shape = None
        self._weights_changed = False

    def weights_changed(self):
        """Call after writing to ``weight`` (the Caffe layer's changeWeights flag, reference
        external/caffe/src/caffe/layers/xnor_nn_conv_layer.cpp:55-58)."""
        self._weights_changed = True

    def _build(self, x):
        mb, ic, ih, iw = x.shape
        if self._conv is not None:
            self._conv.close()
        (kh, kw), (sh, sw), (ph, pw) = self.kernel_size, self.stride, self.padding
        self._conv = Convolution(capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW,
                                 capi.FMT_NCHW, mb, self.out_channels, ic, ih, iw,
                                 kh, kw, sh, sw, ph, pw, self.weight.data,
                                 stream=torch.cuda.current_stream(x.device))
        self._shape = tuple(x.shape)
        self._weights_changed = False

    def forward(self, x):
        if not (x.is_cuda and x.dtype == torch.float32 and x.dim() == 4
                and x.shape[1] == self.in_channels):
            raise ValueError("XnorConv2d takes a float32 NCHW tensor on the GPU with %d channels"
                             % self.in_channels)
        if self.weight.device != x.device:
            raise ValueError("weight and input live on different devices")
        x = x.contiguous()
        # every kernel of this call, the weight stage included, goes to torch's current stream:
        # that orders it behind the writes to `weight` and `x` already enqueued there
        if self._conv is None or self._shape != tuple(x.shape):
            self._build(x)
        else:
            self._conv.set_stream(torch.cuda.current_stream(x.device))
            if self._weights_changed:
                self._conv.change_weights(self.weight.data)
                self._weights_changed = False
        d = self._conv.desc
        y = torch.empty((d.mb, d.oc, d.oh, d.ow), dtype=torch.float32, device=x.device)
        self._conv.forward(x, y)
        return y

    def binarized_weights(self):
        """sign(w) * mean(w) as floats, what the reference's backward multiplies with
        (reference external/caffe/src/caffe/layers/xnor_nn_conv_layer.cpp:98,
        src/binarize_weights_float.cpp:3-25)."""
        if self._conv is None:
            raise RuntimeError("run a forward pass first (the descriptor is built there)")
        out = torch.empty_like(self.weight.data)
        self._conv.set_stream(torch.cuda.current_stream(out.device))
        self._conv.binarizeWeightsFloat(self.weight.data, out)
        return out
