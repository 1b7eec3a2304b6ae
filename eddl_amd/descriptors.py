"""Host-side mirrors of the reference's ConvolDescriptor and PoolDescriptor: the same field
names and the same geometry rules (src/descriptors/descriptor_conv2D.cpp:24-59,88-160,295-360;
src/descriptors/descriptor_pool2D.cpp:15-42,50-117,162-211), without any tensor storage.
Errors follow the reference's msg() convention (src/utils.cpp:57-67): a RuntimeError whose
text is "RuntimeError: <where>" after the explanation.
"""
import numpy as np

_f32 = np.float32


def msg(text, title):
    raise RuntimeError("%s (RuntimeError: %s)" % (text, title))


def _out_named(padding, input_size, kernel_size, stride, dilation_rate, where):
    if padding in ("same", "zeros"):
        return int(np.ceil(_f32(input_size) / _f32(stride)))
    if padding in ("valid", "none"):
        return int(np.ceil((_f32(input_size) - (_f32(kernel_size) - _f32(1)) * _f32(dilation_rate)) / _f32(stride)))
    msg("Incorrect padding type", where)


def _out_custom(pad2, input_size, kernel_size, stride, dilation_rate=1):
    v = (_f32(input_size) - (_f32(kernel_size) - _f32(1)) * _f32(dilation_rate) + _f32(pad2[0]) + _f32(pad2[1]) - _f32(1)) \
        / _f32(stride) + _f32(1)
    return int(v)  # truncation, as the reference's (int) cast


def _pads_named(output_size, input_size, kernel_size, stride, padding, dilation_rate, where):
    if padding in ("same", "zeros"):
        pad = (output_size - 1) * stride + kernel_size - input_size + (dilation_rate - 1) * (kernel_size - 1)
        pad = max(pad, 0)
        return [pad // 2, pad - pad // 2]
    if padding in ("valid", "none"):
        return [0, 0]
    msg("Incorrect padding type", where)


class ConvolDescriptor:
    """Geometry of one Conv2D layer.  ``pads`` (custom padding) = [top, bottom, left, right]."""

    def __init__(self, filters, kernel_size, strides, padding, pads=(), groups=1, dilation_rate=(1, 1), use_bias=True, mem=0):
        where = "ConvolDescriptor::ConvolDescriptor"
        if groups > 1:
            msg("Grouped convolutions are only available with CuDNN", where)
        if len(kernel_size) != 2:
            msg("Kernels must have 3 dimensions", where)
        if len(strides) != 2:
            msg("Strides must have 2 dimensions", where)
        if len(dilation_rate) != 2:
            msg("Dilations must have 2 elements", where)
        if groups < 1:
            msg("The number of groups should be greater or equal to 1", where)
        if padding not in ("custom", "same", "none", "valid", "zeros", "same,none", "none,same"):
            msg("Incorrect padding type (" + padding + ")", where)
        self.filters = filters
        self.kernel_size = list(kernel_size)
        self.strides = list(strides)
        self.padding = padding
        self.pads = list(pads)
        self.groups = groups
        self.dilation_rate = list(dilation_rate)
        self.use_bias = use_bias
        self.mem_level = mem
        self.ksize = [filters] + list(kernel_size)
        self.stride = list(strides)

    @staticmethod
    def compute_output(padding, input_size, kernel_size, stride, dilation_rate=1):
        if isinstance(padding, str):
            return _out_named(padding, input_size, kernel_size, stride, dilation_rate, "ConvolDescriptor::compute_output")
        return _out_custom(padding, input_size, kernel_size, stride, dilation_rate)

    @staticmethod
    def compute_padding(output_size, input_size, kernel_size, stride, padding="same", row=False, dilation_rate=1):
        if padding == "same,none":
            padding = "same" if row else "none"
        if padding == "none,same":
            padding = "none" if row else "same"
        return _pads_named(output_size, input_size, kernel_size, stride, padding, dilation_rate, "ConvolDescriptor::compute_padding")

    def build(self, in_shape):
        if len(in_shape) != 4:
            msg("Tensors are not 4D", "ConvolDescriptor::build")
        if any(d != 1 for d in self.dilation_rate):
            # the non-cuDNN backends of the reference reject dilation at run time (src/tensor/nn/tensor_conv.cpp:48-51)
            msg("Dilated convolutions are only available with CuDNN", "tensorNN::Conv2D")
        self.nk, self.kr, self.kc = self.ksize
        self.kz = in_shape[1] // self.groups
        self.sr, self.sc = self.stride
        self.in_, self.iz, self.ir, self.ic = in_shape  # `in` is a Python keyword
        self.z = self.nk
        d0, d1 = self.dilation_rate
        # (the reference reads these without a check; a graph from a file can hold anything)
        if min(self.kr, self.kc, self.sr, self.sc, d0, d1) < 1:
            msg("Kernel sizes, strides and dilations must be positive", "ConvolDescriptor::build")
        if self.padding == "custom" and len(self.pads) != 4:
            msg("Custom padding takes four values (top, bottom, left, right), got %d" % len(self.pads), "ConvolDescriptor::build")
        if self.padding == "custom":
            self.r = _out_custom(self.pads[0:2], self.ir, self.kr, self.sr, d0)
            self.c = _out_custom(self.pads[2:4], self.ic, self.kc, self.sc, d1)
        else:
            pr = {"same,none": "same", "none,same": "none"}.get(self.padding, self.padding)
            pc = {"same,none": "none", "none,same": "same"}.get(self.padding, self.padding)
            self.r = self.compute_output(pr, self.ir, self.kr, self.sr, d0)
            self.c = self.compute_output(pc, self.ic, self.kc, self.sc, d1)
            padr = self.compute_padding(self.r, self.ir, self.kr, self.sr, self.padding, True, d0)
            padc = self.compute_padding(self.c, self.ic, self.kc, self.sc, self.padding, False, d1)
            self.pads = [padr[0], padr[1], padc[0], padc[1]]
        self.padrt, self.padrb, self.padcl, self.padcr = self.pads
        if self.r <= 0 or self.c <= 0:
            msg("Invalid output shape", "ConvolDescriptor::build")
        self.out_shape = [in_shape[0], self.z, self.r, self.c]
        self.K_shape = [self.nk, self.kz, self.kr, self.kc]
        return self

    def resize(self, b):
        self.in_ = b
        self.out_shape[0] = b


class PoolDescriptor:
    """Geometry of one 2-D pooling layer.  ``padding`` is a name, or a 4-list
    [top, bottom, left, right] for custom pads."""

    def __init__(self, ks, st, p, mem=0):
        where = "PoolDescriptor::PoolDescriptor"
        if len(ks) != 2:
            msg("Pooling Kernels must have 2 dimensions", where)
        if len(st) != 2:
            msg("Strides must have 2 dimensions", where)
        self.ksize = list(ks)
        self.stride = list(st)
        self.mem_level = mem
        if isinstance(p, str):
            if p not in ("same", "none", "valid", "zeros"):
                msg("Incorrect padding type", where)
            self.padding = p
            self.pad = []
        else:
            self.padding = "custom"
            self.pad = list(p)

    def build(self, in_shape):
        if len(in_shape) != 4:
            msg("Tensors are not 4D", "PoolDescriptor::build")
        self.kr, self.kc = self.ksize
        self.sr, self.sc = self.stride
        self.in_, self.iz, self.ir, self.ic = in_shape
        self.z = self.iz
        if min(self.kr, self.kc, self.sr, self.sc) < 1:
            msg("Kernel sizes, strides and dilations must be positive", "PoolDescriptor::build")
        if self.padding == "custom" and len(self.pad) != 4:
            msg("Custom padding takes four values (top, bottom, left, right), got %d" % len(self.pad), "PoolDescriptor::build")
        if self.padding == "custom":
            # the reference passes the whole 4-vector and reads entries [0] and [1] for BOTH axes
            self.r = _out_custom(self.pad, self.ir, self.kr, self.sr)
            self.c = _out_custom(self.pad, self.ic, self.kc, self.sc)
        else:
            where = "PoolDescriptor::compute_output"
            self.r = _out_named(self.padding, self.ir, self.kr, self.sr, 1, where)
            self.c = _out_named(self.padding, self.ic, self.kc, self.sc, 1, where)
            padr = _pads_named(self.r, self.ir, self.kr, self.sr, self.padding, 1, where)
            padc = _pads_named(self.c, self.ic, self.kc, self.sc, self.padding, 1, where)
            self.pad = [padr[0], padr[1], padc[0], padc[1]]
        self.padrt, self.padrb, self.padcl, self.padcr = self.pad
        if self.r <= 0 or self.c <= 0:
            msg("Invalid output shape", "PoolDescriptor::build")
        self.out_shape = [in_shape[0], self.z, self.r, self.c]
        # number of outputs per image the loops write (descriptor_pool2D.cpp:113-117)
        rows = len(range(-self.padrt, self.ir + self.padrb - self.kr + 1, self.sr))
        cols = len(range(-self.padcl, self.ic + self.padcr - self.kc + 1, self.sc))
        self.loop_rows, self.loop_cols = rows, cols
        self.size = self.iz * rows * cols
        return self

    def resize(self, b):
        self.in_ = b
        self.out_shape[0] = b
