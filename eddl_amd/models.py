"""The model graphs of the benchmark configurations, written with the factories of
:mod:`eddl_amd.net` the way the reference's examples write theirs, plus seeded synthetic
parameters (He-normal filters as src/initializers/initializer_he_normal.cpp:31-46 computes
the deviation; the reference's own generator cannot be seeded, src/random.cpp:25-26).
"""
import numpy as np

from . import net as L


# ---------------------------------------------------------------------------- synthetic parameters
def init_he_normal(model, seed, bn_stats=True):
    """Fill every parameter of ``model`` from one seeded stream (:class:`eddl_amd.synth.Synth`: mt19937 + Box-Muller,
    the generator the C++ host shares), layer by layer in graph order, tensor by tensor in the layer's parameter order,
    row-major:
      conv filters  N(0, sqrt(2 / (C*R*S))), conv bias 0
      dense weights N(0, sqrt(2 / in)), dense bias 0
      batch-norm    gamma U(0.8, 1.2), beta N(0, 0.1), running mean N(0, 0.1), running variance U(0.5, 1.5)
    ``eddl_hip::synth_he_normal`` (C++) makes the same calls in the same order.
    """
    from .synth import Synth
    rng = Synth(seed)
    f32 = np.float32
    for l in model.layers:
        if l.kind == "conv2d":
            k = l.params["K"]
            fan_in = k.shape[1] * k.shape[2] * k.shape[3]
            l.params["K"] = rng.normal(k.shape, 0.0, f32(np.sqrt(2.0 / fan_in)))
            l.params["bias"] = np.zeros_like(l.params["bias"])
        elif l.kind == "dense":
            w = l.params["W"]
            l.params["W"] = rng.normal(w.shape, 0.0, f32(np.sqrt(2.0 / w.shape[0])))
            l.params["bias"] = np.zeros_like(l.params["bias"])
        elif l.kind == "batchnorm" and bn_stats:
            C = l.params["mean"].shape[0]
            if "bn_g" in l.params:
                l.params["bn_g"] = rng.uniform(C, 0.8, 1.2)
                l.params["bn_b"] = rng.normal(C, 0.0, 0.1)
            l.params["mean"] = rng.normal(C, 0.0, 0.1)
            l.params["variance"] = rng.uniform(C, 0.5, 1.5)
    if model.backend is not None:
        model._push_parameters()
    return model


def synthetic_input(shape, seed, dist):
    """The input batch of a configuration: ``dist`` "uniform" = U(0, 1), "normal" = N(0, 1), from a stream of its own
    (``seed``), so that the parameters do not depend on the batch size."""
    from .synth import Synth
    rng = Synth(seed)
    return rng.uniform(shape, 0.0, 1.0) if dist == "uniform" else rng.normal(shape, 0.0, 1.0)


# ---------------------------------------------------------------------------- graphs
def conv_bn_relu_pool_block(batch=64, channels=64, size=56, filters=64):
    """Conv3x3(no bias) -> BatchNorm(eps 1e-5) -> ReLU -> MaxPool 2x2 s2."""
    x = L.Input([channels, size, size], batch)
    l = L.Conv2D(x, filters, [3, 3], [1, 1], "same", use_bias=False)
    l = L.BatchNormalization(l, True, 0.99, 1e-5)
    l = L.ReLu(l)
    l = L.MaxPool2D(l, [2, 2], [2, 2], "none")
    return L.Net([x], [l])


def single_conv(batch=8, channels=3, size=32, filters=32):
    """One Conv2D 3x3, stride 1, "same", with bias: the smallest configuration (the one the reference's CPU path runs today)."""
    x = L.Input([channels, size, size], batch)
    return L.Net([x], [L.Conv2D(x, filters, [3, 3], [1, 1], "same", use_bias=True)])


def vgg16(batch=32, size=224, num_classes=1000, widths=(64, 128, 256, 512, 512), dense=4096):
    """VGG-16, all 3x3 convolutions with bias and ReLU, five 2x2 max-pools, three dense layers, softmax."""
    x = L.Input([3, size, size], batch)
    l = x
    for w, reps in zip(widths, (2, 2, 3, 3, 3)):
        for _ in range(reps):
            l = L.ReLu(L.Conv2D(l, w, [3, 3], [1, 1], "same", use_bias=True))
        l = L.MaxPool2D(l, [2, 2], [2, 2], "none")
    l = L.Flatten(l)
    l = L.ReLu(L.Dense(l, dense))
    l = L.ReLu(L.Dense(l, dense))
    l = L.Softmax(L.Dense(l, num_classes))
    return L.Net([x], [l])


def _bn(l):
    return L.BatchNormalization(l, True, 0.99, 1e-5)


def resnet50(batch=64, size=224, num_classes=1000, stages=(3, 4, 6, 3), base=64):
    """ResNet-50, inference batch-norm after every convolution, convolutions without bias.
    Strided layers use explicit symmetric pads (stem 7x7 s2 p3, 3x3 s2 p1, max-pool 3x3 s2 p1):
    "same" would be asymmetric for them and the convolution layer refuses asymmetric padding."""
    x = L.Input([3, size, size], batch)
    l = L.ReLu(_bn(L.Conv2D(x, base, [7, 7], [2, 2], "custom", use_bias=False, pads=[3, 3, 3, 3])))
    l = L.MaxPool2D(l, [3, 3], [2, 2], [1, 1, 1, 1])
    width = base
    for si, blocks in enumerate(stages):
        for bi in range(blocks):
            stride = 2 if (bi == 0 and si > 0) else 1
            out_ch = width * 4
            if bi == 0:  # projection shortcut where the shape changes (built first so it precedes the main path)
                sc = _bn(L.Conv2D(l, out_ch, [1, 1], [stride, stride], "valid", use_bias=False))
            else:
                sc = l
            m = L.ReLu(_bn(L.Conv2D(l, width, [1, 1], [1, 1], "valid", use_bias=False)))
            if stride == 1:
                m = L.Conv2D(m, width, [3, 3], [1, 1], "same", use_bias=False)
            else:
                m = L.Conv2D(m, width, [3, 3], [2, 2], "custom", use_bias=False, pads=[1, 1, 1, 1])
            m = L.ReLu(_bn(m))
            m = _bn(L.Conv2D(m, out_ch, [1, 1], [1, 1], "valid", use_bias=False))
            l = L.ReLu(L.Add(m, sc))
        width *= 2
    l = L.GlobalAveragePool2D(l)
    l = L.Flatten(l)
    l = L.Dense(l, num_classes)
    return L.Net([x], [l])


def unet(batch=4, size=512, in_channels=1, widths=(64, 128, 256, 512), bottleneck=1024):
    """U-Net: [Conv3x3-BN-ReLU]x2 per level with 2x2 max-pools, UpSampling2D x2 + Conv2x2 on the way up,
    Concat with the skip, final 1x1 convolution to one channel and sigmoid.  The 2x2 convolution
    "same" would need pads (0,1): it is written Pad({0,1,1,0}) + Conv2x2 "valid", the rewrite the
    reference's ONNX importer applies (src/serialization/onnx/net/layers/conv/conv_onnx.cpp:149-173)."""
    def double(l, w):
        for _ in range(2):
            l = L.ReLu(_bn(L.Conv2D(l, w, [3, 3], [1, 1], "same", use_bias=True)))
        return l

    x = L.Input([in_channels, size, size], batch)
    l, skips = x, []
    for w in widths:
        l = double(l, w)
        skips.append(l)
        l = L.MaxPool2D(l, [2, 2], [2, 2], "none")
    l = double(l, bottleneck)
    for w, skip in zip(reversed(widths), reversed(skips)):
        l = L.UpSampling2D(l, [2, 2])
        l = L.Conv2D(L.Pad(l, [0, 1, 1, 0]), w, [2, 2], [1, 1], "valid", use_bias=True)
        l = L.Concat([skip, l])
        l = double(l, w)
    l = L.Sigmoid(L.Conv2D(l, 1, [1, 1], [1, 1], "valid", use_bias=True))
    return L.Net([x], [l])
