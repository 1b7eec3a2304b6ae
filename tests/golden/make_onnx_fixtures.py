"""Writes the ONNX fixtures under tests/golden/onnx/: three small networks defined and exported
with PyTorch (an independent producer of ONNX files: nothing of this repository takes part), each with
a seeded input and PyTorch's own output for it.

    python tests/golden/make_onnx_fixtures.py

For every model: <name>.onnx (the exported file) and <name>.npz (x = input, y = PyTorch's output in
eval mode, fp32 on the CPU).  The importer tests read these files; PyTorch is not needed to run them.

PyTorch's TorchScript exporter serialises the model itself; only its last step, which merges
onnxscript functions into the file, imports the `onnx` package.  That package is not installed here
and no model below uses such functions, so that step is replaced by the identity for this script.
"""
import io
import os
import warnings

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "onnx")


class VggLike(nn.Module):
    """conv+relu, maxpool, conv+relu+bn, avgpool, flatten, two linear layers, softmax.  The batch norm
    follows the ReLU so that the exporter cannot fold it into the convolution and the file keeps a
    BatchNormalization node."""

    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(3, 6, 3, padding=1)
        self.c2 = nn.Conv2d(6, 8, 3, padding=1, bias=False)
        self.bn = nn.BatchNorm2d(8, eps=1e-5)
        self.f1 = nn.Linear(8 * 4 * 4, 12)
        self.f2 = nn.Linear(12, 5)

    def forward(self, x):
        y = F.max_pool2d(F.relu(self.c1(x)), 2)
        y = self.bn(F.relu(self.c2(y)))
        y = F.avg_pool2d(y, 2)
        y = torch.flatten(y, 1)
        return torch.softmax(self.f2(F.relu(self.f1(y))), dim=1)


class ResNetLike(nn.Module):
    """strided stem + bn + relu, 3x3 stride-2 padded max-pool, an identity block and a projection block
    (conv-bn-relu-conv-bn, + shortcut, relu), global average pool, linear."""

    def __init__(self):
        super().__init__()
        self.stem = nn.Conv2d(3, 8, 3, stride=2, padding=1, bias=False)
        self.bn0 = nn.BatchNorm2d(8)
        self.a1, self.abn1 = nn.Conv2d(8, 8, 3, padding=1, bias=False), nn.BatchNorm2d(8)
        self.a2, self.abn2 = nn.Conv2d(8, 8, 3, padding=1, bias=False), nn.BatchNorm2d(8)
        self.b1, self.bbn1 = nn.Conv2d(8, 16, 1, stride=2, bias=False), nn.BatchNorm2d(16)
        self.b2, self.bbn2 = nn.Conv2d(16, 16, 3, padding=1, bias=False), nn.BatchNorm2d(16)
        self.proj, self.pbn = nn.Conv2d(8, 16, 1, stride=2, bias=False), nn.BatchNorm2d(16)
        self.fc = nn.Linear(16, 7)

    def forward(self, x):
        y = F.max_pool2d(F.relu(self.bn0(self.stem(x))), 3, stride=2, padding=1)
        r = self.abn2(self.a2(F.relu(self.abn1(self.a1(y)))))
        y = F.relu(r + y)
        r = self.bbn2(self.b2(F.relu(self.bbn1(self.b1(y)))))
        y = F.relu(r + self.pbn(self.proj(y)))
        y = F.adaptive_avg_pool2d(y, 1)
        return self.fc(torch.flatten(y, 1))


class UNetLike(nn.Module):
    """conv-bn-relu, maxpool, conv-relu, nearest x2 upsampling, zero pad (right, bottom) + 2x2 conv,
    concat with the skip, 1x1 conv, sigmoid.  Exported at opset 9, where the paddings of Pad are an
    attribute and the upsampling is an Upsample node with constant scales (from opset 11 on PyTorch
    writes the paddings as a computed tensor, which the reference's importer does not read either)."""

    def __init__(self):
        super().__init__()
        self.c1, self.bn1 = nn.Conv2d(1, 4, 3, padding=1), nn.BatchNorm2d(4)
        self.c2 = nn.Conv2d(4, 8, 3, padding=1)
        self.up = nn.Conv2d(8, 4, 2)
        self.c3 = nn.Conv2d(8, 4, 3, padding=1)
        self.out = nn.Conv2d(4, 1, 1)

    def forward(self, x):
        s = F.relu(self.bn1(self.c1(x)))
        y = F.relu(self.c2(F.max_pool2d(s, 2)))
        y = F.interpolate(y, scale_factor=2, mode="nearest")
        y = self.up(F.pad(y, (0, 1, 0, 1)))
        y = F.relu(self.c3(torch.cat([s, y], dim=1)))
        return torch.sigmoid(self.out(y))


def randomise(model, seed):
    g = torch.Generator().manual_seed(seed)
    for m in model.modules():
        if isinstance(m, nn.BatchNorm2d):  # running statistics away from their initial 0 / 1
            m.running_mean.copy_(torch.randn(m.num_features, generator=g) * 0.1)
            m.running_var.copy_(torch.rand(m.num_features, generator=g) + 0.5)
            m.weight.data.copy_(torch.rand(m.num_features, generator=g) * 0.4 + 0.8)
            m.bias.data.copy_(torch.randn(m.num_features, generator=g) * 0.1)
        elif isinstance(m, (nn.Conv2d, nn.Linear)):
            m.weight.data.copy_(torch.randn(m.weight.shape, generator=g) * (2.0 / m.weight[0].numel()) ** 0.5)
            if m.bias is not None:
                m.bias.data.copy_(torch.randn(m.bias.shape, generator=g) * 0.1)


def export(name, model, shape, seed, opset):
    from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto
    torch.manual_seed(seed)
    with torch.no_grad():
        randomise(model, seed)
    model.eval()
    x = torch.randn(shape, generator=torch.Generator().manual_seed(seed + 1))
    with torch.no_grad():
        y = model(x)
    buf = io.BytesIO()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.onnx.export(model, (x,), buf, dynamo=False, opset_version=opset, do_constant_folding=True,
                          input_names=["input"], output_names=["output"])
    os.makedirs(OUT, exist_ok=True)
    with open(os.path.join(OUT, name + ".onnx"), "wb") as fh:
        fh.write(buf.getvalue())
    np.savez(os.path.join(OUT, name + ".npz"), x=x.numpy(), y=y.numpy())
    print(name, "opset", opset, len(buf.getvalue()), "bytes, output", tuple(y.shape))


if __name__ == "__main__":
    torch.set_num_threads(1)
    torch.backends.mkldnn.enabled = False  # plain fp32 kernels
    export("vgg_like", VggLike(), (2, 3, 16, 16), 11, 13)
    export("resnet_like", ResNetLike(), (2, 3, 32, 32), 12, 11)
    export("unet_like", UNetLike(), (2, 1, 16, 16), 13, 9)
