"""Networks imported from ONNX files run on the GPU: the files PyTorch wrote (tests/golden/onnx) have to
give PyTorch's outputs, through the layer-by-layer plan and through the fused plan alike."""
import os

import numpy as np
import pytest

from eddl_amd import onnx_io as O
from oracle import net_oracle

pytestmark = pytest.mark.gpu

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "onnx")


def close(ref, out):
    ref = np.asarray(ref, np.float32)
    return bool(np.all(np.abs(ref - out) <= 1e-5 * np.abs(ref).max() + 1e-4 * np.abs(ref)))


@pytest.mark.parametrize("name", ["vgg_like", "resnet_like", "unet_like"])
def test_imported_networks_reproduce_pytorch_outputs(hip, oracle, name):
    d = np.load(os.path.join(FIX, name + ".npz"))
    net = O.import_net_from_onnx_file(os.path.join(FIX, name + ".onnx"))
    net.build(hip, fuse=False)
    plain = net.predict([d["x"]])[0]
    n_plain = len(net.ops)
    assert plain.shape == d["y"].shape and close(d["y"], plain), np.abs(plain - d["y"]).max()
    # the CPU oracle on the same graph: the usual bar of the model tests
    want = net_oracle.forward(oracle, net, [d["x"]], conv_algo="direct")[0]
    assert close(want, plain)
    net.build(hip, fuse=True)
    fused = net.predict([d["x"]])[0]
    assert np.array_equal(fused, plain)
    assert len(net.ops) < n_plain
    if name == "resnet_like":
        # both residual additions (LAdd of two layers, followed by a ReLU) went into a convolution's epilogue
        assert not [op for op in net.ops if op.kind == "add_n"]
        assert sum(1 for op in net.ops if op.kind == "conv2d" and "/Add" in op.name) == 2, [op.name for op in net.ops]


def test_exported_network_comes_back_with_the_same_outputs(hip):
    from eddl_amd import models
    m = models.resnet50(batch=2, size=64, num_classes=10, base=8)
    models.init_he_normal(m, 9)
    x = np.random.default_rng(9).standard_normal(m.lin[0].out_shape, dtype=np.float32)
    m.build(hip)
    want = m.predict([x])[0]
    back = O.import_net_from_onnx_bytes(O.export_net_to_onnx_bytes(m))
    back.build(hip)
    assert np.array_equal(back.predict([x])[0], want)


@pytest.mark.parametrize("seed", range(48))
def test_random_graphs_on_the_device(hip, oracle, seed):
    """Random small graphs over the whole layer set (tests/test_onnx_cpu.py:random_net), sent through the
    exporter and the importer first: the layer walk agrees with the CPU oracle, the fused plan with the
    layer walk bit for bit, whatever chains the graph happens to contain."""
    from test_onnx_cpu import random_net
    rng = np.random.default_rng(500 + seed)
    net = O.import_net_from_onnx_bytes(O.export_net_to_onnx_bytes(random_net(rng)))
    x = rng.standard_normal([3] + net.lin[0].out_shape[1:]).astype(np.float32)
    want = net_oracle.forward(oracle, net, [x], conv_algo="direct")[0]
    net.build(hip, fuse=False)
    plain = net.predict([x])[0]
    assert plain.shape == want.shape
    assert np.all(np.abs(plain - want) <= 1e-5 * np.abs(want).max() + 2e-4 * np.abs(want)), np.abs(plain - want).max()
    net.build(hip, fuse=True)
    assert np.array_equal(net.predict([x])[0], plain)
