"""Host-side graph logic that needs no GPU: the reference's layer order and its "bin" parameter
files (Net::save / Net::load).  No file in that format ships with the reference, so the layout is
pinned by the source lines cited in eddl_amd/net.py and checked here against bytes assembled by
hand with struct.pack."""
import struct

import numpy as np
import pytest

from eddl_amd import models, net as L


def test_layer_order_is_the_reference_walk_then_first_ready_sort():
    # shortcut branch created BEFORE the main branch: x.children = [s, c1].
    # walk from x along children (pre-order, stop at the output):  x, s, add, r, c1, c2
    # sort, always the first layer of that list whose parents are done:  x, s, c1, c2, add, r
    x = L.Input([4, 8, 8], 1, name="x")
    s = L.Conv2D(x, 4, [1, 1], name="s")
    c1 = L.Conv2D(x, 4, [3, 3], name="c1")
    c2 = L.Conv2D(c1, 4, [3, 3], name="c2")
    add = L.Add(c2, s, name="add")
    r = L.ReLu(add, name="r")
    assert [l.name for l in L.Net([x], [r]).layers] == ["x", "s", "c1", "c2", "add", "r"]
    # main branch first: x.children = [c1, s]; walk x, c1, c2, add, r, s; sort x, c1, c2, s, add, r
    x = L.Input([4, 8, 8], 1, name="x")
    c1 = L.Conv2D(x, 4, [3, 3], name="c1")
    c2 = L.Conv2D(c1, 4, [3, 3], name="c2")
    s = L.Conv2D(x, 4, [1, 1], name="s")
    r = L.ReLu(L.Add(c2, s, name="add"), name="r")
    assert [l.name for l in L.Net([x], [r]).layers] == ["x", "c1", "c2", "s", "add", "r"]
    # a skip connection whose consumer is created late (U-Net): a.children = [p, cat]
    x = L.Input([2, 8, 8], 1, name="x")
    a = L.Conv2D(x, 2, [3, 3], name="a")
    p = L.MaxPool2D(a, name="p")
    b = L.Conv2D(p, 2, [3, 3], name="b")
    u = L.UpSampling2D(b, [2, 2], name="u")
    cat = L.Concat([a, u], name="cat")
    assert [l.name for l in L.Net([x], [cat]).layers] == ["x", "a", "p", "b", "u", "cat"]


def test_every_order_is_topological_for_the_benchmark_graphs():
    for m in (models.resnet50(batch=1, size=32, num_classes=10, base=8), models.unet(batch=1, size=32, widths=(4, 8), bottleneck=16),
              models.vgg16(batch=1, size=32, num_classes=10, dense=16)):
        pos = {id(l): i for i, l in enumerate(m.layers)}
        assert len(pos) == len(m.layers)
        for l in m.layers:
            for p in l.parents:
                assert pos[id(p)] < pos[id(l)]


def test_bin_parameter_file_layout(tmp_path):
    m = models.conv_bn_relu_pool_block(batch=1, channels=3, size=6, filters=5)
    models.init_he_normal(m, 21)
    conv = [l for l in m.layers if l.kind == "conv2d"][0]
    bn = [l for l in m.layers if l.kind == "batchnorm"][0]
    f = tmp_path / "block.bin"
    m.save(str(f))

    def rec(a):
        return struct.pack("<i", a.ndim) + struct.pack("<%di" % a.ndim, *a.shape) + a.astype("<f4").tobytes()

    # convolution: K then bias (present even without use_bias); batch-norm: bn_g, bn_b, mean, variance
    expect = rec(conv.params["K"]) + rec(conv.params["bias"]) + rec(bn.params["bn_g"]) + rec(bn.params["bn_b"]) + \
        rec(bn.params["mean"]) + rec(bn.params["variance"])
    assert f.read_bytes() == expect
    assert conv.params["K"].shape == (5, 3, 3, 3) and conv.params["bias"].shape == (5,)


def test_bin_parameter_file_round_trip_and_errors(tmp_path):
    m = models.resnet50(batch=1, size=32, num_classes=10, base=8)
    models.init_he_normal(m, 22)
    want = m.get_parameters()
    f = tmp_path / "resnet.bin"
    m.save(str(f))
    models.init_he_normal(m, 23)
    assert any(not np.array_equal(a, b) for la, lb in zip(want, m.get_parameters()) for a, b in zip(la, lb))
    m.load(str(f))
    for la, lb in zip(want, m.get_parameters()):
        for a, b in zip(la, lb):
            assert np.array_equal(a, b)
    with pytest.raises(RuntimeError, match="File not found"):
        m.load(str(tmp_path / "missing.bin"))
    data = f.read_bytes()
    (tmp_path / "short.bin").write_bytes(data[: len(data) // 2])
    with pytest.raises(RuntimeError):
        m.load(str(tmp_path / "short.bin"))
    other = models.resnet50(batch=1, size=32, num_classes=10, base=16)
    with pytest.raises(RuntimeError, match="different size"):
        other.load(str(f))
    with pytest.raises(RuntimeError, match="Format not implemented"):
        m.save(str(f), "onnx")
