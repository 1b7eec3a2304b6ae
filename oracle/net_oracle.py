"""Runs a graph of eddl_amd.net layers on the CPU oracle, layer by layer, the way the
reference's Net::do_forward walks its layers (src/net/net_func.cpp:49-55).
TEST INFRASTRUCTURE ONLY (imported by tests/ and the cpu_baseline leg of bench.py)."""
import numpy as np


def forward(ora, model, xs, conv_algo="im2col", keep=False, timings=None):
    """Returns the list of output arrays (and, with ``keep``, a dict layer-name -> output)."""
    import time
    if not isinstance(xs, (list, tuple)):
        xs = [xs]
    out = {}
    aux = {}
    for l, x in zip(model.lin, xs):
        out[id(l)] = np.ascontiguousarray(x, np.float32)
    for l in model.layers:
        if l.kind == "input":
            continue
        t0 = time.perf_counter()
        ins = [out[id(p)] for p in l.parents]
        k = l.kind
        if k == "conv2d":
            cd = l.attrs["cd"]
            bias = l.params["bias"] if cd.use_bias else None
            y = ora.conv2d(ins[0], l.params["K"], bias, (cd.sr, cd.sc), cd.padrt, cd.padcl, cd.r, cd.c, algo=conv_algo)
        elif k == "batchnorm":
            y, _, _ = ora.batchnorm_inference(ins[0], l.params["mean"], l.params["variance"], l.params.get("bn_g"),
                                              l.params.get("bn_b"), l.attrs["epsilon"])
        elif k == "relu":
            y = ora.relu(ins[0])
        elif k == "sigmoid":
            y = ora.sigmoid(ins[0])
        elif k == "softmax":
            y = ora.softmax(ins[0], l.attrs["axis"])
        elif k == "maxpool2d":
            pd = l.attrs["pd"]
            y, ix, iy = ora.maxpool2d(ins[0], pd.ksize, pd.stride, pd.pad, fill=0.0)
            aux[id(l)] = (ix, iy)
        elif k == "avgpool2d":
            pd = l.attrs["pd"]
            y = ora.avgpool2d(ins[0], pd.ksize, pd.stride, pd.pad)
        elif k == "resize":
            y = ora.scale_nearest(ins[0], l.attrs["new_shape"])
        elif k == "concat":
            y = ora.concat(ins, l.attrs["axis"])
        elif k == "sum":
            y = ora.add(ins[0], ins[1])
        elif k == "add_n":
            y = np.zeros_like(ins[0])
            for t in ins:
                y = y + t
        elif k == "pad":
            y = ora.pad(ins[0], l.attrs["pads"], l.attrs["constant"])
        elif k == "reshape":
            y = ins[0].reshape([ins[0].shape[0]] + l.out_shape[1:])
        elif k == "dense":
            a = ins[0].reshape(-1, ins[0].shape[-1])
            y = ora.dense(a, l.params["W"], l.params["bias"] if l.attrs["use_bias"] else None).reshape(
                list(ins[0].shape[:-1]) + [l.params["W"].shape[1]])
        else:
            raise ValueError("no oracle for layer kind " + k)
        out[id(l)] = y
        if timings is not None:
            timings[l.kind] = timings.get(l.kind, 0.0) + time.perf_counter() - t0
    res = [out[id(o)] for o in model.lout]
    if keep:
        return res, {l.name: out[id(l)] for l in model.layers}, {l.name: aux[id(l)] for l in model.layers if id(l) in aux}
    return res
