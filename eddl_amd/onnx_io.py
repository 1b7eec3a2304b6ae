"""ONNX files for the CNN forward path: import into, and export from, ``eddl_amd.net.Net``.

Mirrors, for the layers of this path, the reference's importer and exporter
(src/serialization/onnx/net/eddl_onnx_import.cpp:19-63, import_helpers.cpp:210-243,529-710,
export_helpers.cpp:8-120 and the per-layer files under src/serialization/onnx/net/layers/):
the same node-queue walk from the graph inputs, the same mapping of operators to layers, the same
repairs (an asymmetric padding becomes an explicit zero Pad layer in front of a "valid" layer; an Add
of a constant onto a Conv / Gemm / BatchNormalization becomes that layer's bias), the same things
ignored (ceil_mode, count_include_pad, the axis of a concat counted without the batch).

The reference reads the file with protobuf-generated classes; protobuf is not a dependency of this
package, so the handful of messages involved (ModelProto, GraphProto, NodeProto, AttributeProto,
TensorProto, ValueInfoProto; field numbers from onnx.proto, the file the reference vendors under
src/serialization/onnx/onnx_third_party/) are decoded and encoded here directly from the protobuf
wire format: a sequence of (field number << 3 | wire type) keys, wire type 0 = varint, 1 = 64-bit,
2 = length-delimited, 5 = 32-bit.
"""
import struct
import sys
from collections import deque

import numpy as np

from . import net as N
from .descriptors import msg

# ---------------------------------------------------------------------------- wire format: reading


def _varint(buf, pos):
    shift = value = 0
    while True:
        if pos >= len(buf):
            raise ValueError("truncated varint")
        b = buf[pos]
        pos += 1
        value |= (b & 0x7F) << shift
        if not b & 0x80:
            return value, pos
        shift += 7
        if shift > 63:
            raise ValueError("varint longer than 64 bits")


def _signed(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _fields(buf):
    """Yields (field number, wire type, value); value is an int for wire types 0, 1, 5 and a memoryview for 2."""
    buf = memoryview(buf)
    pos, n = 0, len(buf)
    while pos < n:
        key, pos = _varint(buf, pos)
        field, wt = key >> 3, key & 7
        if wt == 0:
            v, pos = _varint(buf, pos)
        elif wt == 1:
            if pos + 8 > n:
                raise ValueError("truncated 64-bit field")
            v = int.from_bytes(buf[pos:pos + 8], "little")
            pos += 8
        elif wt == 2:
            ln, pos = _varint(buf, pos)
            if pos + ln > n:
                raise ValueError("truncated length-delimited field")
            v = buf[pos:pos + ln]
            pos += ln
        elif wt == 5:
            if pos + 4 > n:
                raise ValueError("truncated 32-bit field")
            v = int.from_bytes(buf[pos:pos + 4], "little")
            pos += 4
        else:
            raise ValueError("unsupported wire type %d" % wt)
        yield field, wt, v


def _packed_varints(v, wt, out):
    if wt == 2:  # packed
        pos = 0
        while pos < len(v):
            x, pos = _varint(v, pos)
            out.append(_signed(x))
    else:
        out.append(_signed(v))


def _packed_fixed(v, wt, out, fmt, size):
    if wt == 2:
        out.extend(struct.unpack("<%d%s" % (len(v) // size, fmt), bytes(v)))
    else:
        out.append(struct.unpack("<" + fmt, int(v).to_bytes(size, "little"))[0])


# TensorProto.DataType (onnx.proto)
FLOAT, UINT8, INT8, UINT16, INT16, INT32, INT64, STRING, BOOL, FLOAT16, DOUBLE = 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11
_RAW_DTYPES = {FLOAT: "<f4", UINT8: "u1", INT8: "i1", UINT16: "<u2", INT16: "<i2", INT32: "<i4", INT64: "<i8", BOOL: "u1",
               FLOAT16: "<f2", DOUBLE: "<f8"}


class TensorProto:
    """dims = 1, data_type = 2, float_data = 4, int32_data = 5, int64_data = 7, name = 8, raw_data = 9, double_data = 10."""

    def __init__(self, buf=None):
        self.dims, self.data_type, self.name = [], 0, ""
        floats, int32s, int64s, doubles, raw = [], [], [], [], None
        for f, wt, v in (_fields(buf) if buf is not None else ()):
            if f == 1:
                _packed_varints(v, wt, self.dims)
            elif f == 2:
                self.data_type = v
            elif f == 4:
                _packed_fixed(v, wt, floats, "f", 4)
            elif f == 5:
                _packed_varints(v, wt, int32s)
            elif f == 7:
                _packed_varints(v, wt, int64s)
            elif f == 8:
                self.name = bytes(v).decode()
            elif f == 9:
                raw = bytes(v)
            elif f == 10:
                _packed_fixed(v, wt, doubles, "d", 8)
        # as parseTensorValues does (src/serialization/onnx/net/utils_onnx.cpp:24-120): every type becomes floats
        if raw is not None and self.data_type in _RAW_DTYPES:
            vals = np.frombuffer(raw, _RAW_DTYPES[self.data_type])
        elif self.data_type == FLOAT:
            vals = np.array(floats, np.float32)
        elif self.data_type == INT64:
            vals = np.array(int64s, np.int64)
        elif self.data_type == DOUBLE:
            vals = np.array(doubles, np.float64)
        else:
            vals = np.array(int32s, np.int64)
        self.values = vals.astype(np.float32)


class AttributeProto:
    """name = 1, f = 2, i = 3, s = 4, t = 5, floats = 7, ints = 8, strings = 9, type = 20."""

    def __init__(self, buf):
        self.name, self.f, self.i, self.s, self.t, self.floats, self.ints, self.strings = "", 0.0, 0, "", None, [], [], []
        for f, wt, v in _fields(buf):
            if f == 1:
                self.name = bytes(v).decode()
            elif f == 2:
                self.f = struct.unpack("<f", int(v).to_bytes(4, "little"))[0]
            elif f == 3:
                self.i = _signed(v)
            elif f == 4:
                self.s = bytes(v).decode(errors="replace")
            elif f == 5:
                self.t = TensorProto(v)
            elif f == 7:
                _packed_fixed(v, wt, self.floats, "f", 4)
            elif f == 8:
                _packed_varints(v, wt, self.ints)
            elif f == 9:
                self.strings.append(bytes(v).decode(errors="replace"))


class NodeProto:
    """input = 1, output = 2, name = 3, op_type = 4, attribute = 5."""

    def __init__(self, buf):
        self.input, self.output, self.name, self.op_type, self.attribute = [], [], "", "", []
        for f, wt, v in _fields(buf):
            if f == 1:
                self.input.append(bytes(v).decode())
            elif f == 2:
                self.output.append(bytes(v).decode())
            elif f == 3:
                self.name = bytes(v).decode()
            elif f == 4:
                self.op_type = bytes(v).decode()
            elif f == 5:
                self.attribute.append(AttributeProto(v))

    def attr(self, name):
        for a in self.attribute:
            if a.name == name:
                return a
        return None


class ValueInfoProto:
    """name = 1, type = 2 { tensor_type = 1 { elem_type = 1, shape = 2 { dim = 1 { dim_value = 1, dim_param = 2 } } } }."""

    def __init__(self, buf):
        self.name, self.elem_type, self.dims = "", 0, []
        for f, wt, v in _fields(buf):
            if f == 1:
                self.name = bytes(v).decode()
            elif f == 2:
                for f2, _, v2 in _fields(v):
                    if f2 != 1:
                        continue
                    for f3, _, v3 in _fields(v2):
                        if f3 == 1:
                            self.elem_type = v3
                        elif f3 == 2:
                            for f4, _, v4 in _fields(v3):
                                if f4 != 1:
                                    continue
                                dim = None
                                for f5, _, v5 in _fields(v4):
                                    if f5 == 1:
                                        dim = _signed(v5)
                                    elif f5 == 2:
                                        dim = bytes(v5).decode()
                                self.dims.append(dim)


class GraphProto:
    """node = 1, name = 2, initializer = 5, input = 11, output = 12."""

    def __init__(self, buf):
        self.node, self.name, self.initializer, self.input, self.output = [], "", [], [], []
        for f, wt, v in _fields(buf):
            if f == 1:
                self.node.append(NodeProto(v))
            elif f == 2:
                self.name = bytes(v).decode()
            elif f == 5:
                self.initializer.append(TensorProto(v))
            elif f == 11:
                self.input.append(ValueInfoProto(v))
            elif f == 12:
                self.output.append(ValueInfoProto(v))


class ModelProto:
    """ir_version = 1, producer_name = 2, producer_version = 3, graph = 7, opset_import = 8 { domain = 1, version = 2 }."""

    def __init__(self, buf):
        self.ir_version, self.producer_name, self.producer_version, self.graph, self.opset_import = 0, "", "", None, []
        for f, wt, v in _fields(buf):
            if f == 1:
                self.ir_version = v
            elif f == 2:
                self.producer_name = bytes(v).decode()
            elif f == 3:
                self.producer_version = bytes(v).decode()
            elif f == 7:
                self.graph = GraphProto(v)
            elif f == 8:
                dom, ver = "", 0
                for f2, _, v2 in _fields(v):
                    if f2 == 1:
                        dom = bytes(v2).decode()
                    elif f2 == 2:
                        ver = v2
                self.opset_import.append((dom, ver))


# ---------------------------------------------------------------------------- import
def _log(text):
    print("[ONNX::INFO] " + text, file=sys.stderr)


class _Importer:
    def __init__(self, model, input_shape):
        self.graph = g = model.graph
        if g is None:
            msg("the file holds no graph", "ONNX::ImportNet")
        self.values = {t.name: t.values for t in g.initializer}        # map_init_values
        self.dims = {t.name: [int(d) for d in t.dims] for t in g.initializer}  # map_init_dims
        for n in g.node:  # constant nodes are always available (initialize_constant_nodes)
            if n.op_type == "Constant" and n.output:
                a = n.attr("value")
                if a is not None and a.t is not None:
                    self.values[n.output[0]] = a.t.values
                    self.dims[n.output[0]] = [int(d) for d in a.t.dims]
        self.layers = {}  # output_node_map: value name -> layer
        self.users = {}   # input_node_map: value name -> nodes that read it
        for n in g.node:
            for i in n.input:
                self.users.setdefault(i, []).append(n)
        init_names = set(self.values)
        true_inputs = [vi for vi in g.input if vi.name not in init_names]  # get_inputs (import_helpers.cpp:246-278)
        if not true_inputs:
            msg("the graph has no input", "ONNX::ImportNet")
        self.inputs = []
        if input_shape:
            if len(true_inputs) > 1:
                msg("The imported model has more than 1 input layer and the shape provided to reshape the model can only be applied"
                    "if the model has only one input layer.", "ONNX::ImportNet")
            self.inputs.append(N.Input(list(input_shape), name=true_inputs[0].name))
        else:
            for vi in true_inputs:
                shape = [d for d in vi.dims[1:]]
                if not shape or any(not isinstance(d, int) or d <= 0 for d in shape):
                    msg("input %s has no fixed shape after the batch dimension (%s); pass input_shape" % (vi.name, vi.dims),
                        "ONNX::ImportNet")
                self.inputs.append(N.Input(shape, name=vi.name))
        self.true_inputs = true_inputs

    # -- the queue walk of process_node_queue (import_helpers.cpp:529-598)
    def run(self):
        q = deque()
        for vi, layer in zip(self.true_inputs, self.inputs):
            self.layers[vi.name] = layer
            q.extend(self.users.get(vi.name, []))
        for n in self.graph.node:  # nodes fed by initializers and constants only (queue_constant_nodes)
            if n.op_type != "Constant" and n.input and all((not i) or i in self.values for i in n.input):
                q.append(n)
        built = set()
        while q:
            n = q.popleft()
            if n.op_type == "Constant" or not n.output or id(n) in built or n.output[0] in self.layers:
                continue  # constants are in the value map already; the node was created on an earlier visit
            n.positional = list(n.input)          # Resize addresses its inputs by position
            n.input = [i for i in n.input if i]   # empty names some exporters leave behind
            if not all(i in self.values or i in self.layers for i in n.input):
                continue  # comes back when the missing input's producer is created
            built.add(id(n))
            layer = self.build(n)
            for o in n.output:
                if layer is not None:
                    self.layers[o] = layer
                q.extend(self.users.get(o, []))
        outs = []
        for vi in self.graph.output:
            if vi.name not in self.layers:
                msg("graph output %s was not produced by any imported node" % vi.name, "ONNX::ImportNet")
            outs.append(self.layers[vi.name])
        return N.Net(self.inputs, outs)

    def parent(self, n, i=0):
        name = n.input[i]
        if name not in self.layers:
            msg("node %s (%s): input %s is a constant where a layer is expected" % (n.name, n.op_type, name), "ONNX::ImportNet")
        return self.layers[name]

    def build(self, n):
        fn = getattr(self, "op_" + n.op_type, None)
        if fn is None:
            msg("The ONNX node type %s (node %s) is outside the forward path this backend implements" % (n.op_type, n.name),
                "ONNX::ImportNet")
        return fn(n)

    # -- layers/conv/conv_onnx.cpp:6-213
    def op_Conv(self, n):
        parent = self.parent(n)
        auto_pad, pads, strides, dilations, groups = "custom", [], [], [], 1
        for a in n.attribute:
            if a.name == "auto_pad":
                auto_pad = {"NOTSET": "custom", "VALID": "valid", "SAME_UPPER": "same", "SAME_LOWER": "same"}.get(a.s, auto_pad)
            elif a.name == "dilations":
                dilations = list(a.ints)
            elif a.name == "group":
                groups = a.i
            elif a.name == "pads":
                pads = list(a.ints)
                if len(pads) == 4:  # [top, left, bottom, right] -> [top, bottom, left, right]
                    pads[1], pads[2] = pads[2], pads[1]
            elif a.name == "strides":
                strides = list(a.ints)
        if len(parent.out_shape) != 4:
            msg("node %s: only 2D convolutions are on this backend's path" % n.name, "ONNX::ImportNet")
        if n.input[1] not in self.values:
            msg("node %s: the filters are not an initializer" % n.name, "ONNX::ImportNet")
        wdims = self.dims[n.input[1]]
        kernel = wdims[2:]
        use_bias = len(n.input) > 2
        dilations = dilations or [1, 1]
        strides = strides or [1, 1]
        if not pads and auto_pad == "custom":
            pads = [0, 0, 0, 0]
        try:
            layer = N.Conv2D(parent, wdims[0], kernel, strides, auto_pad, use_bias, groups, dilations, n.name, pads)
        except N.AsymmetricPaddingException as e:
            _log("Detected a padding asymmetry in layer %s. Going to add an explicit Pad layer before to fix it." % n.name)
            parent.children.pop()  # the refused layer had linked itself to the parent
            t, b, le, r = e.pads
            pad = N.Pad(parent, [t, r, b, le], 0.0, n.name + "__asymmetric_padding")
            layer = N.Conv2D(pad, wdims[0], kernel, strides, "valid", use_bias, groups, dilations, n.name, [0, 0, 0, 0])
        layer.params["K"] = self._param(n.input[1], layer.params["K"].shape, n)
        if use_bias:
            layer.params["bias"] = self._param(n.input[2], layer.params["bias"].shape, n)
        return layer

    def _param(self, name, shape, n):
        if name not in self.values:
            msg("node %s: parameter %s is not an initializer" % (n.name, name), "ONNX::ImportNet")
        v = self.values[name]
        if v.size != int(np.prod(shape)):
            msg("node %s: parameter %s holds %d values, the layer needs %s" % (n.name, name, v.size, list(shape)), "Tensor::copy")
        return np.ascontiguousarray(v, np.float32).reshape(shape).copy()

    # -- layers/normalization/batchnorm_onnx.cpp:6-72
    def op_BatchNormalization(self, n):
        eps = n.attr("epsilon").f if n.attr("epsilon") else 1e-5
        momentum = n.attr("momentum").f if n.attr("momentum") else 0.9
        layer = N.BatchNormalization(self.parent(n), True, momentum, eps, n.name)
        for key, i in (("bn_g", 1), ("bn_b", 2), ("mean", 3), ("variance", 4)):
            layer.params[key] = self._param(n.input[i], layer.params[key].shape, n)
        return layer

    # -- layers/core/activation_onnx.cpp
    def op_Relu(self, n):
        return N.ReLu(self.parent(n), n.name)

    def op_Sigmoid(self, n):
        return N.Sigmoid(self.parent(n), n.name)

    def op_Softmax(self, n):
        parent = self.parent(n)
        nd = len(parent.out_shape)
        axis = n.attr("axis").i if n.attr("axis") else 1
        if axis < 0:
            axis += nd
        if axis < 0 or axis >= nd:
            msg("The target axis for Softmax is not valid: axis = %d" % axis, "ONNX::ImportNet")
        if axis == 0 and nd == 2:
            axis = 1
        if axis == 0:
            msg("The target axis for Softmax is not valid: axis = %d" % axis, "ONNX::ImportNet")
        return N.Softmax(parent, axis, n.name)

    # -- layers/pool/maxpool_onnx.cpp:6-128, avgpool_onnx.cpp
    def _pool(self, n, make, what):
        parent = self.parent(n)
        if len(parent.out_shape) != 4:
            msg("node %s: only 2D pooling is on this backend's path" % n.name, "ONNX::ImportNet")
        kernel, strides, pads = [], [], []
        for a in n.attribute:
            if a.name == "kernel_shape":
                kernel = list(a.ints)
            elif a.name == "strides":
                strides = list(a.ints)
            elif a.name == "pads":
                pads = list(a.ints)
                if len(pads) == 4:
                    pads[1], pads[2] = pads[2], pads[1]
            elif a.name == "ceil_mode" and a.i:
                _log("node %s: ceil_mode is ignored, as the reference ignores it (output sizes round down)" % n.name)
            elif a.name == "count_include_pad" and not a.i:
                pass  # the average always divides by the window size (count-include-pad); nothing to tell without paddings
        strides = strides or [1] * len(kernel)
        pads = pads or [0, 0, 0, 0]
        if what == "AveragePool" and any(pads) and not (n.attr("count_include_pad") and n.attr("count_include_pad").i):
            _log("node %s: padded taps count in the average, as in the reference's AveragePool" % n.name)
        try:
            return make(parent, kernel, strides, pads, n.name)
        except N.AsymmetricPaddingException as e:
            _log('Detected a padding asymmetry in the %s layer "%s". Going to add an explicit Pad layer before to fix it.' % (what, n.name))
            t, b, le, r = e.pads
            pad = N.Pad(parent, [t, r, b, le], 0.0, n.name + "__asymmetric_padding")
            return make(pad, kernel, strides, [0, 0, 0, 0], n.name)

    def op_MaxPool(self, n):
        return self._pool(n, N.MaxPool2D, "MaxPool")

    def op_AveragePool(self, n):
        return self._pool(n, N.AveragePool2D, "AveragePool")

    def op_GlobalAveragePool(self, n):
        p = self.parent(n)
        if len(p.out_shape) != 4:
            msg("node %s: only 2D pooling is on this backend's path" % n.name, "ONNX::ImportNet")
        return N.AveragePool2D(p, [p.out_shape[2], p.out_shape[3]], [1, 1], "none", n.name)

    def op_GlobalMaxPool(self, n):
        p = self.parent(n)
        if len(p.out_shape) != 4:
            msg("node %s: only 2D pooling is on this backend's path" % n.name, "ONNX::ImportNet")
        return N.MaxPool2D(p, [p.out_shape[2], p.out_shape[3]], [1, 1], "none", n.name)

    # -- layers/core/dense_onnx.cpp:5-93 (Gemm), layers/merge/matmul_onnx.cpp (MatMul against an initializer)
    def op_Gemm(self, n):
        transB = n.attr("transB").i if n.attr("transB") else 0
        for key, default in (("alpha", 1.0), ("beta", 1.0)):
            a = n.attr(key)
            if a is not None and a.f != default:
                msg("node %s: Gemm with %s = %g is not a Dense layer" % (n.name, key, a.f), "ONNX::ImportNet")
        if n.attr("transA") and n.attr("transA").i:
            msg("node %s: Gemm with transA is not a Dense layer" % n.name, "ONNX::ImportNet")
        return self._dense(n, transB)

    def op_MatMul(self, n):
        return self._dense(n, 0)

    def _dense(self, n, transB):
        wi = 1 if n.input[1] in self.values else 0
        if n.input[wi] not in self.values or n.input[1 - wi] not in self.layers:
            msg("node %s: a product of two layers is outside the forward path this backend implements" % n.name, "ONNX::ImportNet")
        if wi == 0:
            msg("node %s: weights on the left of a product are not a Dense layer" % n.name, "ONNX::ImportNet")
        parent = self.layers[n.input[0]]
        dims = self.dims[n.input[1]]
        if len(dims) != 2:
            msg("node %s: the weights of a Dense layer must be a matrix" % n.name, "ONNX::ImportNet")
        W = np.ascontiguousarray(self.values[n.input[1]], np.float32).reshape(dims)
        if transB:
            W = W.T
        use_bias = len(n.input) > 2
        if W.shape[0] != parent.out_shape[-1]:
            msg("node %s: weights %s do not match the input %s" % (n.name, list(W.shape), parent.out_shape), "ONNX::ImportNet")
        layer = N.Dense(parent, W.shape[1], use_bias, n.name)
        layer.params["W"] = np.ascontiguousarray(W)
        if use_bias:
            layer.params["bias"] = self._param(n.input[2], layer.params["bias"].shape, n)
        return layer

    # -- layers/merge/add_onnx.cpp:11-143
    def op_Add(self, n):
        parents = [self.layers[i] for i in n.input if i in self.layers]
        consts = [i for i in n.input if i not in self.layers and i in self.values]
        if consts:
            bias = np.ascontiguousarray(self.values[consts[0]], np.float32).ravel()
            p = parents[0] if parents else None
            if p is not None and p.kind == "conv2d":
                cd = p.attrs["cd"]
                if bias.size != cd.nk:
                    msg("node %s: %d values added onto %d filters" % (n.name, bias.size, cd.nk), "ONNX::ImportNet")
                p.params["bias"] = bias.copy() if not cd.use_bias else (p.params["bias"] + bias).astype(np.float32)
                cd.use_bias = True
                return p
            if p is not None and p.kind == "dense":
                if bias.size != p.params["bias"].size:
                    msg("node %s: %d values added onto %d outputs" % (n.name, bias.size, p.params["bias"].size), "ONNX::ImportNet")
                p.params["bias"] = bias.copy() if not p.attrs["use_bias"] else (bias + p.params["bias"]).astype(np.float32)
                p.attrs["use_bias"] = True
                return p
            if p is not None and p.kind == "batchnorm":
                p.params["bn_b"] = self._param(consts[0], p.params["bn_b"].shape, n)
                return p
            msg("node %s: adding a constant tensor to a %s layer is outside the forward path this backend implements"
                % (n.name, p.kind if p is not None else "missing"), "ONNX::ImportNet")
        if len(parents) < 2:
            msg("Error in Add node %s. Unable to process its inputs" % n.name, "ONNX::ImportNet")
        return N.Add(parents, name=n.name)  # an LAdd, as the reference creates

    # -- layers/operators/sum_onnx.cpp:6-35: Sum of two layers is an LSum
    def op_Sum(self, n):
        if len(n.input) != 2 or n.input[1] in self.values:
            msg("Error: The second input summand of the Sum layer %s is not valid" % n.name, "ONNX::ImportNet")
        return N.Add(self.parent(n, 0), self.parent(n, 1), name=n.name)

    # -- layers/merge/concat_onnx.cpp:5-49
    def op_Concat(self, n):
        parents = [self.parent(n, i) for i in range(len(n.input))]
        axis = n.attr("axis").i if n.attr("axis") else 1
        if axis < 0:
            axis += len(parents[0].out_shape)
        if axis == 0:
            msg("Error in Concat layer %s. Concat by the dimension 0 is not allowed." % n.name, "ONNX::ImportNet")
        return N.Concat(parents, axis - 1, n.name)

    # -- layers/conv/upsampling2D_onnx.cpp:5-72 (Upsample: scales are input 1), layers/core/resize_onnx.cpp:5-62
    def op_Upsample(self, n):
        parent = self.parent(n)
        if len(n.input) > 1:
            scales = self.values.get(n.input[1])
        else:
            scales = np.array(n.attr("scales").floats, np.float32) if n.attr("scales") else None  # opset 7 keeps them in an attribute
        if scales is None or scales.size != 4:
            msg("Error in node %s. Unexpected number of scale values, expected 4." % n.name, "ONNX::ImportNet")
        self._nearest_only(n)
        return N.UpSampling2D(parent, [int(scales[2]), int(scales[3])], "nearest", n.name)

    def _nearest_only(self, n):
        mode = n.attr("mode").s if n.attr("mode") else "nearest"
        if mode != "nearest":
            msg('In Resize operator, the mode "%s" is not supported. It must be "nearest".' % mode, "ONNX::ImportNet")

    def op_Resize(self, n):
        parent = self.parent(n)
        self._nearest_only(n)
        s = parent.out_shape
        if len(s) != 4:
            msg("node %s: only 2D resizing is on this backend's path" % n.name, "ONNX::ImportNet")
        # inputs by position: X, roi, scales, sizes; an absent one is an empty name
        pos = n.positional + [""] * 4
        if pos[3] in self.values:
            target = [int(v) for v in self.values[pos[3]]][2:4]
        elif pos[2] in self.values and self.values[pos[2]].size == 4:
            sc = self.values[pos[2]]
            target = [int(s[2] * sc[2]), int(s[3] * sc[3])]
        elif pos[1] in self.values and self.values[pos[1]].size == 4 and not pos[2]:  # opset 10: X, scales
            sc = self.values[pos[1]]
            target = [int(s[2] * sc[2]), int(s[3] * sc[3])]
        else:
            msg("node %s: neither sizes nor scales are constants" % n.name, "ONNX::ImportNet")
        mode = n.attr("coordinate_transformation_mode").s if n.attr("coordinate_transformation_mode") else "half_pixel"
        if target[0] % s[2] or target[1] % s[3]:
            msg("node %s: only whole-number upscaling is on this backend's path (%s -> %s)" % (n.name, s[2:], target), "ONNX::ImportNet")
        if mode != "asymmetric" and (target[0] != s[2] or target[1] != s[3]):
            # for whole-number scale factors and nearest rounding the source pixel floor(dst / scale) is the one every mode picks
            # except where ties round differently; 'asymmetric' is what the reference's UpSampling2D layer computes
            _log("node %s: coordinate_transformation_mode %s computed as asymmetric (same pixels for whole-number nearest upscaling "
                 "with floor rounding)" % (n.name, mode))
        return N.UpSampling2D(parent, [target[0] // s[2], target[1] // s[3]], "nearest", n.name)

    # -- layers/da/pad_onnx.cpp:5-110
    def op_Pad(self, n):
        parent = self.parent(n)
        mode = n.attr("mode").s if n.attr("mode") else "constant"
        if mode != "constant":
            msg('Error importing layer %s. Only "constant" mode is supported (passed "%s").' % (n.name, mode), "ONNX::ImportNet")
        constant = n.attr("value").f if n.attr("value") else 0.0
        if n.attr("pads"):  # before opset 11
            pads = list(n.attr("pads").ints)
        else:
            if len(n.input) < 2 or n.input[1] not in self.values:
                msg("Error importing layer %s. The padding values are not constants." % n.name, "ONNX::ImportNet")
            pads = [int(v) for v in self.values[n.input[1]]]
            if len(n.input) > 2 and n.input[2] in self.values:
                c = self.values[n.input[2]]
                if c.size != 1:
                    msg("Unexpected error importing layer %s. The number of constant values is not 1" % n.name, "ONNX::ImportNet")
                constant = float(c.ravel()[0])
        if len(pads) != 8:
            msg("Error importing layer %s. The expected number of padding values is 8, got %d." % (n.name, len(pads)), "ONNX::ImportNet")
        if pads[0] or pads[1] or pads[4] or pads[5]:
            msg("Error importing layer %s. Padding the batch or the channels is not supported." % n.name, "ONNX::ImportNet")
        # (batch_b, ch_b, h_b, w_b, batch_e, ch_e, h_e, w_e) -> (top, right, bottom, left)
        return N.Pad(parent, [pads[2], pads[7], pads[6], pads[3]], constant, n.name)

    # -- layers/core/reshape_onnx.cpp:5-78
    def op_Flatten(self, n):
        return N.Reshape(self.parent(n), [-1], n.name)

    def op_Reshape(self, n):
        if len(n.input) < 2 or n.input[1] not in self.values:
            msg("node %s: the target shape is not a constant" % n.name, "ONNX::ImportNet")
        shape = [int(v) for v in self.values[n.input[1]]]
        if n.input[0] in self.layers:
            parent = self.layers[n.input[0]]
            shape = [parent.out_shape[i] if d == 0 else d for i, d in enumerate(shape)]  # 0 copies the input dimension (ONNX)
            return N.Reshape(parent, shape[1:], n.name)  # the first entry is the batch
        for o in n.output:  # a reshaped parameter stays a parameter
            self.values[o] = self.values[n.input[0]]
            self.dims[o] = shape
        return None

    def op_Identity(self, n):
        if n.input[0] in self.layers:
            return self.layers[n.input[0]]
        for o in n.output:
            self.values[o] = self.values[n.input[0]]
            self.dims[o] = self.dims[n.input[0]]
        return None


def import_net_from_onnx_bytes(data, input_shape=None):
    """import_net_from_onnx_pointer / _string (eddl_onnx_import.cpp:65-93); ``input_shape`` excludes the batch."""
    try:
        model = ModelProto(data)
    except (ValueError, struct.error, UnicodeDecodeError) as e:
        msg("Failed to parse model: %s" % e, "ONNX::ImportNet")
    return _Importer(model, input_shape).run()


def import_net_from_onnx_file(path, input_shape=None):
    """import_net_from_onnx_file (eddl_onnx_import.cpp:19-63)."""
    try:
        with open(path, "rb") as fh:
            data = fh.read()
    except OSError:
        msg("The specified path does not exist: " + str(path), "ONNX::ImportNet")
    return import_net_from_onnx_bytes(data, input_shape)


# ---------------------------------------------------------------------------- wire format: writing
def _wvarint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _wkey(field, wt):
    return _wvarint(field << 3 | wt)


def _wbytes(field, data):
    data = data.encode() if isinstance(data, str) else bytes(data)
    return _wkey(field, 2) + _wvarint(len(data)) + data


def _wint(field, v):
    return _wkey(field, 0) + _wvarint(int(v))


def _wfloat(field, v):
    return _wkey(field, 5) + struct.pack("<f", float(v))


# AttributeProto.AttributeType
_A_FLOAT, _A_INT, _A_STRING, _A_TENSOR, _A_FLOATS, _A_INTS = 1, 2, 3, 4, 6, 7


def _attr(name, value):
    out = _wbytes(1, name)
    if isinstance(value, float):
        out += _wfloat(2, value) + _wint(20, _A_FLOAT)
    elif isinstance(value, int):
        out += _wint(3, value) + _wint(20, _A_INT)
    elif isinstance(value, str):
        out += _wbytes(4, value) + _wint(20, _A_STRING)
    elif isinstance(value, bytes):  # an encoded TensorProto
        out += _wbytes(5, value) + _wint(20, _A_TENSOR)
    else:
        out += _wbytes(8, b"".join(_wvarint(int(v)) for v in value)) + _wint(20, _A_INTS)  # packed
    return out


def _tensor(name, array, dtype=FLOAT):
    """float_data / int64_data, not raw_data: what the reference's exporter writes (e.g. conv_onnx.cpp:283-297)."""
    out = b""
    a = np.asarray(array)
    if a.ndim:
        out += _wbytes(1, b"".join(_wvarint(d) for d in a.shape))
    out += _wint(2, dtype)
    if dtype == FLOAT:
        out += _wbytes(4, np.ascontiguousarray(a, "<f4").tobytes())
    else:
        out += _wbytes(7, b"".join(_wvarint(int(v)) for v in a.ravel()))
    return out + _wbytes(8, name)


def _node(op, name, inputs, outputs, attrs=()):
    out = b"".join(_wbytes(1, i) for i in inputs) + b"".join(_wbytes(2, o) for o in outputs)
    out += _wbytes(3, name) + _wbytes(4, op)
    return out + b"".join(_wbytes(5, _attr(k, v)) for k, v in attrs)


def _value_info(name, shape):
    dims = _wbytes(1, _wbytes(2, "batch"))
    for d in shape[1:]:
        dims += _wbytes(1, _wint(1, d))
    tensor_type = _wint(1, FLOAT) + _wbytes(2, dims)
    return _wbytes(1, name) + _wbytes(2, _wbytes(1, tensor_type))


def export_net_to_onnx_bytes(net):
    """build_onnx_model / set_graph (export_helpers.cpp:8-120): producer "EDDL" 1.0, opset 11, inputs and
    outputs with a symbolic batch, one node per layer in layer order, values named after the layers,
    parameters as initializers <layer>_W, _b, _scale, _bias, _mean, _variance."""
    nodes, inits = [], []
    for l in net.layers:
        ins = [p.name for p in l.parents]
        k = l.kind
        if k == "input":
            continue
        if k == "conv2d":
            cd = l.attrs["cd"]
            ins.append(l.name + "_W")
            inits.append(_tensor(l.name + "_W", l.params["K"]))
            if cd.use_bias:
                ins.append(l.name + "_b")
                inits.append(_tensor(l.name + "_b", l.params["bias"]))
            nodes.append(_node("Conv", l.name, ins, [l.name], [
                ("dilations", list(cd.dilation_rate)), ("group", int(cd.groups)), ("kernel_shape", [cd.kr, cd.kc]),
                ("pads", [cd.padrt, cd.padcl, cd.padrb, cd.padcr]), ("strides", [cd.sr, cd.sc])]))
        elif k == "batchnorm":
            C = l.out_shape[1]
            g = l.params.get("bn_g", np.ones(C, np.float32))
            b = l.params.get("bn_b", np.zeros(C, np.float32))
            for suffix, v in (("_scale", g), ("_bias", b), ("_mean", l.params["mean"]), ("_variance", l.params["variance"])):
                ins.append(l.name + suffix)
                inits.append(_tensor(l.name + suffix, v))
            nodes.append(_node("BatchNormalization", l.name, ins, [l.name],
                               [("epsilon", float(l.attrs["epsilon"])), ("momentum", float(l.attrs["momentum"]))]))
        elif k in ("relu", "sigmoid"):
            nodes.append(_node("Relu" if k == "relu" else "Sigmoid", l.name, ins, [l.name]))
        elif k == "softmax":
            nodes.append(_node("Softmax", l.name, ins, [l.name], [("axis", int(l.attrs["axis"]))]))
        elif k in ("maxpool2d", "avgpool2d"):
            pd = l.attrs["pd"]
            nodes.append(_node("MaxPool" if k == "maxpool2d" else "AveragePool", l.name, ins, [l.name], [
                ("kernel_shape", [pd.kr, pd.kc]), ("pads", [pd.padrt, pd.padcl, pd.padrb, pd.padcr]), ("strides", [pd.sr, pd.sc])]))
        elif k == "resize":
            s = l.parents[0].out_shape
            inits.append(_tensor(l.name + "_roi", np.array([0, 0, 0, 0, 1, 1, 1, 1], np.float32)))
            inits.append(_tensor(l.name + "_scales", np.array([1, 1, l.out_shape[2] // s[2], l.out_shape[3] // s[3]], np.float32)))
            nodes.append(_node("Resize", l.name, ins + [l.name + "_roi", l.name + "_scales"], [l.name],
                               [("coordinate_transformation_mode", "asymmetric"), ("mode", "nearest")]))
        elif k == "concat":
            nodes.append(_node("Concat", l.name, ins, [l.name], [("axis", int(l.attrs["axis"]))]))
        elif k == "add_n":
            nodes.append(_node("Add", l.name, ins, [l.name]))
        elif k == "sum":
            nodes.append(_node("Sum", l.name, ins, [l.name]))
        elif k == "pad":
            t, r, b, le = l.attrs["pads"]
            inits.append(_tensor(l.name + "_pads", np.array([0, 0, t, le, 0, 0, b, r], np.int64), INT64))
            inits.append(_tensor(l.name + "_value", np.array(l.attrs["constant"], np.float32)))
            nodes.append(_node("Pad", l.name, ins + [l.name + "_pads", l.name + "_value"], [l.name], [("mode", "constant")]))
        elif k == "reshape":
            shape = _tensor("const_tensor", np.array([-1] + l.out_shape[1:], np.int64), INT64)
            nodes.append(_node("Constant", "", [], [l.name + "_target_shape"], [("value", shape)]))
            nodes.append(_node("Reshape", l.name, ins + [l.name + "_target_shape"], [l.name]))
        elif k == "dense":
            ins.append(l.name + "_W")
            inits.append(_tensor(l.name + "_W", l.params["W"]))
            if l.attrs["use_bias"]:
                ins.append(l.name + "_b")
                inits.append(_tensor(l.name + "_b", l.params["bias"]))
            if len(l.parents[0].out_shape) == 2:
                nodes.append(_node("Gemm", l.name, ins, [l.name], [("alpha", 1.0), ("beta", 1.0), ("transA", 0), ("transB", 0)]))
            else:  # build_dense_with_matmul_node: MatMul, then Add of the bias
                mm = l.name + "_MatMul" if l.attrs["use_bias"] else l.name
                nodes.append(_node("MatMul", mm, ins[:2], [mm]))
                if l.attrs["use_bias"]:
                    nodes.append(_node("Add", l.name, [mm, ins[2]], [l.name]))
        else:
            msg("layer %s of kind %s has no ONNX form here" % (l.name, k), "ONNX::ExportNet")
    graph = b"".join(_wbytes(1, n) for n in nodes) + _wbytes(2, "Computational Graph")
    graph += b"".join(_wbytes(5, t) for t in inits)
    graph += b"".join(_wbytes(11, _value_info(l.name, l.out_shape)) for l in net.layers if l.kind == "input")
    graph += b"".join(_wbytes(12, _value_info(l.name, l.out_shape)) for l in net.lout)
    model = _wint(1, 6) + _wbytes(2, "EDDL") + _wbytes(3, "1.0") + _wbytes(7, graph) + _wbytes(8, _wint(2, 11))
    return model


def save_net_to_onnx_file(net, path):
    """save_net_to_onnx_file (src/serialization/onnx/net/eddl_onnx_export.cpp:17-35)."""
    with open(path, "wb") as fh:
        fh.write(export_net_to_onnx_bytes(net))
