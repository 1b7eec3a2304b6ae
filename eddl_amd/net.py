"""Forward-only model graphs over the HIP backend.

The layer factories carry the names and arguments of the reference's API
(src/apis/eddl.cpp:521-539,604-608,680-704,852-854,894-905,931-943,1067-1069,1150-1190,1264-1273)
and each layer's unfused forward is the one call its reference counterpart makes
(LConv::forward -> Conv2D, LBatchNorm::forward -> BatchNormForward in inference mode,
LActivation -> ReLu/Sigmoid/FullSoftmax, LMaxPool -> MPool2D, LAveragePool -> AvgPool2D,
LResize -> scale, LConcat -> concat, LAdd -> fill_+inc, LSum -> add, LPad -> pad,
LDense -> mult2D + sum2D_rowwise, LReshape -> shared storage).

``Net.build(backend, fuse=True)`` additionally runs a fusion pass in the spirit of the
reference's FPGA model transformation (src/apis/fpga.cpp:173-331,656+): chains
Pad(0) -> Conv -> BatchNorm -> Add -> ReLU whose intermediate results have one consumer become
ONE convolution launch with a fused epilogue.  The arithmetic per element is unchanged
(same operations, same order, each rounded to fp32).
"""
import numpy as np

from .descriptors import ConvolDescriptor, PoolDescriptor, msg


class Layer:
    """A node of the graph: ``kind``, parents, output shape (batch first) and host parameters."""
    _count = {}

    def __init__(self, kind, parents, out_shape, name="", **attrs):
        Layer._count[kind] = Layer._count.get(kind, 0) + 1
        self.kind = kind
        self.name = name or "%s%d" % (kind, Layer._count[kind])
        self.parents = list(parents)
        self.children = []
        for p in self.parents:
            p.children.append(self)
        self.out_shape = [int(d) for d in out_shape]
        self.attrs = attrs
        self.params = {}  # name -> float32 numpy array (host copy; pushed to the device by Net.build)

    def __repr__(self):
        return "<%s %s %s>" % (self.kind, self.name, self.out_shape)


class AsymmetricPaddingException(RuntimeError):
    """Raised like the reference's (src/layers/conv/layer_conv2D.cpp:57-61)."""

    def __init__(self, text, pads):
        super().__init__(text)
        self.pads = list(pads)


# ---------------------------------------------------------------------------- layer factories
def Input(shape, batch=1, name=""):
    """``shape`` excludes the batch dimension, as in eddl::Input."""
    return Layer("input", [], [batch] + list(shape), name)


def Conv2D(parent, filters, kernel_size, strides=(1, 1), padding="same", use_bias=True, groups=1, dilation_rate=(1, 1), name="",
           pads=()):
    """eddl::Conv2D; ``padding="custom"`` with ``pads=[top, bottom, left, right]`` is the LConv constructor form."""
    if len(parent.out_shape) != 4:
        msg("LConv only works over 4D tensors", "LConv::LConv")
    cd = ConvolDescriptor(filters, kernel_size, strides, padding, pads, groups, dilation_rate, use_bias).build(parent.out_shape)
    l = Layer("conv2d", [parent], cd.out_shape, name, cd=cd)
    if cd.pads[0] != cd.pads[1] or cd.pads[2] != cd.pads[3]:
        raise AsymmetricPaddingException(
            "In layer %s: Padding asymmetry detected (top=%d, bottom=%d, left=%d, right=%d). The padding asymmetry is not "
            "allowed in a Conv layer, we suggest you to use an explicit padding layer before this layer to fix the asymmetry."
            % (l.name, cd.pads[0], cd.pads[1], cd.pads[2], cd.pads[3]), cd.pads)
    l.params["K"] = np.zeros(cd.K_shape, np.float32)
    l.params["bias"] = np.zeros(cd.nk, np.float32)
    return l


def BatchNormalization(parent, affine=True, momentum=0.99, epsilon=1e-3, name=""):
    C = parent.out_shape[1]
    l = Layer("batchnorm", [parent], parent.out_shape, name, affine=affine, momentum=momentum, epsilon=float(epsilon))
    # parameter order of the reference layer: bn_g, bn_b, mean, variance (layer_batchnorm.cpp:70-71)
    if affine:
        l.params["bn_g"] = np.ones(C, np.float32)
        l.params["bn_b"] = np.zeros(C, np.float32)
    l.params["mean"] = np.zeros(C, np.float32)
    # the running variance starts at 0 when momentum > 0 (layer_batchnorm.cpp:51-56)
    l.params["variance"] = np.zeros(C, np.float32) if momentum > 0.0 else np.ones(C, np.float32)
    return l


def ReLu(parent, name=""):
    return Layer("relu", [parent], parent.out_shape, name)


def Sigmoid(parent, name=""):
    return Layer("sigmoid", [parent], parent.out_shape, name)


def Softmax(parent, axis=-1, name=""):
    nd = len(parent.out_shape)
    if axis < 0:
        axis += nd
    if axis <= 0 or axis >= nd:
        msg("The axis of a softmax must not be the batch", "LActivation::LActivation")
    return Layer("softmax", [parent], parent.out_shape, name, axis=axis)


def _pool(kind, parent, pool_size, strides, padding, name):
    pd = PoolDescriptor(pool_size, strides, padding).build(parent.out_shape)
    if pd.pad[0] != pd.pad[1] or pd.pad[2] != pd.pad[3]:
        # src/layers/pool/layer_maxpool.cpp:46-51, layer_avgpool2D.cpp:43-48 (the layer is not linked to its parent)
        raise AsymmetricPaddingException(
            "In layer %s: Padding asymmetry detected (top=%d, bottom=%d, left=%d, right=%d). The padding asymmetry is not "
            "allowed in a %s layer, we suggest you to use an explicit padding layer before this layer to fix the asymmetry."
            % (name or kind, pd.pad[0], pd.pad[1], pd.pad[2], pd.pad[3], "MaxPool" if kind == "maxpool2d" else "AveragePool"), pd.pad)
    if pd.loop_rows != pd.r or pd.loop_cols != pd.c:
        msg("pooling window walk (%dx%d) disagrees with the descriptor's output shape (%dx%d)"
            % (pd.loop_rows, pd.loop_cols, pd.r, pd.c), "LPool::LPool")
    return Layer(kind, [parent], pd.out_shape, name, pd=pd)


def MaxPool2D(parent, pool_size=(2, 2), strides=(2, 2), padding="none", name=""):
    """``padding`` may also be a 4-list [top, bottom, left, right] (the LMaxPool vector<int> constructor)."""
    return _pool("maxpool2d", parent, pool_size, strides, padding, name)


def AveragePool2D(parent, pool_size=(2, 2), strides=(2, 2), padding="none", name=""):
    return _pool("avgpool2d", parent, pool_size, strides, padding, name)


def GlobalAveragePool2D(parent, name=""):
    if len(parent.out_shape) != 4:
        msg("GlobalAveragePool only works over 4D tensors", "GlobalAveragePool2D")
    return AveragePool2D(parent, [parent.out_shape[2], parent.out_shape[3]], [1, 1], "none", name or "GlobalAveragePool2D")


def UpSampling2D(parent, size, interpolation="nearest", name=""):
    if len(parent.out_shape) != 4:
        msg("The number of dimensions of the input tensor must be 4", "EDDL::UpSampling2D")
    if len(size) != 2:
        msg('The number of dimensions of the "size" parameter must be 2', "EDDL::UpSampling2D")
    if min(size) < 1:
        msg('The scale factors in "size" parameter must be greater or equal to 1', "EDDL::UpSampling2D")
    s = parent.out_shape
    target = [s[2] * size[0], s[3] * size[1]]
    return Layer("resize", [parent], [s[0], s[1]] + target, name, new_shape=target)


def Concat(layers, axis=0, name=""):
    """``axis`` excludes the batch dimension (0 = channels), as in eddl::Concat."""
    if len(layers) < 2:
        msg("Concat requires a minimum of two tensors", "Tensor::concat")
    ax = axis + 1
    shape = list(layers[0].out_shape)
    for l in layers[1:]:
        if len(l.out_shape) != len(shape):
            msg("The number of dimensions of all tensors must match", "Tensor::concat")
        for j, (a, b) in enumerate(zip(shape, l.out_shape)):
            if j != ax and a != b:
                msg("The dimensions across of all tensors must match (%d!=%d)" % (a, b), "Tensor::concat")
        shape[ax] += l.out_shape[ax]
    return Layer("concat", layers, shape, name, axis=ax)


def Add(l1, l2=None, name=""):
    """eddl::Add(l1, l2) (an LSum: one add) or eddl::Add({l1, l2, ...}) (an LAdd: fill_(0) then inc per parent)."""
    if l2 is None:
        layers = list(l1)
        for l in layers[1:]:
            if l.out_shape != layers[0].out_shape:
                msg("Error adding layers with different tensor shape", "LAdd::LAdd")
        return Layer("add_n", layers, layers[0].out_shape, name)
    if l1.out_shape != l2.out_shape:
        msg("Error adding layers with different tensor shape", "LSum::LSum")
    return Layer("sum", [l1, l2], l1.out_shape, name)


def Pad(parent, pads, constant=0.0, name=""):
    """``pads`` = [top, right, bottom, left], or [rows, cols]."""
    if len(pads) == 2:
        pads = [pads[0], pads[1], pads[0], pads[1]]
    elif len(pads) != 4:
        msg("The padding on each border must follow this format (top-bottom, left-right) or (top, right, bottom, left)", "LPad::LPad")
    if min(pads) < 0:
        msg("Pad margin must be greater or equal than zero", "Tensor::pad")
    s = parent.out_shape
    return Layer("pad", [parent], [s[0], s[1], s[2] + pads[0] + pads[2], s[3] + pads[1] + pads[3]], name, pads=list(pads),
                 constant=float(constant))


def Reshape(parent, shape, name=""):
    """``shape`` excludes the batch; one entry may be -1."""
    per_image = int(np.prod(parent.out_shape[1:]))
    shape = list(shape)
    if shape.count(-1) > 1:
        msg("Ambiguous reshape, more than one -1", "Reshape")
    if -1 in shape:
        known = int(np.prod([d for d in shape if d != -1])) if len(shape) > 1 else 1
        shape[shape.index(-1)] = per_image // known
    if int(np.prod(shape)) != per_image:
        msg("Incompatible shapes", "Reshape")
    return Layer("reshape", [parent], [parent.out_shape[0]] + shape, name)


def Flatten(parent, name=""):
    return Reshape(parent, [-1], name)


def Dense(parent, ndim, use_bias=True, name=""):
    in_dim = parent.out_shape[-1]
    l = Layer("dense", [parent], parent.out_shape[:-1] + [ndim], name, use_bias=use_bias)
    l.params["W"] = np.zeros((in_dim, ndim), np.float32)  # [in, out], as the reference stores it
    l.params["bias"] = np.zeros(ndim, np.float32)
    return l


# ---------------------------------------------------------------------------- the net
class Op:
    """One launch group of the built plan.  ``flops``/``bytes`` are the algorithmic figures
    (convolution: 2*N*K*C*R*S*P*Q and 4*(in + filters + out); bandwidth operators: bytes moved once)."""

    def __init__(self, kind, name, run, flops=0, nbytes=0, layers=()):
        self.kind, self.name, self.run, self.flops, self.bytes, self.layers = kind, name, run, flops, nbytes, list(layers)


class Net:
    def __init__(self, inputs, outputs):
        self.lin, self.lout = list(inputs), list(outputs)
        self.layers = self._topological()
        self.backend = None

    def _topological(self):
        """The reference's layer order, which is also the order of a saved parameter file:
        layers collected by a depth-first walk along the children from every input (stopping at
        output layers), then the not yet seen ancestors of the outputs (Net::Net, walk, walk_back:
        src/net/net.cpp:77-114,231-258), then sorted by repeatedly taking the FIRST layer of that
        list whose parents have all been taken (Net::fts, src/net/net_build.cpp:34-70)."""
        collected, seen = [], set()
        outs = {id(o) for o in self.lout}
        stack = [[l, None] for l in reversed(self.lin)]
        while stack:  # iterative pre-order walk, children in creation order
            l, it = stack[-1]
            if it is None:
                if id(l) in seen:
                    stack.pop()
                    continue
                seen.add(id(l))
                collected.append(l)
                if id(l) in outs:
                    stack.pop()
                    continue
                stack[-1][1] = it = iter(l.children)
            nxt = next(it, None)
            if nxt is None:
                stack.pop()
            else:
                stack.append([nxt, None])
        back, seen_back = [], set()
        stack = list(reversed(self.lout))
        while stack:  # pre-order walk along the parents
            l = stack.pop()
            if id(l) in seen_back:
                continue
            seen_back.add(id(l))
            back.append(l)
            stack.extend(reversed(l.parents))
        collected += [l for l in back if id(l) not in seen]
        index = {id(l): i for i, l in enumerate(collected)}
        for i in self.lin:
            if id(i) not in seen_back:
                msg("input layer %s does not reach an output" % i.name, "Net::build")
        pending = [sum(1 for p in l.parents if id(p) in index) for l in collected]
        taken = [False] * len(collected)
        order = []
        for _ in collected:
            j = next((k for k in range(len(collected)) if pending[k] == 0 and not taken[k]), None)
            if j is None:
                msg("error recurrent net", "Net.fts")
            taken[j] = True
            order.append(collected[j])
            for c in collected[j].children:
                if id(c) in index:
                    pending[index[id(c)]] -= 1
        return order

    # ---- parameters (host side), in the reference's per-layer order
    def get_parameters(self):
        return [[p.copy() for p in l.params.values()] for l in self.layers]

    def set_parameters(self, params):
        for l, ps in zip(self.layers, params):
            for key, v in zip(list(l.params), ps):
                if tuple(v.shape) != l.params[key].shape:
                    msg("parameter %s of %s has shape %s, expected %s" % (key, l.name, v.shape, l.params[key].shape), "Net::set_parameters")
                l.params[key] = np.ascontiguousarray(v, np.float32)
        if self.backend is not None:
            self._push_parameters()

    # ---- parameter files: the reference's "bin" format (Net::save / Net::load, src/net/net.cpp:411-449):
    # for every layer in layer order, for every parameter in the layer's order (Layer::save,
    # src/layers/layer.cpp:215-227; convolution K, bias; batch-norm bn_g, bn_b, mean, variance;
    # dense W, bias), one record  int32 ndim | int32 shape[ndim] | float32 data[prod(shape)]
    # (Tensor::save2bin / load_from_bin, src/tensor/tensor_serialization.cpp:70-110,252-261).
    def save(self, filename, format="bin"):
        if format != "bin":
            msg("Format not implemented: *.'%s'" % format, "Tensor::save")
        with open(filename, "wb") as fh:
            for l in self.layers:
                for v in l.params.values():
                    fh.write(np.array([v.ndim] + list(v.shape), np.int32).tobytes())
                    fh.write(np.ascontiguousarray(v, np.float32).tobytes())

    def load(self, filename, format="bin"):
        if format != "bin":
            msg("Format not implemented: *.'%s'" % format, "Tensor::load")
        try:
            fh = open(filename, "rb")
        except OSError:
            raise RuntimeError("File not found. Check the file name and try again (Net::load)")
        with fh:
            for l in self.layers:
                for key, cur in l.params.items():
                    head = fh.read(4)
                    if len(head) < 4:
                        msg("parameter file ends before %s of layer %s" % (key, l.name), "Net::load")
                    ndim = int(np.frombuffer(head, np.int32)[0])
                    if ndim < 0 or ndim > 8:
                        msg("parameter file is not in the bin format (ndim %d at %s of layer %s)" % (ndim, key, l.name), "Net::load")
                    shape = np.frombuffer(fh.read(4 * ndim), np.int32)
                    size = int(np.prod(shape, dtype=np.int64)) if ndim else 1
                    # Tensor::copy accepts any shape of the same size (src/tensor/tensor_core.cpp:316-349)
                    if len(shape) != ndim or size != cur.size:
                        msg("Tensors with different size (%s of layer %s: file %s, layer %s)" % (key, l.name, list(shape), list(cur.shape)),
                            "Tensor::copy")
                    data = np.frombuffer(fh.read(4 * size), np.float32)
                    if data.size != size:
                        msg("parameter file ends inside %s of layer %s" % (key, l.name), "Net::load")
                    l.params[key] = data.reshape(cur.shape).copy()
        if self.backend is not None:
            self._push_parameters()

    def _push_parameters(self):
        for l in self.layers:
            for key, v in l.params.items():
                self.dparams[id(l)][key].copy_from(v)

    # ---- build
    def build(self, backend, fuse=True, cache_filters=True):
        """``cache_filters``: the plan is an inference plan whose parameters change only through
        ``set_parameters``, so the library may keep each convolution's repacked filters between calls."""
        self.backend = hip = backend
        self.fused = fuse
        self.cache_filters = cache_filters
        self._staging = None
        self.dparams = {id(l): {k: hip.empty(v.shape) for k, v in l.params.items()} for l in self.layers}
        self._push_parameters()
        self.out = {}   # id(layer) -> DeviceTensor holding its output (absent for layers folded into a fused op)
        self.aux = {}   # id(layer) -> extra tensors (pool indices, bn side outputs)
        self.ops = []
        self.graph = None  # a captured plan names the tensors of the build it was recorded on
        absorbed = set()
        sole_child = lambda l: l.children[0] if len(l.children) == 1 and l not in self.lout else None

        for l in self.layers:
            if id(l) in absorbed:
                continue
            if l.kind == "input":
                self.out[id(l)] = hip.empty(l.out_shape)
                continue
            if fuse and l.kind == "pad" and l.attrs["constant"] == 0.0:
                c = sole_child(l)
                if c is not None and c.kind == "conv2d":
                    continue  # folded into the convolution below (its op is emitted when the conv is reached)
            if fuse and self._concat_folds(l, sole_child):
                continue  # the convolution below reads the two tensors itself; no concatenated copy is made
            if fuse and self._resize_folds(l, sole_child):
                continue  # the convolution below reads the small tensor through the upsampling's index map
            if l.kind == "conv2d":
                self._emit_conv(l, fuse, absorbed, sole_child)
                continue
            if l.kind == "dense":
                self._emit_dense(l, fuse, absorbed, sole_child)
                continue
            self._emit_plain(l)
        for o in self.lout:
            if id(o) not in self.out:
                msg("output layer %s was fused away" % o.name, "Net::build")
        if cache_filters:
            for l in self.layers:
                if l.kind == "conv2d":
                    hip.cache_conv_filters(self.dparams[id(l)]["K"])
        return self

    @staticmethod
    def _concat_folds(l, sole_child):
        """A channel Concat of two equal-shaped 4-D tensors whose only consumer is a 1x1, 2x2 or 3x3 convolution is
        folded into that convolution, which then takes its first and second half of the channels from the two
        tensors (``eddlhip_conv2d_fwd_concat``): the same taps in the same order, so the same result bit for bit."""
        if l.kind != "concat" or l.attrs["axis"] != 1 or len(l.parents) != 2 or len(l.out_shape) != 4:
            return False
        if list(l.parents[0].out_shape) != list(l.parents[1].out_shape) or l.parents[0] is l.parents[1]:
            return False
        c = sole_child(l)
        if c is None or c.kind != "conv2d":
            return False
        cd = c.attrs["cd"]
        return cd.kr == cd.kc and cd.kr in (1, 2, 3)

    @staticmethod
    def _resize_folds(l, sole_child):
        """A nearest UpSampling2D by whole factors whose only consumer is a 1x1, 2x2 or 3x3 convolution - directly
        or through a zero Pad that the convolution absorbs - is folded into that convolution's gather
        (``eddlhip_conv2d_fwd_upsampled``): the enlarged tensor is never written."""
        if l.kind != "resize" or len(l.out_shape) != 4:
            return False
        (H, W), (NH, NW) = l.parents[0].out_shape[2:], l.attrs["new_shape"]
        if NH % H or NW % W or list(l.out_shape[2:]) != [NH, NW]:
            return False
        c = sole_child(l)
        if c is not None and c.kind == "pad" and c.attrs["constant"] == 0.0:
            c = sole_child(c)
        if c is None or c.kind != "conv2d":
            return False
        cd = c.attrs["cd"]
        return cd.kr == cd.kc and cd.kr in (1, 2, 3)

    def _emit_conv(self, l, fuse, absorbed, sole_child):
        hip, cd = self.backend, l.attrs["cd"]
        src = l.parents[0]
        pt, pl = cd.padrt, cd.padcl
        if fuse and src.kind == "pad" and id(src) not in self.out:
            t, r, b, le = src.attrs["pads"]  # (top, right, bottom, left) -> added to the conv's top/left
            pt, pl = pt + t, pl + le
            src = src.parents[0]
        upsample = None
        if fuse and src.kind == "resize" and id(src) not in self.out:
            (NH, NW), (H0, W0) = src.attrs["new_shape"], src.parents[0].out_shape[2:]
            upsample = (NH // H0, NW // W0)
            src = src.parents[0]
        second = None
        if fuse and src.kind == "concat" and id(src) not in self.out:
            second = self.out[id(src.parents[1])]
            src = src.parents[0]
        bn = res = None
        relu = False
        last = l
        if fuse:
            c = sole_child(last)
            if c is not None and c.kind == "batchnorm":
                bn, last = c, c
                c = sole_child(last)
            if c is not None and c.kind == "sum":
                other = c.parents[1] if c.parents[0] is last else c.parents[0]
                if id(other) in self.out and other is not last:
                    res, last = other, c
                    c = sole_child(last)
            elif c is not None and c.kind == "add_n" and len(c.parents) == 2:
                # an LAdd of two layers computes (0 + a) + b, which differs from a + b only in the sign of a zero
                # result; a ReLU behind it maps both to +0, so the pair is taken only together
                other = c.parents[1] if c.parents[0] is last else c.parents[0]
                nxt = sole_child(c)
                if id(other) in self.out and other is not last and nxt is not None and nxt.kind == "relu":
                    res, last = other, c
                    c = nxt
            if c is not None and c.kind == "relu":
                relu, last = True, c
        # collect absorbed layers (everything between l and last)
        chain = []
        cur = l
        while cur is not last:
            cur = cur.children[0]
            chain.append(cur)
        for m in chain:
            absorbed.add(id(m))
        # a 2x2, stride-2, unpadded MaxPool of the chain's output joins the call (eddlhip_conv2d_fwd_maxpool: a convolution
        # in a Winograd form pools in its epilogue); the unpooled tensor is kept only if somebody else reads it
        pool, keep = None, True
        if fuse and cd.out_shape[2] % 2 == 0 and cd.out_shape[3] % 2 == 0:
            for c in last.children:
                pd = c.attrs.get("pd")
                if c.kind == "maxpool2d" and len(c.parents) == 1 and list(pd.ksize) == [2, 2] and list(pd.stride) == [2, 2] and not any(pd.pad):
                    pool = c
                    keep = len(last.children) > 1 or last in self.lout
                    absorbed.add(id(c))
                    break
        O = hip.empty(last.out_shape)
        if keep:
            self.out[id(last)] = O
        pooled = None
        if pool is not None:
            pooled = (hip.empty(pool.out_shape), hip.full(pool.out_shape, 0.0), hip.full(pool.out_shape, 0.0))
            self.out[id(pool)] = pooled[0]
            self.aux[id(pool)] = {"indX": pooled[1], "indY": pooled[2]}
        I = self.out[id(src)]
        dp = self.dparams[id(l)]
        bias = dp["bias"] if cd.use_bias else None
        dbn = None
        if bn is not None:
            bp = self.dparams[id(bn)]
            dbn = (bp.get("bn_g"), bp.get("bn_b"), bp["mean"], bp["variance"], bn.attrs["epsilon"])
        R = self.out[id(res)] if res is not None else None
        N, Kf, P, Q = cd.out_shape
        _, C, H, W = src.out_shape
        if second is not None:
            C = 2 * C
        flops = 2 * N * Kf * cd.kz * cd.kr * cd.kc * P * Q
        nbytes = 4 * (N * C * H * W + Kf * cd.kz * cd.kr * cd.kc + N * Kf * P * Q)
        name = "+".join(m.name for m in ([l] if not chain else [l] + chain))
        if src is not l.parents[0]:
            name = l.parents[0].name + "+" + name
        members = [l] + chain
        if pool is not None:
            name += "+" + pool.name
            members = members + [pool]
            nbytes += 12 * int(np.prod(pool.out_shape)) - (0 if keep else 4 * N * Kf * P * Q)
        self.ops.append(Op("conv2d", name,
                           lambda: hip.conv2D(I, dp["K"], bias, O, cd.sr, cd.sc, pt, pl, bn=dbn, residual=R, relu=relu, second=second,
                                              upsample=upsample, pool=pooled, keep=keep),
                           flops, nbytes, members))

    def _emit_dense(self, l, fuse, absorbed, sole_child):
        """LDense::forward = mult2D + sum2D_rowwise (src/layers/core/layer_dense.cpp:65-73); a fused plan
        makes it one call and takes a following ReLU along."""
        hip = self.backend
        src = self.out[id(l.parents[0])]
        dp = self.dparams[id(l)]
        in_dim, ndim = dp["W"].shape
        rows = int(np.prod(l.out_shape)) // ndim
        bias = dp["bias"] if l.attrs["use_bias"] else None
        last, relu = l, False
        if fuse:
            c = sole_child(l)
            if c is not None and c.kind == "relu":
                last, relu = c, True
                absorbed.add(id(c))
        O = hip.empty(last.out_shape)
        self.out[id(last)] = O
        A2, C2 = src.reshape((rows, in_dim)), O.reshape((rows, ndim))
        if fuse:
            run = lambda: hip.dense(A2, dp["W"], bias, C2, relu=relu)
        else:
            def run():
                hip.mult2D(A2, dp["W"], C2, 0)
                if bias is not None:
                    hip.sum2D_rowwise(C2, bias, C2)
        name = l.name if last is l else l.name + "+" + last.name
        layers = [l] if last is l else [l, last]
        self.ops.append(Op("dense", name, run, 2 * rows * in_dim * ndim, 4 * (rows * in_dim + in_dim * ndim + rows * ndim), layers))

    def _emit_plain(self, l):
        hip = self.backend
        k = l.kind
        ins = [self.out[id(p)] for p in l.parents]
        n_out = int(np.prod(l.out_shape))
        if k == "reshape":
            self.out[id(l)] = ins[0].reshape(l.out_shape)  # shares storage; forward does nothing
            return
        O = hip.empty(l.out_shape)
        self.out[id(l)] = O
        if k == "batchnorm":
            dp = self.dparams[id(l)]
            C = l.out_shape[1]
            opa = hip.empty(l.out_shape) if l.attrs["affine"] else None
            bn_var = hip.empty((C,))
            self.aux[id(l)] = {"opa": opa, "bn_var": bn_var}
            run = lambda: hip.batchnorm_inference(ins[0], O, opa, dp["mean"], dp["variance"], dp.get("bn_g"), dp.get("bn_b"), bn_var,
                                                  l.attrs["epsilon"])
            nbytes = 8 * n_out + 16 * C
        elif k == "relu":
            run, nbytes = (lambda: hip.relu(ins[0], O)), 8 * n_out
        elif k == "sigmoid":
            run, nbytes = (lambda: hip.sigmoid(ins[0], O)), 8 * n_out
        elif k == "softmax":
            run, nbytes = (lambda: hip.full_softmax(ins[0], O, l.attrs["axis"])), 8 * n_out
        elif k in ("maxpool2d", "avgpool2d"):
            pd = l.attrs["pd"]
            n_in = int(np.prod(l.parents[0].out_shape))
            if k == "maxpool2d":
                ix, iy = hip.full(l.out_shape, 0.0), hip.full(l.out_shape, 0.0)
                self.aux[id(l)] = {"indX": ix, "indY": iy}
                run, nbytes = (lambda: hip.mpool2D(ins[0], O, ix, iy, pd.ksize, pd.stride, pd.pad)), 4 * n_in + 12 * n_out
            else:
                run, nbytes = (lambda: hip.avgpool2D(ins[0], O, pd.ksize, pd.stride, pd.pad)), 4 * (n_in + n_out)
        elif k == "resize":
            n_in = int(np.prod(l.parents[0].out_shape))
            run, nbytes = (lambda: hip.scale(ins[0], O, l.attrs["new_shape"])), 4 * (n_in + n_out)
        elif k == "concat":
            run, nbytes = (lambda: hip.concat(O, ins, l.attrs["axis"])), 8 * n_out
        elif k == "sum":
            run, nbytes = (lambda: hip.add(1.0, ins[0], 1.0, ins[1], O, 0)), 12 * n_out
        elif k == "add_n":
            def run():
                hip.fill_(O, 0.0)
                for t in ins:
                    hip.inc(t, O)
            nbytes = 4 * n_out * (1 + 3 * len(ins))
        elif k == "pad":
            hip.fill_(O, l.attrs["constant"])  # the border is written once, here; forward copies the interior
            n_in = int(np.prod(l.parents[0].out_shape))
            run, nbytes = (lambda: hip.pad(ins[0], O, l.attrs["pads"])), 8 * n_in
        else:
            msg("layer kind %s has no forward on this backend" % k, "Net::build")
        self.ops.append(Op(k, l.name, run, 0, nbytes, [l]))

    # ---- run
    def resize(self, batch):
        """Change the batch size: every output and scratch tensor is re-created (pointers change)."""
        for l in self.layers:
            l.out_shape[0] = batch
            for key in ("cd", "pd"):
                if key in l.attrs:
                    l.attrs[key].resize(batch)
        return self.build(self.backend, self.fused, self.cache_filters)

    def forward(self, xs):
        """``xs``: one array (or DeviceTensor) per input layer.  Returns the output DeviceTensors;
        the launches are queued, not awaited."""
        if not isinstance(xs, (list, tuple)):
            xs = [xs]
        if len(xs) != len(self.lin):
            msg("Number of input tensors does not match the number of input layers", "Net::forward")
        batch = xs[0].shape[0]
        if batch != self.lin[0].out_shape[0]:
            self.resize(batch)
        for l, x in zip(self.lin, xs):
            dst = self.out[id(l)]
            if tuple(x.shape) != dst.shape:
                msg("input shape %s does not match %s" % (tuple(x.shape), dst.shape), "Net::forward")
            if isinstance(x, np.ndarray):
                dst.copy_from(x)
            elif x is not dst:
                self.backend._check(self.backend.lib.eddlhip_memcpy_d2d(self.backend.dev, dst.ptr, x.ptr, dst.nbytes))
        self.run()
        return [self.out[id(o)] for o in self.lout]

    def run(self):
        """Queue every op of the plan on the device's stream (inputs already resident)."""
        for op in self.ops:
            op.run()

    def capture(self):
        """Records the plan as a graph (one call replays every launch): for plans whose kernels are so short
        that queueing them one at a time takes longer than running them.  Runs the plan once first, so that
        the library's workspace has its final size.  The graph names this net's tensors: capture again after
        ``resize``."""
        self.run()
        self.graph = self.backend.record(self.run)
        return self.graph

    def run_graph(self):
        """Replays the captured plan on the device's stream (``capture`` first)."""
        if self.graph is None:
            msg("no captured plan: call capture() after build or resize", "Net::run_graph")
        self.graph.launch()

    def predict(self, xs):
        """Inference forward; returns host arrays (the reference's predict collects outputs to the CPU)."""
        outs = self.forward(xs)
        return [o.numpy() for o in outs]

    def predict_batches(self, batches):
        """Inference over a stream of host batches (each a list with one array per input layer, or
        one array): yields the output arrays of every batch, in order.  Transfers overlap compute:
        batch i+1 goes through a page-locked host buffer and the upload stream into a second device
        buffer while the kernels of batch i run, and the results of batch i come back while batch
        i+1 computes (the reference stages every batch through blocking copies,
        src/net/net_func.cpp:195-249).  All batches must have the built batch size."""
        hip = self.backend
        ins = [self.out[id(l)] for l in self.lin]
        outs = [self.out[id(o)] for o in self.lout]
        d2d = lambda dst, src: hip._check(hip.lib.eddlhip_memcpy_d2d(hip.dev, dst.ptr, src.ptr, dst.nbytes))
        # two staging sets; per set: pinned + device copies of inputs and outputs, and four events:
        # h2d / d2h on the upload / download stream (upload done, results on the host), consumed / computed on the
        # compute stream (device input copy read, device output copy written)
        if getattr(self, "_staging", None) is None:  # kept until the next build (page-locking memory takes milliseconds)
            self._staging = [{"pin_in": [hip.pinned(t.shape) for t in ins], "dev_in": [hip.empty(t.shape) for t in ins],
                              "pin_out": [hip.pinned(t.shape) for t in outs], "dev_out": [hip.empty(t.shape) for t in outs],
                              "h2d": hip.event(), "d2h": hip.event(), "consumed": hip.event(), "computed": hip.event()}
                             for _ in range(2)]
        sets = self._staging
        hip.synchronize()
        for s in sets:
            s["used"] = False

        def collect(s):
            s["d2h"].synchronize()
            return [p.array.copy() for p in s["pin_out"]]

        pending = None
        for i, xs in enumerate(batches):
            if not isinstance(xs, (list, tuple)):
                xs = [xs]
            if len(xs) != len(ins):
                msg("Number of input tensors does not match the number of input layers", "Net::predict_batches")
            s = sets[i % 2]
            if s["used"]:
                s["h2d"].synchronize()            # the upload of batch i-2 has left the pinned buffer
            for t, pin, x in zip(ins, s["pin_in"], xs):
                if tuple(x.shape) != t.shape:
                    msg("input shape %s does not match %s" % (tuple(x.shape), t.shape), "Net::predict_batches")
                np.copyto(pin.array, x, casting="same_kind")
            if s["used"]:
                hip.upload_wait(s["consumed"])  # batch i-2 has been copied out of this device buffer
            for k, (dst, pin) in enumerate(zip(s["dev_in"], s["pin_in"])):
                hip.h2d_async(dst, pin, s["h2d"] if k == len(ins) - 1 else None)
            hip.stream_wait(s["h2d"])
            for t, src in zip(ins, s["dev_in"]):
                d2d(t, src)
            s["consumed"].record()
            self.run()
            if s["used"]:
                hip.stream_wait(s["d2h"])         # the results of batch i-2 have left this device buffer
            for t, dst in zip(outs, s["dev_out"]):
                d2d(dst, t)
            s["computed"].record()
            hip.download_wait(s["computed"])
            for k, (pin, src) in enumerate(zip(s["pin_out"], s["dev_out"])):
                hip.d2h_async(pin, src, s["d2h"] if k == len(outs) - 1 else None)
            s["used"] = True
            if pending is not None:
                yield collect(pending)            # waits for batch i-1 while batch i computes
            pending = s
        if pending is not None:
            yield collect(pending)

    def input_tensor(self, i=0):
        return self.out[id(self.lin[i])]

    def output_of(self, layer):
        return self.out.get(id(layer))
