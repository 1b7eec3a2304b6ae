"""ctypes binding of the C ABI: device tensors and one method per operator.

Every method launches asynchronously on the device's stream; ``DeviceTensor.numpy()`` and
``Backend.synchronize()`` wait.  Shapes follow the reference: NCHW activations, OIHW filters,
[in, out] dense weights, all float32.
"""
import ctypes

import numpy as np

from . import _lib


class EddlHipError(RuntimeError):
    """A C ABI call returned a negative code; the text is eddlhip_last_error()."""


class DeviceTensor:
    """A float32 tensor in HBM owned by this object (freed when collected)."""

    def __init__(self, backend, shape):
        self.backend = backend
        self.shape = tuple(int(d) for d in shape)
        self.size = int(np.prod(self.shape)) if len(self.shape) else 1
        self.nbytes = self.size * 4
        self.ptr = backend._malloc(self.nbytes)

    def __del__(self):
        try:
            if getattr(self, "ptr", None):
                self.backend._free(self.ptr)
                self.ptr = None
        except Exception:
            pass

    def numpy(self):
        out = np.empty(self.shape, np.float32)
        self.backend._check(self.backend.lib.eddlhip_memcpy_d2h(self.backend.dev, out.ctypes.data, self.ptr, self.nbytes))
        return out

    def copy_from(self, host):
        host = np.ascontiguousarray(host, dtype=np.float32)
        if host.size != self.size:
            raise ValueError("size mismatch: %s vs %s" % (host.shape, self.shape))
        self.backend._check(self.backend.lib.eddlhip_memcpy_h2d(self.backend.dev, self.ptr, host.ctypes.data, self.nbytes))
        return self

    def reshape(self, shape):
        """A view with another shape sharing the storage (the reference's reshape_)."""
        view = object.__new__(DeviceTensor)
        view.backend, view.ptr, view.nbytes, view.size = self.backend, self.ptr, self.nbytes, self.size
        view.shape = tuple(int(d) for d in shape)
        if int(np.prod(view.shape)) != self.size:
            raise ValueError("reshape changes the size")
        view._base = self  # keeps the owner alive
        view.__class__ = _View
        return view


class _View(DeviceTensor):
    def __del__(self):  # storage belongs to the base tensor
        pass


class PinnedArray:
    """A float32 numpy array over page-locked host memory of the library (``.array``)."""

    def __init__(self, backend, shape):
        self.backend = backend
        self.shape = tuple(int(d) for d in shape)
        n = int(np.prod(self.shape)) if len(self.shape) else 1
        self.nbytes = n * 4
        p = ctypes.c_void_p()
        backend._check(backend.lib.eddlhip_host_malloc(backend.dev, ctypes.byref(p), max(self.nbytes, 4)))
        self.ptr = p.value
        self.array = np.ctypeslib.as_array((ctypes.c_float * max(n, 1)).from_address(self.ptr))[:n].reshape(self.shape)

    def __del__(self):
        try:
            if getattr(self, "ptr", None):
                self.array = None
                self.backend.lib.eddlhip_host_free(self.backend.dev, self.ptr)
                self.ptr = None
        except Exception:
            pass


class Event:
    def __init__(self, backend):
        self.backend = backend
        h = ctypes.c_void_p()
        backend._check(backend.lib.eddlhip_event_create(backend.dev, ctypes.byref(h)))
        self.handle = h

    def record(self):
        self.backend._check(self.backend.lib.eddlhip_event_record(self.backend.dev, self.handle))
        return self

    def synchronize(self):
        self.backend._check(self.backend.lib.eddlhip_event_synchronize(self.backend.dev, self.handle))

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        self.backend._check(self.backend.lib.eddlhip_event_elapsed_ms(self.backend.dev, self.handle, stop.handle, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            self.backend.lib.eddlhip_event_destroy(self.backend.dev, self.handle)
        except Exception:
            pass


class Graph:
    """A recorded sequence of launches (``Backend.record``); ``launch()`` replays it on the device's stream."""

    def __init__(self, backend, handle):
        self.backend, self.handle = backend, handle

    def launch(self):
        self.backend._check(self.backend.lib.eddlhip_graph_launch(self.backend.dev, self.handle))

    def __del__(self):
        try:
            if self.handle:
                self.backend.lib.eddlhip_graph_destroy(self.backend.dev, self.handle)
                self.handle = None
        except Exception:
            pass


def _ptr(t):
    return None if t is None else t.ptr


class Backend:
    """One device of libeddlhip.so."""

    def __init__(self, dev=0):
        self.lib = _lib.load()
        self.dev = int(dev)
        self._deferred_free = []  # pointers whose free was refused (a graph was being recorded)
        self._check(self.lib.eddlhip_init(self.dev))

    # ---- plumbing
    def _check(self, rc):
        if rc != 0:
            raise EddlHipError("%s (code %d)" % (self.lib.eddlhip_last_error().decode(), rc))

    def _malloc(self, nbytes):
        p = ctypes.c_void_p()
        self._check(self.lib.eddlhip_malloc(self.dev, max(nbytes, 4), ctypes.byref(p)))
        return p.value

    def _free(self, ptr):
        """Frees device memory; a free is refused while a graph is being recorded (``record``), so such a pointer is
        kept and freed when the recording has ended."""
        if self.lib.eddlhip_free(self.dev, ptr) != 0:
            self._deferred_free.append(ptr)

    def _free_deferred(self):
        pending, self._deferred_free = self._deferred_free, []
        for ptr in pending:
            if self.lib.eddlhip_free(self.dev, ptr) != 0:
                self._deferred_free.append(ptr)

    def workspace_bytes(self):
        n = ctypes.c_size_t()
        self._check(self.lib.eddlhip_workspace_bytes(self.dev, ctypes.byref(n)))
        return n.value

    def workspace_trim(self):
        """Releases the library's workspace; it grows back to what the calls from now on need (after a plan search)."""
        self._check(self.lib.eddlhip_workspace_trim(self.dev))

    def record(self, fn):
        """Records the launches ``fn()`` makes into a Graph instead of running them.  ``fn`` must have
        run once before (workspace at its final size) and may only launch kernels."""
        self._check(self.lib.eddlhip_graph_begin(self.dev))
        h = ctypes.c_void_p()
        try:
            fn()
        except BaseException:
            self.lib.eddlhip_graph_end(self.dev, ctypes.byref(h))  # leaves recording mode; the first error is the one to report
            if h.value:
                self.lib.eddlhip_graph_destroy(self.dev, h)
            self._free_deferred()
            raise
        rc = self.lib.eddlhip_graph_end(self.dev, ctypes.byref(h))
        self._free_deferred()
        self._check(rc)
        return Graph(self, h)

    @property
    def name(self):
        buf = ctypes.create_string_buffer(256)
        self._check(self.lib.eddlhip_device_name(self.dev, buf, 256))
        return buf.value.decode()

    def synchronize(self):
        self._check(self.lib.eddlhip_synchronize(self.dev))

    def event(self):
        return Event(self)

    # ---- batch staging (upload and download streams)
    def pinned(self, shape):
        return PinnedArray(self, shape)

    def h2d_async(self, dst, pinned, done=None):
        self._check(self.lib.eddlhip_memcpy_h2d_async(self.dev, dst.ptr, pinned.ptr, dst.nbytes, done.handle if done else None))

    def d2h_async(self, pinned, src, done=None):
        self._check(self.lib.eddlhip_memcpy_d2h_async(self.dev, pinned.ptr, src.ptr, src.nbytes, done.handle if done else None))

    def stream_wait(self, event):
        self._check(self.lib.eddlhip_stream_wait_event(self.dev, event.handle))

    def upload_wait(self, event):
        self._check(self.lib.eddlhip_upload_wait_event(self.dev, event.handle))

    def download_wait(self, event):
        self._check(self.lib.eddlhip_download_wait_event(self.dev, event.handle))

    def _probe_lib(self):
        """The device probes live in a library of their own (libeddlhip_probe.so), loaded on first use."""
        if getattr(self, "_probe", None) is None:
            from . import _lib
            self._probe = _lib.load_probe()
        return self._probe

    def probe_mfma_f32(self, vary_operands=True, launches=40):
        """Sustained fp32 MFMA rate of the device with nothing else running: (mean, best launch, worst launch) TFLOP/s."""
        mean, best, worst = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
        self._check(self._probe_lib().eddlhip_probe_mfma_f32(self.dev, int(vary_operands), launches, ctypes.byref(mean), ctypes.byref(best),
                                                    ctypes.byref(worst)))
        return mean.value, best.value, worst.value

    def probe_hbm(self, nbytes=1 << 30):
        """What plain streams over device memory sustain with nothing else running: (read, write, copy) GB/s over
        two buffers of ``nbytes`` each; copy counts bytes read plus bytes written."""
        r, w, c = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
        self._check(self._probe_lib().eddlhip_probe_hbm(self.dev, int(nbytes), ctypes.byref(r), ctypes.byref(w), ctypes.byref(c)))
        return r.value, w.value, c.value

    def empty(self, shape):
        return DeviceTensor(self, shape)

    def array(self, host):
        host = np.ascontiguousarray(host, dtype=np.float32)
        return DeviceTensor(self, host.shape).copy_from(host)

    def full(self, shape, v):
        t = DeviceTensor(self, shape)
        self.fill_(t, v)
        return t

    def set_conv_algo(self, algo):
        self._check(self.lib.eddlhip_conv2d_set_algo({"auto": 0, "mfma": 1, "direct": 2, "mfma_staged": 3, "mfma_lds": 4, "ksplit_off": 5, "ksplit_on": 6, "winograd": 7, "winograd_off": 8, "winograd_never": 9}.get(algo, algo)))

    def force_conv_plan(self, tile=-1, slices=1):
        """Override the convolution launch planner (tile 0..3, K slices; tile 4 .. 7: the Winograd forms where they apply;
        8 / 9: the upsampled-input form of a 2x2 filter); tile -1 restores it."""
        self._check(self.lib.eddlhip_conv2d_force_plan(tile, slices))

    def last_conv_kernel(self):
        return self.lib.eddlhip_conv2d_last_kernel().decode()

    def conv_profile(self, collect):
        """Start (True) or stop (False) bracketing every convolution-kernel launch with events."""
        self._check(self.lib.eddlhip_conv2d_profile(int(bool(collect))))

    def conv_profile_read(self):
        """(launches, total milliseconds) of the convolution-kernel launches since collection started."""
        n, ms = ctypes.c_int(), ctypes.c_float()
        self._check(self.lib.eddlhip_conv2d_profile_read(ctypes.byref(n), ctypes.byref(ms)))
        return n.value, ms.value

    def conv_autotune(self, on=True):
        """Search the launch plans on the first call of every new convolution geometry (True), stop using what was found
        (False), or also forget it (-1)."""
        self._check(self.lib.eddlhip_conv2d_autotune(int(on)))

    def conv_tuned_plans(self):
        return self.lib.eddlhip_conv2d_tuned_plans(self.dev)

    def conv_tuned_save(self, path):
        """Write the plans found so far to a text file."""
        self._check(self.lib.eddlhip_conv2d_tuned_save(self.dev, str(path).encode()))

    def conv_tuned_load(self, path):
        """Merge a file written by ``conv_tuned_save`` into the table (used while the plan search is on)."""
        self._check(self.lib.eddlhip_conv2d_tuned_load(self.dev, str(path).encode()))

    def conv_trace(self, workgroups):
        """Per-workgroup timeline records of the next convolution launches (at most `workgroups` workgroups each);
        returns the device tensor that receives them (two floats hold one 64-bit word), or switches tracing off with 0."""
        if not workgroups:
            self._check(self.lib.eddlhip_conv2d_trace(None, 0))
            return None
        buf = self.full((int(workgroups) * 16,), 0.0)
        self._check(self.lib.eddlhip_conv2d_trace(buf.ptr, int(workgroups)))
        return buf

    # ---- operators (names follow the reference's gpu_* functions)
    def fill_(self, A, v):
        self._check(self.lib.eddlhip_fill(self.dev, A.ptr, A.size, v))

    # ---- parameter initialisation on the device (gpu_rand_*, gpu_mult / gpu_add with a scalar)
    def rand_uniform(self, A, v, seed):
        self._check(self.lib.eddlhip_rand_uniform(self.dev, A.ptr, A.size, v, seed))

    def rand_signed_uniform(self, A, v, seed):
        self._check(self.lib.eddlhip_rand_signed_uniform(self.dev, A.ptr, A.size, v, seed))

    def rand_binary(self, A, v, seed):
        self._check(self.lib.eddlhip_rand_binary(self.dev, A.ptr, A.size, v, seed))

    def rand_normal(self, A, mean, stddev, seed):
        self._check(self.lib.eddlhip_rand_normal(self.dev, A.ptr, A.size, mean, stddev, seed))

    def rand_words(self, n, seed, first_block=0, counter_hi=0):
        """The generator's raw 32-bit words as a numpy uint32 array (known-answer tests)."""
        t = self.empty((n,))
        self._check(self.lib.eddlhip_rand_words(self.dev, t.ptr, n, seed, first_block, counter_hi))
        return t.numpy().view(np.uint32)

    def mult_scalar(self, A, B, v):
        self._check(self.lib.eddlhip_mult_scalar(self.dev, A.ptr, B.ptr, A.size, v))

    def add_scalar(self, A, B, v):
        self._check(self.lib.eddlhip_add_scalar(self.dev, A.ptr, B.ptr, A.size, v))

    def conv2D(self, I, K, bias, O, sr, sc, padrt, padcl, bn=None, residual=None, relu=False, second=None, upsample=None, pool=None,
               keep=True):
        """``bn`` = (g, b, mean, var, eps) device tensors (g, b may be None) or None.  ``second``: the other half
        of the input channels as a tensor of its own (a channel Concat of ``I`` and ``second`` folded into the call).
        ``upsample`` = (rows, columns): whole factors of a nearest-neighbour UpSampling2D of ``I`` folded into the call
        (paddings and the output size then refer to the enlarged image).  ``pool`` = (pooled, indX, indY): the 2x2,
        stride-2 max-pool of the output in the same call (``eddlhip_conv2d_fwd_maxpool``); ``keep=False``: the
        unpooled output ``O`` is scratch space whose contents nobody reads afterwards."""
        N, C, H, W = I.shape
        Kf, C2, R, S = K.shape
        if second is not None:
            if tuple(second.shape) != tuple(I.shape):
                raise ValueError("the two input tensors differ in shape: %s, %s" % (I.shape, second.shape))
            C = 2 * C
        if C2 != C:
            raise ValueError("filter depth %d != input channels %d" % (C2, C))
        if O.shape[0] != N or O.shape[1] != Kf:
            raise ValueError("output shape %s does not match" % (O.shape,))
        g = b = mean = var = None
        eps = 0.0
        if bn is not None:
            g, b, mean, var, eps = bn
        tail = (K.ptr, _ptr(bias), O.ptr, N, C, H, W, Kf, R, S, sr, sc, padrt, padcl, O.shape[2], O.shape[3], _ptr(g), _ptr(b),
                _ptr(mean), _ptr(var), eps, _ptr(residual), int(relu))
        if second is not None and upsample is not None:
            raise ValueError("a two-tensor input and an upsampled input do not combine")
        if pool is not None:
            up = upsample if upsample is not None else (1, 1)
            PO, IX, IY = pool
            if tuple(PO.shape) != (N, Kf, O.shape[2] // 2, O.shape[3] // 2) or tuple(IX.shape) != tuple(PO.shape) or tuple(IY.shape) != tuple(PO.shape):
                raise ValueError("pooled shapes %s %s %s do not match output %s" % (PO.shape, IX.shape, IY.shape, O.shape))
            self._check(self.lib.eddlhip_conv2d_fwd_maxpool(self.dev, I.ptr, _ptr(second), int(up[0]), int(up[1]), *tail, PO.ptr, IX.ptr, IY.ptr,
                                                            int(bool(keep))))
        elif upsample is not None:
            self._check(self.lib.eddlhip_conv2d_fwd_upsampled(self.dev, I.ptr, int(upsample[0]), int(upsample[1]), *tail))
        elif second is None:
            self._check(self.lib.eddlhip_conv2d_fwd(self.dev, I.ptr, *tail))
        else:
            self._check(self.lib.eddlhip_conv2d_fwd_concat(self.dev, I.ptr, second.ptr, *tail))

    def cache_conv_filters(self, K):
        """Keep the kernels' repacked copy of filter tensor ``K`` (fixed between calls) in the library."""
        Kf, C, R, S = K.shape
        self._check(self.lib.eddlhip_conv2d_cache_filters(self.dev, K.ptr, Kf, C, R, S))

    def uncache_conv_filters(self, K=None):
        self._check(self.lib.eddlhip_conv2d_uncache_filters(self.dev, _ptr(K)))

    def batchnorm_inference(self, x, y, opa, gmean, gvar, g, b, variance, eps):
        N, C = x.shape[0], x.shape[1]
        rc = x.size // (N * C) if N * C else 1
        self._check(self.lib.eddlhip_batchnorm_inference(self.dev, N, C, rc, x.ptr, y.ptr, _ptr(opa), gmean.ptr, gvar.ptr, _ptr(g),
                                                         _ptr(b), variance.ptr, eps))

    def relu(self, A, B):
        self._check(self.lib.eddlhip_relu(self.dev, A.ptr, B.ptr, A.size))

    def sigmoid(self, A, B):
        self._check(self.lib.eddlhip_sigmoid(self.dev, A.ptr, B.ptr, A.size))

    def full_softmax(self, A, B, axis, stable=True):
        outer = int(np.prod(A.shape[:axis])) if axis > 0 else 1
        inner = int(np.prod(A.shape[axis + 1:])) if axis + 1 < len(A.shape) else 1
        self._check(self.lib.eddlhip_softmax(self.dev, A.ptr, B.ptr, outer, A.shape[axis], inner, int(stable)))

    def pool_out_dims(self, H, W, k, stride, pads):
        lp, lq = ctypes.c_int(), ctypes.c_int()
        self._check(self.lib.eddlhip_pool2d_out_dims(H, W, k[0], k[1], stride[0], stride[1], *pads, ctypes.byref(lp), ctypes.byref(lq)))
        return lp.value, lq.value

    def mpool2D(self, I, O, indX, indY, k, stride, pads):
        N, C, H, W = I.shape
        self._check(self.lib.eddlhip_maxpool2d(self.dev, I.ptr, O.ptr, indX.ptr, indY.ptr, N, C, H, W, k[0], k[1], stride[0],
                                               stride[1], *pads))

    def avgpool2D(self, I, O, k, stride, pads):
        N, C, H, W = I.shape
        self._check(self.lib.eddlhip_avgpool2d(self.dev, I.ptr, O.ptr, N, C, H, W, k[0], k[1], stride[0], stride[1], *pads))

    def scale(self, A, B, new_shape):
        N, C, H, W = A.shape
        self._check(self.lib.eddlhip_scale_nearest(self.dev, A.ptr, B.ptr, N, C, H, W, B.shape[2], B.shape[3], new_shape[0],
                                                   new_shape[1]))

    def concat(self, out, ts, axis):
        outer = int(np.prod(out.shape[:axis])) if axis > 0 else 1
        inner = int(np.prod(out.shape[axis + 1:])) if axis + 1 < len(out.shape) else 1
        ptrs = (ctypes.c_void_p * len(ts))(*[t.ptr for t in ts])
        ext = (ctypes.c_int * len(ts))(*[t.shape[axis] for t in ts])
        if sum(t.shape[axis] for t in ts) != out.shape[axis]:
            raise ValueError("The dimension of the output tensor is incorrect")
        self._check(self.lib.eddlhip_concat(self.dev, out.ptr, ptrs, ext, len(ts), outer, inner))

    def add(self, scA, A, scB, B, C, incC=0):
        self._check(self.lib.eddlhip_add(self.dev, scA, A.ptr, scB, B.ptr, C.ptr, incC, A.size))

    def inc(self, A, B):
        self._check(self.lib.eddlhip_inc(self.dev, A.ptr, B.ptr, A.size))

    def pad(self, A, B, pads):
        N, C, H, W = A.shape
        self._check(self.lib.eddlhip_pad(self.dev, A.ptr, B.ptr, N, C, H, W, *pads))

    def mult2D(self, A, B, C, incC=0):
        m, k = A.shape
        k2, n = B.shape
        if k != k2 or C.shape != (m, n):
            raise ValueError("mult2D shapes %s x %s -> %s" % (A.shape, B.shape, C.shape))
        self._check(self.lib.eddlhip_mult2d(self.dev, A.ptr, B.ptr, C.ptr, m, k, n, incC))

    def dense(self, A, W, bias, C, relu=False):
        """C = A W (+ bias per column) (then ReLU): LDense::forward (+ a following ReLU) in one call."""
        m, k = A.shape
        k2, n = W.shape
        if k != k2 or C.shape != (m, n):
            raise ValueError("dense shapes %s x %s -> %s" % (A.shape, W.shape, C.shape))
        self._check(self.lib.eddlhip_dense_fwd(self.dev, A.ptr, W.ptr, _ptr(bias), C.ptr, m, k, n, int(relu)))

    def sum2D_rowwise(self, A, B, C):
        self._check(self.lib.eddlhip_sum2d_rowwise(self.dev, A.ptr, B.ptr, C.ptr, A.shape[0], A.shape[1]))
