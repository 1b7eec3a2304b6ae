"""ctypes binding of the CPU oracle (oracle/eddl_cpu_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``; the shipped package never imports it.

All arrays are C-contiguous float32 numpy arrays in the reference's layouts (NCHW
activations, OIHW filters, [in, out] dense weights).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_f = ctypes.POINTER(ctypes.c_float)
_i = ctypes.c_int
_sz = ctypes.c_size_t


def build():
    """Compile both oracle libraries (strict and HPC flags) next to the source."""
    subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, stdout=subprocess.DEVNULL)


def _host_has(flags):
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.startswith("flags"):
                    have = set(line.split(":", 1)[1].split())
                    return all(f in have for f in flags)
    except OSError:
        pass
    return False


class Oracle:
    """One loaded oracle library.  ``hpc=True`` loads the -ffast-math build (timing only)."""

    def __init__(self, hpc=False):
        name = "libeddl_oracle_hpc.so" if hpc else "libeddl_oracle.so"
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        if hpc and not _host_has(["avx2", "fma", "bmi2"]):
            raise RuntimeError("host CPU lacks AVX2/FMA needed by the HPC oracle build")
        self.hpc = hpc
        self.lib = L = ctypes.CDLL(path)
        L.eddl_oracle_num_threads.restype = _i
        L.eddl_oracle_set_num_threads.argtypes = [_i]
        L.eddl_oracle_out_size_named.argtypes = [_i] * 5
        L.eddl_oracle_out_size_custom.argtypes = [_i] * 6
        L.eddl_oracle_same_pads.argtypes = [_i] * 5 + [ctypes.POINTER(_i)] * 2
        L.eddl_oracle_pool_loop_count.argtypes = [_i] * 5
        L.eddl_oracle_conv2d_direct.argtypes = [_f, _f, _f, _f] + [_i] * 13
        L.eddl_oracle_conv2d_direct_at.argtypes = [_f, _f, _f, _f, ctypes.POINTER(_i)] + [_i] * 12
        L.eddl_oracle_conv2d_im2col.argtypes = [_f, _f, _f, _f] + [_i] * 13
        L.eddl_oracle_conv2d_im2col.restype = _i
        L.eddl_oracle_batchnorm_inference.argtypes = [_i, _i, _i, _f, _f, _f, _f, _f, _f, _f, _f, ctypes.c_float]
        L.eddl_oracle_relu.argtypes = [_f, _f, _sz]
        L.eddl_oracle_sigmoid.argtypes = [_f, _f, _sz]
        L.eddl_oracle_softmax.argtypes = [_f, _f, _i, _i, _i, _i]
        L.eddl_oracle_maxpool2d.argtypes = [_f, _f, _f, _f] + [_i] * 12
        L.eddl_oracle_avgpool2d.argtypes = [_f, _f] + [_i] * 12
        L.eddl_oracle_scale_nearest.argtypes = [_f, _f] + [_i] * 8
        L.eddl_oracle_scale_nearest.restype = _i
        L.eddl_oracle_concat.argtypes = [_f, ctypes.POINTER(_f), ctypes.POINTER(_i), _i, _i, _i]
        L.eddl_oracle_add.argtypes = [ctypes.c_float, _f, ctypes.c_float, _f, _f, _i, _sz]
        L.eddl_oracle_pad.argtypes = [_f, _f] + [_i] * 8
        L.eddl_oracle_mult2d.argtypes = [_f, _f, _f, _i, _i, _i]
        L.eddl_oracle_sum2d_rowwise.argtypes = [_f, _f, _f, _i, _i]

    # ---- helpers
    @staticmethod
    def _p(a):
        if a is None:
            return None
        assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], "oracle takes contiguous float32"
        return a.ctypes.data_as(_f)

    @property
    def num_threads(self):
        return self.lib.eddl_oracle_num_threads()

    def set_num_threads(self, n):
        self.lib.eddl_oracle_set_num_threads(int(n))

    def set_inner_parallel(self, on):
        """Let the threads that a small batch leaves idle share each image's lowering and product in the im2col
        convolution (for checking runs; results are unchanged, the reference's one-thread-per-image timing is not)."""
        self.lib.eddl_oracle_set_inner_parallel(int(bool(on)))

    # ---- geometry (descriptor_conv2D.cpp / descriptor_pool2D.cpp)
    def out_size(self, padding, in_size, k, stride, dilation=1):
        """``padding`` is "same"/"zeros", "valid"/"none", or a (lo, hi) pair for custom pads."""
        if isinstance(padding, str):
            same = {"same": 1, "zeros": 1, "valid": 0, "none": 0}[padding]
            return self.lib.eddl_oracle_out_size_named(same, in_size, k, stride, dilation)
        return self.lib.eddl_oracle_out_size_custom(padding[0], padding[1], in_size, k, stride, dilation)

    def same_pads(self, out_size, in_size, k, stride, dilation=1):
        lo, hi = _i(), _i()
        self.lib.eddl_oracle_same_pads(out_size, in_size, k, stride, dilation, ctypes.byref(lo), ctypes.byref(hi))
        return lo.value, hi.value

    def conv_geometry(self, H, W, R, S, sr, sc, padding, pads=None, dilation=(1, 1)):
        """Mirror of ConvolDescriptor::build: returns (P, Q, (top, bottom, left, right))."""
        if padding == "custom":
            P = self.out_size((pads[0], pads[1]), H, R, sr, dilation[0])
            Q = self.out_size((pads[2], pads[3]), W, S, sc, dilation[1])
            return P, Q, tuple(pads)
        P = self.out_size(padding, H, R, sr, dilation[0])
        Q = self.out_size(padding, W, S, sc, dilation[1])
        if padding in ("same", "zeros"):
            pr = self.same_pads(P, H, R, sr, dilation[0])
            pc = self.same_pads(Q, W, S, sc, dilation[1])
        else:
            pr = pc = (0, 0)
        return P, Q, (pr[0], pr[1], pc[0], pc[1])

    def pool_geometry(self, H, W, kr, kc, sr, sc, padding, pads=None):
        """Mirror of PoolDescriptor::build: returns (r, c, pads4, loopP, loopQ).  With custom
        pads the column count is computed from the ROW pads, as descriptor_pool2D.cpp:69-70
        passes the whole 4-vector and only its first two entries are read."""
        if padding == "custom":
            r = self.out_size((pads[0], pads[1]), H, kr, sr)
            c = self.out_size((pads[0], pads[1]), W, kc, sc)
            p4 = tuple(pads)
        else:
            r = self.out_size(padding, H, kr, sr)
            c = self.out_size(padding, W, kc, sc)
            if padding in ("same", "zeros"):
                pr = self.same_pads(r, H, kr, sr)
                pc = self.same_pads(c, W, kc, sc)
            else:
                pr = pc = (0, 0)
            p4 = (pr[0], pr[1], pc[0], pc[1])
        lp = self.lib.eddl_oracle_pool_loop_count(H, kr, sr, p4[0], p4[1])
        lq = self.lib.eddl_oracle_pool_loop_count(W, kc, sc, p4[2], p4[3])
        return r, c, p4, lp, lq

    # ---- operators
    def conv2d(self, x, w, bias, stride, pt, pl, P, Q, algo="direct"):
        N, C, H, W = x.shape
        Kf, C2, R, S = w.shape
        assert C2 == C
        out = np.empty((N, Kf, P, Q), np.float32)
        args = (self._p(x), self._p(w), self._p(bias), self._p(out), N, C, H, W, Kf, R, S, stride[0], stride[1], pt, pl, P, Q)
        if algo == "direct":
            self.lib.eddl_oracle_conv2d_direct(*args)
        else:
            if self.lib.eddl_oracle_conv2d_im2col(*args) != 0:
                raise MemoryError("oracle im2col scratch")
        return out

    def conv2d_at(self, x, w, bias, stride, pt, pl, idx):
        N, C, H, W = x.shape
        Kf, _, R, S = w.shape
        idx = np.ascontiguousarray(idx, dtype=np.int32)
        out = np.empty(len(idx), np.float32)
        self.lib.eddl_oracle_conv2d_direct_at(self._p(x), self._p(w), self._p(bias), self._p(out),
                                              idx.ctypes.data_as(ctypes.POINTER(_i)), len(idx), N, C, H, W, Kf, R, S,
                                              stride[0], stride[1], pt, pl)
        return out

    def batchnorm_inference(self, x, gmean, gvar, g, b, eps):
        """Returns (y, opa, sd).  ``g``/``b`` None means no affine (then opa is None)."""
        N, C = x.shape[0], x.shape[1]
        rc = int(np.prod(x.shape[2:])) if x.ndim > 2 else 1
        y = np.empty_like(x)
        opa = np.empty_like(x) if g is not None else None
        sd = np.empty(C, np.float32)
        self.lib.eddl_oracle_batchnorm_inference(N, C, rc, self._p(x), self._p(y), self._p(opa), self._p(gmean),
                                                 self._p(gvar), self._p(g), self._p(b), self._p(sd), eps)
        return y, opa, sd

    def relu(self, x):
        y = np.empty_like(x)
        self.lib.eddl_oracle_relu(self._p(x), self._p(y), x.size)
        return y

    def sigmoid(self, x):
        y = np.empty_like(x)
        self.lib.eddl_oracle_sigmoid(self._p(x), self._p(y), x.size)
        return y

    def softmax(self, x, axis, stable=True):
        y = np.empty_like(x)
        outer = int(np.prod(x.shape[:axis])) if axis > 0 else 1
        inner = int(np.prod(x.shape[axis + 1:])) if axis + 1 < x.ndim else 1
        self.lib.eddl_oracle_softmax(self._p(x), self._p(y), outer, x.shape[axis], inner, int(stable))
        return y

    def maxpool2d(self, x, k, stride, pads, fill=np.nan):
        """Returns (O, indX, indY), each flat per image in loop order reshaped to
        (N, C, loopP, loopQ).  Index slots the reference would leave untouched hold ``fill``."""
        N, C, H, W = x.shape
        lp = self.lib.eddl_oracle_pool_loop_count(H, k[0], stride[0], pads[0], pads[1])
        lq = self.lib.eddl_oracle_pool_loop_count(W, k[1], stride[1], pads[2], pads[3])
        O = np.empty((N, C, lp, lq), np.float32)
        ix = np.full((N, C, lp, lq), fill, np.float32)
        iy = np.full((N, C, lp, lq), fill, np.float32)
        self.lib.eddl_oracle_maxpool2d(self._p(x), self._p(O), self._p(ix), self._p(iy), N, C, H, W, k[0], k[1],
                                       stride[0], stride[1], *pads)
        return O, ix, iy

    def avgpool2d(self, x, k, stride, pads):
        N, C, H, W = x.shape
        lp = self.lib.eddl_oracle_pool_loop_count(H, k[0], stride[0], pads[0], pads[1])
        lq = self.lib.eddl_oracle_pool_loop_count(W, k[1], stride[1], pads[2], pads[3])
        O = np.empty((N, C, lp, lq), np.float32)
        self.lib.eddl_oracle_avgpool2d(self._p(x), self._p(O), N, C, H, W, k[0], k[1], stride[0], stride[1], *pads)
        return O

    def scale_nearest(self, x, out_hw, new_shape=None):
        N, C, H, W = x.shape
        new_shape = new_shape or out_hw
        y = np.zeros((N, C, out_hw[0], out_hw[1]), np.float32)
        bad = self.lib.eddl_oracle_scale_nearest(self._p(x), self._p(y), N, C, H, W, out_hw[0], out_hw[1],
                                                 new_shape[0], new_shape[1])
        if bad:
            raise ValueError("nearest wrapping: %d destination elements map outside the source" % bad)
        return y

    def concat(self, xs, axis):
        shape = list(xs[0].shape)
        shape[axis] = sum(a.shape[axis] for a in xs)
        out = np.empty(shape, np.float32)
        outer = int(np.prod(shape[:axis])) if axis > 0 else 1
        inner = int(np.prod(shape[axis + 1:])) if axis + 1 < len(shape) else 1
        ptrs = (_f * len(xs))(*[self._p(a) for a in xs])
        ext = (_i * len(xs))(*[a.shape[axis] for a in xs])
        self.lib.eddl_oracle_concat(self._p(out), ptrs, ext, len(xs), outer, inner)
        return out

    def add(self, a, b, scA=1.0, scB=1.0, c=None):
        inc = c is not None
        out = c.copy() if inc else np.empty_like(a)
        self.lib.eddl_oracle_add(scA, self._p(a), scB, self._p(b), self._p(out), int(inc), a.size)
        return out

    def pad(self, x, pads, cval=0.0):
        """pads = (top, right, bottom, left), the reference's order."""
        N, C, H, W = x.shape
        t, r, b, l = pads
        out = np.full((N, C, H + t + b, W + l + r), cval, np.float32)
        self.lib.eddl_oracle_pad(self._p(x), self._p(out), N, C, H, W, t, r, b, l)
        return out

    def dense(self, x, w, bias=None):
        m, k = x.shape
        k2, n = w.shape
        assert k == k2
        out = np.empty((m, n), np.float32)
        self.lib.eddl_oracle_mult2d(self._p(x), self._p(w), self._p(out), m, k, n)
        if bias is not None:
            self.lib.eddl_oracle_sum2d_rowwise(self._p(out), self._p(bias), self._p(out), m, n)
        return out
