"""eddlhip_conv2d_fwd_noalloc, the convolution entry point that allocates nothing, against
eddlhip_conv2d_fwd on the same inputs: same kernels, same launch plan, so the outputs are compared
bit for bit.  Every case makes two calls in a row, the second on a smaller input, because every call on
a device shares that device's one scratch array, which keeps the previous call's contents.

Called through the C ABI (ctypes), device memory from eddlhip_malloc.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 64 << 20  # EDDLHIP_CONV_NOALLOC_SCRATCH_BYTES of include/eddlhip.h


def _out_dim(size, k, stride, pad_lo, pad_hi):
    return (size + pad_lo + pad_hi - k) // stride + 1


def _both(hip, rng, N, C, H, W, Kf, R, S, stride, pad, epilogue):
    """Runs eddlhip_conv2d_fwd and eddlhip_conv2d_fwd_noalloc on one seeded case; returns both outputs and
    the kernel each call reported."""
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
    P, Q = _out_dim(H, R, stride, pad, pad), _out_dim(W, S, stride, pad, pad)
    dx, dw = hip.array(x), hip.array(w)
    bias = g = b = mean = var = res = None
    if epilogue:
        bias = hip.array(rng.standard_normal(Kf).astype(np.float32))
        g = hip.array(rng.uniform(0.8, 1.2, Kf).astype(np.float32))
        b = hip.array((rng.standard_normal(Kf) * 0.1).astype(np.float32))
        mean = hip.array((rng.standard_normal(Kf) * 0.1).astype(np.float32))
        var = hip.array(rng.uniform(0.5, 1.5, Kf).astype(np.float32))
        res = hip.array(rng.standard_normal((N, Kf, P, Q), dtype=np.float32))
    ptr = lambda t: None if t is None else t.ptr
    outs, kernels = [], []
    for fn in (hip.lib.eddlhip_conv2d_fwd, hip.lib.eddlhip_conv2d_fwd_noalloc):
        O = hip.full((N, Kf, P, Q), float("nan"))
        hip._check(fn(hip.dev, dx.ptr, dw.ptr, ptr(bias), O.ptr, N, C, H, W, Kf, R, S, stride, stride, pad, pad, P, Q,
                      ptr(g), ptr(b), ptr(mean), ptr(var), 1e-5, ptr(res), int(epilogue)))
        kernels.append(hip.last_conv_kernel())
        outs.append(O.numpy())
    return outs, kernels


# (first call, second smaller call): N, C, H, W, Kf, R, S, stride, pad
CASES = {
    # 3x3, 128x128 tiles; 28x28x512 at batch 32 leaves tiles over that are divided along K: repacked filters + partial tiles
    "3x3_ksplit": ((32, 256, 28, 28, 512, 3, 3, 1, 1), (3, 64, 14, 14, 96, 3, 3, 1, 1)),
    # 7x7 stride 2 (the 16-tap kernel): repacked filters + tap table; then a 5x5
    "7x7_taptable": ((8, 3, 112, 112, 64, 7, 7, 2, 3), (2, 5, 30, 30, 40, 5, 5, 1, 2)),
    # 1x1 short K with the whole fused tail, then a 2x2
    "1x1_epilogue": ((16, 64, 56, 56, 256, 1, 1, 1, 0), (4, 32, 17, 17, 48, 2, 2, 1, 0)),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_noalloc_equals_conv2d_fwd_two_calls_in_a_row(hip, name):
    rng = np.random.default_rng(71)
    saw_split = False
    for shape in CASES[name]:
        N, C, H, W, Kf, R, S, stride, pad = shape
        (ref, got), (k_ref, k_got) = _both(hip, rng, N, C, H, W, Kf, R, S, stride, pad, epilogue=(name == "1x1_epilogue"))
        assert k_ref == k_got, "the two entry points planned different launches: %s vs %s" % (k_ref, k_got)
        assert np.all(np.isfinite(got)), "%s %s: the output holds values that were never written" % (name, shape)
        assert np.array_equal(ref, got), "%s %s (%s): %d values differ" % (name, shape, k_got, int((ref != got).sum()))
        saw_split = saw_split or "+ksplit" in k_got
    if name == "3x3_ksplit":
        assert saw_split, "this case is meant to cover the partial tiles of a K-split launch"


def test_noalloc_leaves_the_workspace_alone(hip):
    """The property the entry point exists for: with the library's workspace released beforehand, a call larger than any
    before it (repacked filters and the partial tiles of a K-split launch come from the fixed array) leaves the workspace
    at zero bytes - nothing was allocated - and the allocating entry point, called afterwards, gives the same bits."""
    rng = np.random.default_rng(73)
    N, C, H, W, Kf = 32, 320, 28, 28, 512
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, 3, 3)) * 0.03).astype(np.float32)
    dx, dw = hip.array(x), hip.array(w)
    O1, O2 = hip.full((N, Kf, H, W), float("nan")), hip.full((N, Kf, H, W), float("nan"))
    hip.synchronize()
    hip.workspace_trim()
    assert hip.workspace_bytes() == 0
    args = lambda O: (hip.dev, dx.ptr, dw.ptr, None, O.ptr, N, C, H, W, Kf, 3, 3, 1, 1, 1, 1, H, W, None, None, None, None, 0.0, None, 0)
    hip._check(hip.lib.eddlhip_conv2d_fwd_noalloc(*args(O1)))
    kernel = hip.last_conv_kernel()
    assert hip.workspace_bytes() == 0, "eddlhip_conv2d_fwd_noalloc took a workspace"
    assert "+ksplit" in kernel, kernel
    hip._check(hip.lib.eddlhip_conv2d_fwd(*args(O2)))
    assert hip.last_conv_kernel() == kernel and hip.workspace_bytes() > 0
    assert np.array_equal(O1.numpy(), O2.numpy())


def test_noalloc_uses_registered_filters(hip):
    """With the filters registered the call needs no room for a repacked copy; the result is unchanged."""
    rng = np.random.default_rng(72)
    N, C, H, W, Kf = 4, 64, 28, 28, 128
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, 3, 3)) * 0.05).astype(np.float32)
    dx, dw = hip.array(x), hip.array(w)
    outs = []
    for cached in (False, True):
        if cached:
            hip.cache_conv_filters(dw)
        O = hip.full((N, Kf, H, W), float("nan"))
        hip._check(hip.lib.eddlhip_conv2d_fwd_noalloc(hip.dev, dx.ptr, dw.ptr, None, O.ptr, N, C, H, W, Kf, 3, 3, 1, 1, 1, 1, H, W,
                                                      None, None, None, None, 0.0, None, 0))
        outs.append(O.numpy())
    hip.uncache_conv_filters(dw)
    assert np.array_equal(outs[0], outs[1])


def test_noalloc_refuses_what_does_not_fit(hip):
    """A filter tensor whose repacked copy is larger than the scratch array: EDDLHIP_EINVAL with the figures, nothing
    launched, nothing written; the allocating entry point takes the same call."""
    Kf, C = 2048, 1024  # 3x3: 9216 taps x 2048 channels x 4 bytes = 75 MB
    assert 9 * C * Kf * 4 > SCRATCH_BYTES
    N, H, W = 1, 8, 8
    dx, dw = hip.full((N, C, H, W), 1.0), hip.full((Kf, C, 3, 3), 0.5)
    O = hip.full((N, Kf, H, W), -7.0)
    args = (hip.dev, dx.ptr, dw.ptr, None, O.ptr, N, C, H, W, Kf, 3, 3, 1, 1, 1, 1, H, W, None, None, None, None, 0.0, None, 0)
    rc = hip.lib.eddlhip_conv2d_fwd_noalloc(*args)
    assert rc == -1
    text = hip.lib.eddlhip_last_error().decode()
    assert "scratch" in text and str(SCRATCH_BYTES) in text, text
    hip.synchronize()
    assert np.all(O.numpy() == -7.0)
    hip._check(hip.lib.eddlhip_conv2d_fwd(*args))
    out = O.numpy()
    assert out[0, 0, 4, 4] == np.float32(9 * C * 0.5) and out[0, 0, 0, 0] == np.float32(4 * C * 0.5)


def test_noalloc_refused_while_profiling(hip):
    dx, dw, O = hip.full((1, 8, 8, 8), 1.0), hip.full((8, 8, 3, 3), 1.0), hip.empty((1, 8, 8, 8))
    hip.conv_profile(True)
    try:
        rc = hip.lib.eddlhip_conv2d_fwd_noalloc(hip.dev, dx.ptr, dw.ptr, None, O.ptr, 1, 8, 8, 8, 8, 3, 3, 1, 1, 1, 1, 8, 8,
                                                None, None, None, None, 0.0, None, 0)
    finally:
        hip.conv_profile(False)
    assert rc == -1 and "profile" in hip.lib.eddlhip_last_error().decode()
