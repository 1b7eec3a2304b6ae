"""The C++ host layer under AddressSanitizer and UndefinedBehaviorSanitizer (the reference's own sanitizer build:
CMakeLists.txt:89-95; here `make -C eddl_amd/host asan`, host code only, g++).

What runs in the instrumented executable, without a device: the geometry rules of ConvolDescriptor / PoolDescriptor
(the error cases of `net_driver errors`), the reader of the reference's `bin` parameter files (Net::load) and the ONNX
decoder (a wire-format parser for untrusted files) - each on the committed fixtures and on truncated and corrupted
copies of them.  A malformed file must end in an exception raised through msg() (exit code 1 of the driver) or be
accepted; it must never make a sanitizer speak (a read past a buffer, an overflow, an allocation of a size taken from
the file).
"""
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
HOST = os.path.join(os.path.dirname(HERE), "eddl_amd", "host")
DRIVER = os.path.join(HOST, "net_driver_asan")
ONNX_DIR = os.path.join(HERE, "golden", "onnx")


@pytest.fixture(scope="module")
def asan_driver():
    res = subprocess.run(["make", "-C", HOST, "asan"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-3000:]
    return DRIVER


def run(driver, args):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:allocator_may_return_null=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    res = subprocess.run([driver] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, errors="replace", timeout=120,
                         env=env)   # (a corrupted file's names come back as they are: not always valid text)
    spoke = [w for w in ("AddressSanitizer", "runtime error:", "UndefinedBehaviorSanitizer", "LeakSanitizer") if w in res.stderr]
    assert not spoke and res.returncode in (0, 1), "sanitizer report or crash (rc %d) for %s:\n%s" % (res.returncode, args, res.stderr[-3000:])
    return res


def test_geometry_rules_under_the_sanitizers(asan_driver):
    res = run(asan_driver, ["errors"])
    assert "ok asymmetric pads 0 1 0 1" in res.stdout, res.stdout


@pytest.mark.parametrize("name", ["vgg_like", "resnet_like", "unet_like"])
def test_onnx_decoder_under_the_sanitizers(asan_driver, name, tmp_path):
    """The PyTorch-exported fixture decodes cleanly; every truncation and a few hundred corruptions of it (single bytes
    replaced, runs of 0xff - the longest varints and lengths a field can claim -, zeroed runs) either decode or are refused."""
    data = open(os.path.join(ONNX_DIR, name + ".onnx"), "rb").read()
    good = run(asan_driver, ["onnxinfo", os.path.join(ONNX_DIR, name + ".onnx"), tmp_path / "back.onnx"])
    assert good.returncode == 0 and good.stdout.count("layer ") >= 5
    rng = np.random.default_rng(len(data))
    variants = [data[:n] for n in list(range(0, 48)) + [int(len(data) * f) for f in np.linspace(0.02, 0.999, 40)]]
    for _ in range(120):
        b = bytearray(data)
        # (most of a file is weights, whose bytes no parser looks at: two corruptions in three go to the structure in front)
        pos = int(rng.integers(0, min(len(b), 4096))) if rng.random() < 0.67 else int(rng.integers(0, len(b)))
        kind = rng.integers(0, 3)
        if kind == 0:
            b[pos] = int(rng.integers(0, 256))
        elif kind == 1:
            b[pos:pos + int(rng.integers(1, 11))] = b"\xff" * int(rng.integers(1, 11))
        else:
            b[pos:pos + 4] = b"\x00\x00\x00\x00"
        variants.append(bytes(b))
    refused = 0
    for i, v in enumerate(variants):
        path = tmp_path / "v.onnx"
        path.write_bytes(v)
        res = run(asan_driver, ["onnxinfo", path])
        refused += res.returncode == 1
        assert res.returncode == 0 or "exception:" in res.stderr, (i, res.stderr[-500:])
    assert refused >= 60          # the truncations at least


def test_bin_reader_under_the_sanitizers(asan_driver, tmp_path):
    """A parameter file written by the Python host loads with the right sums; cut short anywhere, or with a record header
    that claims another rank or shape (negative, zero, enormous, a product that wraps around), it is refused with the
    reference-style exception and nothing is allocated from the numbers in the file."""
    from eddl_amd import models
    m = models.vgg16(batch=1, size=32, num_classes=10, widths=(4, 8, 8, 8, 8), dense=16)
    models.init_he_normal(m, 9)
    good = tmp_path / "params.bin"
    m.save(str(good))
    args = ["vgg16", None, 32, 10, 4, 8, 8, 8, 8, 16]
    call = lambda path: run(asan_driver, ["loadbin", args[0], path] + args[2:])
    res = call(good)
    assert res.returncode == 0, res.stderr
    sums = [float(l.split()[3]) for l in res.stdout.splitlines() if l.startswith("param ")]
    want = [float(np.sum(v.astype(np.float64))) for l in m.layers for v in l.params.values()]
    assert len(sums) == len(want) and np.allclose(sums, want, rtol=1e-6, atol=1e-6)
    data = open(good, "rb").read()
    bad = tmp_path / "bad.bin"
    for n in list(range(0, 40)) + [int(len(data) * f) for f in np.linspace(0.05, 0.999, 25)]:
        bad.write_bytes(data[:n])
        res = call(bad)
        assert res.returncode == 1 and "exception:" in res.stderr, (n, res.stderr[-300:])
    first = np.frombuffer(data[:20], np.int32)           # ndim = 4, then the shape of the first convolution's filters
    assert first[0] == 4
    for header in ([-1], [0], [9], [2 ** 31 - 1], [4, -4, 3, 3, 3], [4, 0, 3, 3, 3], [4, 2 ** 30, 2 ** 30, 4, 4], [4, 65536, 65536, 1, 1],
                   [4, 2 ** 31 - 1, 1, 1, 1], [2, int(first[1]) * int(first[2]), 9], [4, int(first[1]), int(first[2]), 3, 4]):
        blob = np.array(header, np.int32).tobytes() + data[20:]          # the first record's own header is five words
        bad.write_bytes(blob)
        res = call(bad)
        same_size = int(np.prod(header[1:], dtype=np.int64)) == int(np.prod(first[1:5])) if len(header) > 1 else False
        # (another shape of the same size is accepted, as the reference's copy accepts it)
        assert res.returncode == (0 if same_size and len(header) - 1 == header[0] else 1), (header, res.returncode, res.stderr[-300:])
