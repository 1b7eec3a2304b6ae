"""CPU-side checks of the C ABI and of the host-side descriptor mirrors (no GPU needed)."""
import ctypes
import os
import re

import numpy as np
import pytest

from conftest import ROOT


def _declared_functions(header="eddlhip.h"):
    src = open(os.path.join(ROOT, "include", header)).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(eddlhip_\w+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    from eddl_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_functions()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "libeddlhip.so lacks %s" % n
    assert set(names) == set(_lib.PROTOTYPES), "ctypes prototypes out of step with include/eddlhip.h"
    # the benchmark's device probes: a library and a header of their own, outside the drop-in boundary
    probe = _lib.load_probe()
    probes = _declared_functions("eddlhip_probe.h")
    assert probes == sorted(_lib.PROBE_PROTOTYPES) and all(hasattr(probe, n) for n in probes)
    assert not any(hasattr(lib, n) for n in probes), "the probes are meant to stay out of libeddlhip.so"


def test_version_and_argument_errors_without_a_device():
    from eddl_amd import _lib
    lib = _lib.load()
    assert b"gfx950" in lib.eddlhip_version()
    assert lib.eddlhip_conv2d_set_algo(10) == -1
    assert b"unknown algorithm" in lib.eddlhip_last_error()
    assert lib.eddlhip_conv2d_set_algo(0) == 0
    lp, lq = ctypes.c_int(), ctypes.c_int()
    assert lib.eddlhip_pool2d_out_dims(5, 5, 3, 3, 2, 2, 0, 1, 0, 1, ctypes.byref(lp), ctypes.byref(lq)) == 0
    assert (lp.value, lq.value) == (2, 2)
    assert lib.eddlhip_pool2d_out_dims(5, 5, 0, 3, 2, 2, 0, 1, 0, 1, ctypes.byref(lp), ctypes.byref(lq)) == -1


def test_tuned_plan_table_round_trips_through_a_file(tmp_path):
    """eddlhip_conv2d_tuned_save / _load need no device: a file of plans is merged into the table and written back."""
    from eddl_amd import _lib
    lib = _lib.load()
    lib.eddlhip_conv2d_autotune(-1)
    assert lib.eddlhip_conv2d_tuned_plans(0) == 0
    src = tmp_path / "plans.txt"
    src.write_text("# comment\n"
                   "64 64 64 3 3 1 1 56 56 1 | 2 4\n"
                   "32 512 512 3 3 1 1 28 28 1 | -1 1\n")
    assert lib.eddlhip_conv2d_tuned_load(0, str(src).encode()) == 0
    assert lib.eddlhip_conv2d_tuned_plans(0) == 2
    assert lib.eddlhip_conv2d_tuned_load(0, str(src).encode()) == 0     # known geometries are replaced, not repeated
    assert lib.eddlhip_conv2d_tuned_plans(0) == 2
    dst = tmp_path / "out.txt"
    assert lib.eddlhip_conv2d_tuned_save(0, str(dst).encode()) == 0
    body = [l for l in dst.read_text().splitlines() if not l.startswith("#")]
    assert body == ["64 64 64 3 3 1 1 56 56 1 | 2 4", "32 512 512 3 3 1 1 28 28 1 | -1 1"]
    bad = tmp_path / "bad.txt"
    bad.write_text("64 64 56 56 | 9 9\n")
    assert lib.eddlhip_conv2d_tuned_load(0, str(bad).encode()) < 0
    assert b"not a plan" in lib.eddlhip_last_error()
    assert lib.eddlhip_conv2d_tuned_load(0, str(tmp_path / "missing.txt").encode()) < 0
    assert lib.eddlhip_conv2d_tuned_plans(0) == 2
    # every plan number the library knows is accepted - 0..3 direct tiles, 4 / 5 / 6 / 7 the Winograd forms, 8 / 9 the
    # upsampled-input form of a 2x2 filter, whose geometries carry kind 2 / 3 - and the first unknown one is refused
    forms = tmp_path / "forms.txt"
    forms.write_text("".join("4 %d 64 2 2 1 1 128 128 3 | %d 1\n" % (128 + t, t) for t in range(0, 10)))
    assert lib.eddlhip_conv2d_tuned_load(0, str(forms).encode()) == 0
    assert lib.eddlhip_conv2d_tuned_plans(0) == 12
    bad.write_text("4 128 64 2 2 1 1 128 128 3 | 10 1\n")
    assert lib.eddlhip_conv2d_tuned_load(0, str(bad).encode()) < 0
    bad.write_text("4 128 64 2 2 1 1 128 128 3 | 8 17\n")      # (no search tries more than 16 slices)
    assert lib.eddlhip_conv2d_tuned_load(0, str(bad).encode()) < 0
    assert lib.eddlhip_conv2d_tuned_plans(0) == 12
    lib.eddlhip_conv2d_autotune(-1)
    assert lib.eddlhip_conv2d_tuned_plans(0) == 0


def test_committed_plans_files_load():
    """The plans files the profiled commands name (profiles/plans_<workload>.txt) are in the loader's format, and what the
    loader keeps of each is what the file says, line for line."""
    import glob
    import tempfile
    from eddl_amd import _lib
    lib = _lib.load()
    files = sorted(glob.glob(os.path.join(ROOT, "profiles", "plans_*.txt")))
    assert len(files) >= 4, files
    for path in files:
        lib.eddlhip_conv2d_autotune(-1)
        assert lib.eddlhip_conv2d_tuned_load(0, path.encode()) == 0, (path, lib.eddlhip_last_error())
        want = sorted(l.strip() for l in open(path).read().splitlines() if l.strip() and not l.startswith("#"))
        assert lib.eddlhip_conv2d_tuned_plans(0) == len(want) > 0, path
        with tempfile.TemporaryDirectory() as tmp:
            out = os.path.join(tmp, "saved.txt")
            assert lib.eddlhip_conv2d_tuned_save(0, out.encode()) == 0
            got = sorted(l.strip() for l in open(out).read().splitlines() if l.strip() and not l.startswith("#"))
        assert got == want, path
    lib.eddlhip_conv2d_autotune(-1)


def test_descriptor_mirrors_match_the_oracle_geometry(oracle, golden):
    from eddl_amd.descriptors import ConvolDescriptor, PoolDescriptor
    t = golden["output_sizes"]
    i = 0
    for p in t["padding"]:
        for isz in t["input_sizes"]:
            for s in t["strides"]:
                for k in t["kernels"]:
                    assert ConvolDescriptor.compute_output(p, isz, k, s) == t["output_sizes"][i]
                    i += 1
    rng = np.random.default_rng(3)
    for _ in range(300):
        H, W = int(rng.integers(1, 70)), int(rng.integers(1, 70))
        kr, kc = int(rng.integers(1, 8)), int(rng.integers(1, 8))
        sr, sc = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        for padding in ("same", "valid"):
            try:
                cd = ConvolDescriptor(4, [kr, kc], [sr, sc], padding).build([2, 3, H, W])
                got = (cd.r, cd.c, tuple(cd.pads))
            except RuntimeError:
                got = None
            P, Q, pads = oracle.conv_geometry(H, W, kr, kc, sr, sc, padding)
            exp = (P, Q, pads) if P > 0 and Q > 0 else None
            assert got == exp
            try:
                pd = PoolDescriptor([kr, kc], [sr, sc], padding).build([2, 3, H, W])
                got = (pd.r, pd.c, tuple(pd.pad), pd.loop_rows, pd.loop_cols)
            except RuntimeError:
                got = None
            r, c, p4, lp, lq = oracle.pool_geometry(H, W, kr, kc, sr, sc, padding)
            assert got == ((r, c, p4, lp, lq) if r > 0 and c > 0 else None)
        pads = [int(v) for v in rng.integers(0, 4, 4)]
        P, Q, _ = oracle.conv_geometry(H, W, kr, kc, sr, sc, "custom", pads)
        if P > 0 and Q > 0:
            cd = ConvolDescriptor(4, [kr, kc], [sr, sc], "custom", pads).build([2, 3, H, W])
            assert (cd.r, cd.c) == (P, Q)


def test_descriptor_errors_follow_the_reference():
    from eddl_amd.descriptors import ConvolDescriptor, PoolDescriptor
    with pytest.raises(RuntimeError, match="ConvolDescriptor::ConvolDescriptor"):
        ConvolDescriptor(4, [3, 3], [1, 1], "bogus")
    with pytest.raises(RuntimeError, match="Grouped"):
        ConvolDescriptor(4, [3, 3], [1, 1], "same", groups=2)
    with pytest.raises(RuntimeError, match="ConvolDescriptor::build"):
        ConvolDescriptor(4, [3, 3], [1, 1], "same").build([1, 3, 8])
    with pytest.raises(RuntimeError, match="Invalid output shape"):
        ConvolDescriptor(4, [5, 5], [1, 1], "valid").build([1, 3, 4, 4])
    with pytest.raises(RuntimeError, match="PoolDescriptor::PoolDescriptor"):
        PoolDescriptor([2, 2], [2, 2], "bogus")


def test_host_layer_links_against_the_c_abi():
    """The C++ host layer builds with g++ alone and resolves every symbol against libeddlhip.so."""
    import subprocess
    host = os.path.join(ROOT, "eddl_amd", "host")
    lib = os.path.join(host, "libeddlhip_host.so")
    if not os.path.exists(lib):
        subprocess.run(["make", "-C", host, "all"], check=True, stdout=subprocess.DEVNULL)
    h = ctypes.CDLL(lib)
    for sym in ("_ZN8eddl_hip10gpu_conv2DEPNS_16ConvolDescriptorE", "_ZN8eddl_hip8tensorNN6Conv2DEPNS_16ConvolDescriptorE",
                "_ZN8eddl_hip11gpu_mpool2DEPNS_14PoolDescriptorE", "_ZN8eddl_hip8gpu_reluEPNS_6TensorES1_",
                # the model-building API: eddl::Model, eddl::Conv2D, eddl::predict, Net::load
                "_ZN8eddl_hip4eddl5ModelESt6vectorIPNS_5LayerESaIS3_EES5_",
                "_ZN8eddl_hip4eddl6Conv2DEPNS_5LayerEiRKSt6vectorIiSaIiEES7_NSt7__cxx1112basic_stringIcSt11char_traitsIcESaIcEEEbiS7_SD_",
                "_ZN8eddl_hip4eddl7predictEPNS_3NetERKSt6vectorIPNS_6TensorESaIS5_EE",
                "_ZN8eddl_hip3Net4loadERKNSt7__cxx1112basic_stringIcSt11char_traitsIcESaIcEEES8_",
                # this backend's additions: the fused plan and the asynchronous mode of the wrappers
                "_ZN8eddl_hip4eddl4fuseEPNS_3NetE", "_ZN8eddl_hip3Net4fuseEv", "_ZN8eddl_hip19gpu_set_synchronousEb",
                # ONNX: import_net_from_onnx_file / _pointer, save_net_to_onnx_file
                "_ZN8eddl_hip25import_net_from_onnx_fileERKNSt7__cxx1112basic_stringIcSt11char_traitsIcESaIcEEERKSt6vectorIiSaIiEEi",
                "_ZN8eddl_hip28import_net_from_onnx_pointerEPKvmi",
                "_ZN8eddl_hip21save_net_to_onnx_fileEPNS_3NetERKNSt7__cxx1112basic_stringIcSt11char_traitsIcESaIcEEE"):
        assert hasattr(h, sym), sym
