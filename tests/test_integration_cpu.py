"""The files that go into EDDL itself (integration/eddl): the binding translation unit, the generated stubs, the patch.

With an EDDL tree at hand (/root/reference here; absent on the GPU box, where these tests skip) the three device-seam
headers are parsed and every declaration must be defined exactly once, by hip_backend.cpp or by hip_stubs.cpp; every
member the binding reads through a Tensor / ConvolDescriptor / PoolDescriptor pointer must exist in EDDL's classes; the
patch must apply to the tree.  Without the tree, what does not need it still runs: the stubs parse as C++, and the
binding defines what the backend's own host layer declares.
"""
import os
import re
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INTEG = os.path.join(ROOT, "integration", "eddl")
sys.path.insert(0, INTEG)
import gen_hip_stubs as gen  # noqa: E402

REFERENCE = "/root/reference"
needs_reference = pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "include", "eddl")), reason="no EDDL tree mounted")


def _binding_text():
    return gen.strip_comments(open(gen.BINDING, encoding="utf-8").read())


@needs_reference
def test_every_declaration_is_bound_or_stubbed_exactly_once():
    declared = {(n, t) for _, n, t in gen.declared(REFERENCE)}
    assert len(declared) > 200
    bound = [(n, t) for _, n, t in gen.bound()]
    stubs = [(n, t) for _, n, t in gen.bound(gen.STUBS)]
    assert len(set(bound)) == len(bound) and len(set(stubs)) == len(stubs), "a function is defined twice"
    assert not set(bound) & set(stubs), sorted(set(bound) & set(stubs))
    extras = {"gpu_check", "gpu_set_synchronous", "gpu_get_synchronous", "gpu_synchronize", "gpu_set_random_seed"}  # hip_backend.h
    assert {n for n, _ in set(bound) - declared} == extras
    missing = declared - set(bound) - set(stubs)
    assert not missing, "declared by EDDL's headers but defined nowhere: %s" % sorted(missing)
    assert not set(stubs) - declared, "stubs for functions EDDL does not declare: %s" % sorted(set(stubs) - declared)
    # the functions eddl::build / forward / predict reach on the path are bound, not stubbed
    on_path = ["gpu_init", "gpu_devices", "gpu_create_tensor", "gpu_delete_tensor", "gpu_copy_to_gpu", "gpu_copy_from_gpu", "gpu_copy_gpu",
               "gpu_fill_", "gpu_rand_uniform", "gpu_rand_signed_uniform", "gpu_rand_normal", "gpu_rand_binary", "gpu_mult", "gpu_conv2D",
               "gpu_batchnorm_forward", "gpu_relu", "gpu_sigmoid", "gpu_full_softmax", "gpu_mpool2D", "gpu_avgpool2D", "gpu_scale",
               "gpu_concat", "gpu_add", "gpu_inc", "gpu_pad", "gpu_mult2D", "gpu_sum2D_rowwise"]
    bound_names = {n for n, _ in bound}
    assert not [n for n in on_path if n not in bound_names]


@needs_reference
def test_stub_file_is_up_to_date():
    text, _ = gen.render(REFERENCE)
    assert open(gen.STUBS, encoding="utf-8").read() == text, "run integration/eddl/gen_hip_stubs.py"


def _class_body(text, name):
    m = re.search(r"\bclass\s+%s\s*\{" % name, text)
    assert m, name
    depth, i = 1, m.end()
    while depth:
        depth += {"{": 1, "}": -1}.get(text[i], 0)
        i += 1
    return text[m.end():i]


def _has_member(body, field):
    return re.search(r"[\s\*,]%s\s*(=[^;,]*)?[;,]" % re.escape(field), body) is not None


@needs_reference
def test_every_member_the_binding_reads_exists_in_eddl():
    tensor_h = gen.strip_comments(open(os.path.join(REFERENCE, "include/eddl/tensor/tensor.h"), encoding="utf-8").read())
    desc_h = gen.strip_comments(open(os.path.join(REFERENCE, "include/eddl/descriptors/descriptors.h"), encoding="utf-8").read())
    bodies = {"Tensor": _class_body(tensor_h, "Tensor"), "ConvolDescriptor": _class_body(desc_h, "ConvolDescriptor"),
              "PoolDescriptor": _class_body(desc_h, "PoolDescriptor")}
    text = _binding_text()
    checked = 0
    # one function at a time: parameter and local names -> class
    for m in re.finditer(r"\n(?:static )?[\w \*]+?\b(\w+)\(([^()]*)\)\s*\{(.*?)\n\}", text, flags=re.S):
        params, body = m.group(2), m.group(3)
        types = {}
        for cls in bodies:
            for v in re.findall(r"\b%s\s*\*\s*(\w+)" % cls, params + body):
                types[v] = cls
        for var, m1, m2 in re.findall(r"\b(\w+)->(\w+)(?:->(\w+))?", body):
            if var not in types:
                continue
            assert _has_member(bodies[types[var]], m1), "%s::%s (used in %s)" % (types[var], m1, m.group(1))
            checked += 1
            if m2:
                assert _has_member(bodies["Tensor"], m2), "Tensor::%s (used in %s through %s->%s)" % (m2, m.group(1), var, m1)
    assert checked > 100, checked
    # msg() with the signature the binding relies on
    utils_h = open(os.path.join(REFERENCE, "include/eddl/utils.h"), encoding="utf-8").read()
    assert re.search(r"void\s+msg\(const string&\s*text,\s*const string&\s*title", utils_h)


@needs_reference
def test_patch_applies_to_the_tree(tmp_path):
    patch = os.path.join(INTEG, "eddl_hip.patch")
    files = re.findall(r"^\+\+\+ b/(\S+)", open(patch, encoding="utf-8").read(), flags=re.M)
    assert len(files) == 6
    for f in files:
        os.makedirs(os.path.dirname(tmp_path / f), exist_ok=True)
        shutil.copy(os.path.join(REFERENCE, f), tmp_path / f)
    res = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch", "-i", patch], cwd=tmp_path, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0 and "FAILED" not in res.stdout and "fuzz" not in res.stdout, res.stdout
    # the patched headers parse to the same declarations, and keep the CUDA toolkit out of a cHIP build
    for h in gen.HEADERS:
        text = open(tmp_path / h, encoding="utf-8").read()
        kept, depth_hip = [], 0
        for line in text.split("\n"):
            s = line.strip()
            if re.match(r"#\s*ifndef\s+cHIP", s):
                depth_hip = 1
                continue
            if depth_hip:
                if re.match(r"#\s*if", s):
                    depth_hip += 1
                elif re.match(r"#\s*endif", s):
                    depth_hip -= 1
                continue
            kept.append(line)
        assert not re.search(r"cuda|cublas|curand|cudnn", "\n".join(l for l in kept if not l.strip().startswith("//")), flags=re.I), h
    assert "CS_HIP" in open(tmp_path / "include/eddl/apis/eddl.h").read() and "CS_HIP" in open(tmp_path / "src/apis/eddl.cpp").read()
    cm = open(tmp_path / "src/CMakeLists.txt").read()
    assert "-DcGPU -DcHIP" in cm and "hip_target.cmake" in cm and "${HIP_SOURCES})" in cm


def test_stub_file_parses_as_cpp():
    res = subprocess.run(["g++", "-std=c++14", "-fsyntax-only", "-Wall", "-Wextra", "-Werror", "-DEDDLHIP_SYNTAX_CHECK", gen.STUBS],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout


def test_binding_defines_what_the_host_layer_declares():
    """The backend's own host layer gets its gpu_* functions from the same translation unit: every gpu_* it declares is
    defined there with the same parameter types (the build would fail to link otherwise; this names the culprit)."""
    header = gen.drop_preprocessor(gen.strip_comments(open(os.path.join(ROOT, "eddl_amd", "host", "eddl_hip_host.h"), encoding="utf-8").read()))
    declared = {(n, t) for _, n, t in gen.functions(header, want_definitions=False)
                if n.startswith("gpu_") or n in ("cpu2gpu", "gpu2cpu", "get_gpu_fmem", "free_gpu_ptr")}
    bound = {(n, t) for _, n, t in gen.bound()}
    assert len(declared) >= 39
    assert not declared - bound, sorted(declared - bound)
    assert not bound - declared, sorted(bound - declared)
