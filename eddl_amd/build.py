"""Builds eddl_amd/libeddlhip.so (gfx950 code object + C ABI) with hipcc, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["runtime.hip", "elementwise.hip", "pool.hip", "conv.hip", "dense.hip", "generator.hip"]
LIB = os.path.join(HERE, "libeddlhip.so")
# the benchmark's device probes: a library of their own beside the C ABI (include/eddlhip_probe.h)
PROBE_SOURCES = ["probe.hip"]
PROBE_LIB = os.path.join(HERE, "libeddlhip_probe.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",  # every fused multiply-add in this library is written explicitly
    "-fhip-fp32-correctly-rounded-divide-sqrt",  # '/' and sqrtf are IEEE (the parity tests are bit-exact on them)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no packed-fp32 VALU forms
    "-Wall", "-Wno-unused-function",
]


def _compile(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that line is noise
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _compile([hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB], verbose)
    _compile([hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, s) for s in PROBE_SOURCES] + ["-L" + HERE, "-leddlhip", "-Wl,-rpath,$ORIGIN", "-o", PROBE_LIB], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
