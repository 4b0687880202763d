"""Build recipe for libofi_amd_hotpath.so (gfx950 only) and for the test oracle.

    python -m aws_ofi_nccl_amd.build          # product library
    python -m aws_ofi_nccl_amd.build --oracle # also oracle/liboracle.so (+ oracle/_ref)

The product library is built in-tree (aws_ofi_nccl_amd/lib/) with hipcc; there is
no CPU variant of it.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
LIB = os.path.join(LIBDIR, "libofi_amd_hotpath.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: hipcc must not form packed fp32 instructions.
# -ffp-contract=off: the tuner model has to round exactly like unfused x86-64 code.
COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


HOST_LTO = ["-flto=thin"]


def _sources():
    out = []
    for name in sorted(os.listdir(CSRC)):
        if name.endswith(".hip") or name.endswith(".cpp"):
            out.append(os.path.join(CSRC, name))
    return out


def _compile(src):
    obj = os.path.join(LIBDIR, "obj", os.path.basename(src) + ".o")
    # The host sources go through link-time optimisation: the proxy, the loop-back runs and the entry points
    # make tens of millions of calls a second into each other's translation units (transmit engine, receiver,
    # fabrics), and those calls are inlined at link time.
    cmd = [HIPCC] + COMMON + (["-x", "hip"] if src.endswith(".hip") else HOST_LTO) + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    text = "\n".join(l for l in proc.stdout.splitlines()
                     if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stdout))
    return obj, text


def build_library(verbose=False):
    os.makedirs(os.path.join(LIBDIR, "obj"), exist_ok=True)
    srcs = _sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        results = list(pool.map(_compile, srcs))
    objs = [o for o, _ in results]
    if verbose:
        for _, text in results:
            if text.strip():
                print(text)
    # -Bsymbolic-functions: calls between the library's own entry points (the loop-back runs and the
    # proxy make millions a second) bind inside the library instead of going through the PLT
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-O3"] + HOST_LTO + ["-Wl,-Bsymbolic-functions", "-o", LIB] + \
        objs + ["-lpthread"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n%s" % proc.stdout)
    return LIB


def build_oracle():
    proc = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("oracle build failed:\n%s" % proc.stdout)
    # the reference-side glue of the integration guide against the reference's headers (a test binary; only
    # where the reference tree is present)
    proc = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host")], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("tests/host build failed:\n%s" % proc.stdout)


if __name__ == "__main__":
    print(build_library(verbose=True))
    if "--oracle" in sys.argv:
        build_oracle()
        print("oracle built")
