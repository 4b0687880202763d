"""The product's plain-C++ host code (message buffer, send/receive state machines, wire codec,
host scheduler, GIN receiver) built with AddressSanitizer and UndefinedBehaviorSanitizer and
run side by side with the oracle on random programs (tests/host/sanitize_driver.cpp).
CPU only; the GPU sources are not part of this build."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "aws_ofi_nccl_amd", "csrc")
HOST_SOURCES = ["sendrecv_proto.cpp", "wire_codec.cpp", "sched_host.cpp", "gin_rx.cpp", "gin_wire.cpp"]
SAN = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-g", "-O1"]


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    if not shutil.which("g++") or not shutil.which("gcc"):
        pytest.skip("no host compiler")
    out = tmp_path_factory.mktemp("sanitize")
    objs = []
    for src in sorted(glob.glob(os.path.join(ROOT, "oracle", "oracle_*.c"))):
        obj = os.path.join(out, os.path.basename(src) + ".o")
        subprocess.run(["gcc", "-std=gnu11", "-ffp-contract=off", "-pthread", *SAN, "-c", os.path.basename(src),
                        "-o", obj], cwd=os.path.join(ROOT, "oracle"), check=True)
        objs.append(obj)
    exe = os.path.join(out, "sanitize_driver")
    subprocess.run(["g++", "-std=c++17", "-pthread", *SAN, "-I", os.path.join(ROOT, "include"),
                    "-I", os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests", "host", "sanitize_driver.cpp"),
                    *[os.path.join(CSRC, s) for s in HOST_SOURCES], *objs, "-lm", "-o", exe], check=True)
    return exe


def test_host_state_machines_clean_under_sanitizers_and_equal_to_the_oracle(driver):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)
    proc = subprocess.run([driver, "6"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                          timeout=300)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "agree over 6 seeds" in proc.stdout
