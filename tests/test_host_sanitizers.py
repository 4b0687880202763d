"""The product's plain-C++ host code (message buffer, send/receive state machines, wire codec,
host scheduler, GIN derivation, transmit engine and receiver, and the RMA entry points over them) built with AddressSanitizer and UndefinedBehaviorSanitizer and
run side by side with the oracle on random programs (tests/host/sanitize_driver.cpp), and the
descriptor rings' host push/pop and proxy threads built with ThreadSanitizer
(tests/host/tsan_rings_driver.cpp).  CPU only; the GPU sources are not part of these builds."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "aws_ofi_nccl_amd", "csrc")
HOST_SOURCES = ["sendrecv_proto.cpp", "wire_codec.cpp", "sched_host.cpp", "gin_rx.cpp", "gin_wire.cpp", "gin_tx.cpp",
                "rma_abi.cpp"]
# the sanitizer runtimes are linked statically: a dynamic AddressSanitizer runtime insists on being the
# first library loaded, which it is not in a process that has other libraries preloaded
SAN = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-g", "-O1"]
SAN_LINK = ["-static-libasan", "-static-libubsan"]


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
                    *[os.path.join(CSRC, s) for s in HOST_SOURCES], *objs, *SAN_LINK, "-lm", "-o", exe], check=True)
    return exe


def test_host_state_machines_clean_under_sanitizers_and_equal_to_the_oracle(driver):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([driver, "6"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                          timeout=300)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "agree over 6 seeds" in proc.stdout
    assert "rma entry points:" in proc.stdout
    print(proc.stdout[-400:])


def test_ring_push_pop_and_proxy_threads_clean_under_thread_sanitizer(tmp_path):
    """Three host producers per ring against two proxy threads, then against one popping thread per
    ring; four threads inserting, reading back and completing sequence numbers in one message buffer
    (tests/host/tsan_rings_driver.cpp): every descriptor once, per-producer order, no data race."""
    if not shutil.which("g++"):
        pytest.skip("no host compiler")
    exe = os.path.join(tmp_path, "tsan_rings")
    subprocess.run(["g++", "-std=c++17", "-pthread", "-fsanitize=thread", "-static-libtsan", "-O1", "-g",
                    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
                    os.path.join(ROOT, "tests", "host", "tsan_rings_driver.cpp"),
                    *[os.path.join(CSRC, s) for s in ("gin_proxy.cpp", "gin_wire.cpp", "sched_host.cpp", "sendrecv_proto.cpp",
                                                      "wire_codec.cpp")],
                    "-o", exe], check=True)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:exitcode=66")
    proc = subprocess.run([exe, "20000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                          timeout=300)
    if proc.returncode != 0 and "unexpected memory mapping" in proc.stdout:
        pytest.skip("ThreadSanitizer cannot map its shadow memory on this kernel")
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "rings clean with 3 producers per ring" in proc.stdout
    assert "proxy threads deriving: 80000 wire records on two threads equal one thread's" in proc.stdout
    assert "message buffer: 80000 sequence numbers on 4 threads" in proc.stdout


LINKS_SOURCES = ["net_abi.cpp", "net_fabric.cpp", "rma_abi.cpp", "gin_devfab.cpp", "gin_tx.cpp", "gin_wire.cpp", "gin_rx.cpp",
                 "gin_loopback.cpp", "gin_proxy.cpp", "sendrecv_loopback.cpp", "sendrecv_proto.cpp", "wire_codec.cpp", "sched_host.cpp"]


def test_in_process_fabrics_and_entry_points_clean_under_sanitizers(tmp_path):
    """The net and RMA entry points over the in-process fabrics (net_abi.cpp + net_fabric.cpp, rma_abi.cpp +
    gin_devfab.cpp) and the GIN loop-back run (gin_loopback.cpp) on random programs, with the device side of
    the library replaced by stand-ins that run each "launch" some calls after it was queued, or on a thread of
    their own (tests/host/links_sanitize_driver.cpp): a table, a sentinel slot or an rx buffer reused or freed
    while a launch still needs it is a sanitizer finding or a wrong byte; every byte, reported size and counter
    is checked."""
    if not shutil.which("g++"):
        pytest.skip("no host compiler")
    exe = os.path.join(tmp_path, "links_sanitize")
    subprocess.run(["g++", "-std=c++17", "-pthread", *SAN, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
                    os.path.join(ROOT, "tests", "host", "links_sanitize_driver.cpp"),
                    *[os.path.join(CSRC, s) for s in LINKS_SOURCES], *SAN_LINK, "-o", exe], check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([exe, "40"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=600)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "links: entry points, fabrics and loop-back runs clean over 40 seeds" in proc.stdout


def test_host_code_never_touches_what_a_queued_launch_still_uses(tmp_path):
    """The same program under ThreadSanitizer with every launch executed by a device thread: the host writes
    launch tables, rx buffers, flush slots and staging areas with plain stores, the device thread reads and
    writes them when the launch runs, and the only order between the two is what the library itself keeps
    (the launch call before, a sentinel seen after).  A table refilled before its launch's sentinel, or a
    buffer handed back before its copy ran, is a data race here.  (With the wait for the other table pair's
    sentinel taken out of gin_loopback.cpp, ThreadSanitizer reports nine races in the first seed.)"""
    if not shutil.which("g++"):
        pytest.skip("no host compiler")
    exe = os.path.join(tmp_path, "links_tsan")
    subprocess.run(["g++", "-std=c++17", "-pthread", "-fsanitize=thread", "-static-libtsan", "-O1", "-g",
                    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
                    os.path.join(ROOT, "tests", "host", "links_sanitize_driver.cpp"),
                    *[os.path.join(CSRC, s) for s in LINKS_SOURCES], "-o", exe], check=True)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:exitcode=66")
    proc = subprocess.run([exe, "3", "threaded"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                          timeout=900)
    if proc.returncode != 0 and "unexpected memory mapping" in proc.stdout:
        pytest.skip("ThreadSanitizer cannot map its shadow memory on this kernel")
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "links: entry points, fabrics and loop-back runs clean over 3 seeds" in proc.stdout
