"""The reference-side glue of the integration guide at the repository root is code, not prose: its sections 1 (the replacement of
src/nccl_ofi_rocm.cpp) and 2 (an nccl_ofi_device_copy implementation) are compiled against the
reference's own headers and linked against the library (tests/host/integration_glue.cpp), the
public headers compile as C11, and on a GPU the compiled glue runs the patterns of the
reference's tests/unit/gdrcopy.cpp through the C++ class."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GLUE_SRC = os.path.join(ROOT, "tests", "host", "integration_glue.cpp")
GLUE_BIN = os.path.join(ROOT, "tests", "host", "bin", "integration_glue")
REFERENCE = os.environ.get("REFERENCE", "/root/reference")
HEADERS = ["ofi_amd_hotpath.h", "ofi_amd_wire.h", "ofi_amd_sendrecv.h", "ofi_amd_rma_abi.h", "ofi_amd_net_abi.h",
           "ofi_amd_nccl_err.h", "ofi_amd_gin_device.h"]


def fenced_cpp_blocks(section_title):
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    start = text.index(section_title)
    end = text.index("\n## ", start + 1)
    return re.findall(r"```cpp\n(.*?)```", text[start:end], flags=re.S)


def test_glue_source_is_the_text_printed_in_the_integration_notes():
    src = open(GLUE_SRC).read()
    for marker, title in (("section 1", "## 1. GPU glue"), ("section 2", "## 2. Device copy")):
        body = src[src.index("// [%s]\n" % marker) + len("// [%s]\n" % marker):src.index("// [end of %s]" % marker)]
        blocks = fenced_cpp_blocks(title)
        assert len(blocks) == 1, title
        assert body == blocks[0], "tests/host/integration_glue.cpp and the guide's %s differ" % title


@pytest.mark.parametrize("header", HEADERS[:6])
def test_public_headers_compile_as_c11(header):
    """The boundary is a C ABI: every header a binding would include is valid C11 on its own."""
    proc = subprocess.run(["gcc", "-std=c11", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c",
                           "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "include", header)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout


def test_public_headers_compile_as_cxx_next_to_nccl_err_h(tmp_path):
    """ofi_amd_rma_abi.h defines ncclResult_t under NCCL's own include guard: including NCCL's err.h
    first or second must both work (where the reference tree is present)."""
    err_h = os.path.join(REFERENCE, "3rd-party", "nccl", "cuda", "include", "nccl", "err.h")
    if not os.path.exists(err_h):
        pytest.skip("reference tree not available")
    for order in (('#include "nccl/err.h"', '#include "ofi_amd_rma_abi.h"'),
                  ('#include "ofi_amd_rma_abi.h"', '#include "nccl/err.h"')):
        src = tmp_path / "both.cpp"
        src.write_text("\n".join(order) + "\nstatic_assert(ncclRemoteError == 6, \"\");\nint main() { return ncclSuccess; }\n")
        proc = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                               "-I", os.path.join(REFERENCE, "3rd-party", "nccl", "cuda", "include"), str(src)],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert proc.returncode == 0, proc.stdout


def test_glue_compiles_against_the_reference_headers_and_links(lib):
    """g++ on the glue with -I<reference>/include, linked against libofi_amd_hotpath.so; its `link`
    mode calls the forwards that answer without a device."""
    if not os.path.exists(os.path.join(REFERENCE, "include", "nccl_ofi_rocm.h")):
        pytest.skip("reference tree not available")
    proc = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host"), "REFERENCE=" + REFERENCE],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    assert os.path.exists(GLUE_BIN)
    run = subprocess.run([GLUE_BIN, "link"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert run.returncode == 0 and "link: ok" in run.stdout, run.stdout


@pytest.mark.gpu
def test_gdrcopy_patterns_through_the_cxx_class_on_the_gpu(gpu):
    """tests/unit/gdrcopy.cpp:15-133 through nccl_ofi_device_copy_amd, in a process of its own (the
    binary was built where the reference headers are; this machine need not have them)."""
    if not os.path.exists(GLUE_BIN):
        pytest.skip("tests/host/bin/integration_glue was not built (no reference tree at build time)")
    run = subprocess.run([GLUE_BIN, "gpu"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert run.returncode == 0 and "gpu: ok" in run.stdout, run.stdout
