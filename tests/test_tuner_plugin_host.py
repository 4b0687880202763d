"""CPU-side checks of the NCCL tuner plugin symbols: they exist with the reference's names and
struct layout, and every hand-back-to-NCCL path of nccl_ofi_tuner_init
(src/tuner/nccl_ofi_tuner.cpp:47-158) behaves as in the reference.  Also the oracle's v2 / masked
decision variants against the plain ones."""
import ctypes
import os

import numpy as np
import pytest

import aws_ofi_nccl_amd as m

ENV_KEYS = ["OFI_NCCL_FORCE_PRODUCT_NAME", "OFI_NCCL_TUNER_TYPE", "OFI_NCCL_FORCE_NUM_RAILS", "NCCL_ALGO",
            "NCCL_PROTO", "OFI_NCCL_TUNER_NUM_CHANNELS", "OFI_NCCL_TUNER_NET_COMP_OVERHEAD"]


@pytest.fixture
def clean_env():
    saved = {k: os.environ.pop(k, None) for k in ENV_KEYS}
    yield
    for k, v in saved.items():
        os.environ.pop(k, None)
        if v is not None:
            os.environ[k] = v


def plugins(lib):
    return (m.NcclTunerV2.in_dll(lib, "ncclTunerPlugin_v2"), m.NcclTunerV3.in_dll(lib, "ncclTunerPlugin_v3"),
            m.NcclTunerV6.in_dll(lib, "ncclTunerPlugin_v6"))


def test_plugin_symbols_and_layout(lib):
    v2, v3, v6 = plugins(lib)
    for p in (v2, v3, v6):
        assert p.name == b"nccl_ofi_tuner"          # src/tuner/nccl_ofi_tuner.cpp:185,242,274
        assert p.init and p.getCollInfo
    assert v2.destroy and v3.destroy and v6.finalize and v6.getChunkSize
    ptr = ctypes.sizeof(ctypes.c_void_p)
    assert ctypes.sizeof(m.NcclTunerV2) == 4 * ptr and ctypes.sizeof(m.NcclTunerV6) == 5 * ptr


def test_init_hands_back_to_nccl(lib, clean_env):
    v2, v3, v6 = plugins(lib)
    ctx = ctypes.c_void_p(0xDEAD)

    def init3():
        ctx.value = 0xDEAD
        rc = v3.init(64, 8, None, ctypes.byref(ctx))
        return rc, ctx.value

    if not os.path.exists("/sys/devices/virtual/dmi/id/product_name"):
        assert init3() == (0, None)                 # platform type unavailable
    os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = "g4dn.xlarge"
    assert init3() == (0, None)                     # no tables for this platform
    os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = "p5en.48xlarge"
    os.environ["OFI_NCCL_TUNER_TYPE"] = "internal"  # case-insensitive, include/nccl_ofi_param_impl.h:35
    assert init3() == (0, None)
    os.environ["OFI_NCCL_TUNER_TYPE"] = "Region"
    os.environ["OFI_NCCL_FORCE_NUM_RAILS"] = "2"
    assert init3() == (0, None)                     # heterogeneous-job key
    del os.environ["OFI_NCCL_FORCE_NUM_RAILS"]
    os.environ["NCCL_ALGO"] = "Ring"
    ctx.value = 0xDEAD
    assert v2.init(64, 8, None, ctypes.byref(ctx)) == 0 and ctx.value is None   # :143-155
    del os.environ["NCCL_ALGO"]
    # a null context is "fall back": every entry point returns success and touches nothing
    table = np.full((7, 3), 1337.0, dtype=np.float32)
    nch = ctypes.c_int(5)
    assert v3.getCollInfo(None, 4, 1 << 20, 1, table.ctypes.data, 7, 3, ctypes.byref(nch)) == 0
    assert v6.getCollInfo(None, 4, 1 << 20, 1, table.ctypes.data, 7, 3, 0, ctypes.byref(nch)) == 0
    a, p = ctypes.c_int(-7), ctypes.c_int(-7)
    assert v2.getCollInfo(None, 4, 1 << 20, 0, 1, 1, ctypes.byref(a), ctypes.byref(p), ctypes.byref(nch)) == 0
    chunk = ctypes.c_size_t(99)
    assert v6.getChunkSize(None, 4, 1 << 20, 0, 1, 8, ctypes.byref(chunk)) == 0
    assert np.all(table == 1337.0) and (nch.value, a.value, p.value, chunk.value) == (5, -7, -7, 99)
    assert v3.destroy(None) == 0 and v6.finalize(None) == 0


def test_init_fails_loudly_without_a_gpu(lib, clean_env):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    _, v3, _ = plugins(lib)
    os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = "p5en.48xlarge"
    ctx = ctypes.c_void_p()
    assert v3.init(64, 8, None, ctypes.byref(ctx)) == 2 and ctx.value is None    # ncclSystemError


def test_oracle_v2_and_masked_variants(oracle):
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    a2, p2, ch2 = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    rng = np.random.default_rng(4)
    differ_nvls = differ_mask = 0
    for _ in range(4000):
        plat, coll = int(rng.integers(0, 4)), int(rng.choice([4, 2, 3]))
        N = int(rng.choice([4, 8, 16, 64, 256])); R = N * int(rng.choice([1, 8]))
        size = int(2 ** rng.uniform(0, 36))
        # full mask == plain decision
        oracle.oracle_region_decide(plat, coll, size, R, N, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
        oracle.oracle_region_decide_masked(plat, coll, size, R, N, 0x1FFFFF, ctypes.byref(a2), ctypes.byref(p2),
                                           ctypes.byref(ch2))
        assert (a.value, p.value) == (a2.value, p2.value)
        if a.value >= 0:
            # forbidding the chosen cell moves the decision to a later region or to "none"
            mask = 0x1FFFFF & ~(1 << (a.value * 3 + p.value))
            oracle.oracle_region_decide_masked(plat, coll, size, R, N, mask, ctypes.byref(a2), ctypes.byref(p2),
                                               ctypes.byref(ch2))
            assert (a2.value, p2.value) != (a.value, p.value)
            differ_mask += 1
        if plat < 2:
            oracle.oracle_model_decide(plat, coll, 1, size, R, N, 8, 3, ctypes.byref(a), ctypes.byref(p))
            oracle.oracle_model_decide_v2(plat, coll, 1, size, R, N, 8, 3, 1, ctypes.byref(a2), ctypes.byref(p2))
            assert (a.value, p.value) == (a2.value, p2.value)
            oracle.oracle_model_decide_v2(plat, coll, 1, size, R, N, 8, 3, 0, ctypes.byref(a2), ctypes.byref(p2))
            assert a2.value != 5                       # never NVLS tree without NVLS support
            differ_nvls += (a.value == 5)
    assert differ_mask > 500
    # the P5 quirk needs NVLS support in v2 (nccl_ofi_model.cpp:262-271)
    oracle.oracle_model_decide_v2(0, 4, 1, 4 << 30, 128, 16, 8, 3, 0, ctypes.byref(a), ctypes.byref(p))
    assert a.value != 5
    oracle.oracle_model_decide_v2(0, 4, 1, 4 << 30, 128, 16, 8, 3, 1, ctypes.byref(a), ctypes.byref(p))
    assert (a.value, p.value) == (5, 2)
