"""CPU-side checks of the product library: it loads, exports every symbol the header declares,
refuses GPU work without a GPU (no silent CPU path), and its host-side logic -- the per-op
scheduler call and the proxy's iputSignal derivation -- matches the oracle bit for bit."""
import ctypes
import errno
import os
import re

import numpy as np
import pytest

import _oracle
import aws_ofi_nccl_amd as m
from aws_ofi_nccl_amd import synthetic

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("ofi_amd_hotpath.h", "ofi_amd_wire.h", "ofi_amd_sendrecv.h",
                                                      "ofi_amd_rma_abi.h", "ofi_amd_net_abi.h", "ofi_amd_nccl_err.h")]


def declared_symbols():
    names = set()
    for header in HEADERS:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
        names |= set(re.findall(r"\b(ofi_amd_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol(lib):
    names = declared_symbols()
    assert len(names) >= 45
    raw = ctypes.CDLL(m.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), "header declares %s but the library lacks it" % name
    # and the Python prototypes cover the same set
    assert sorted(m.PROTOTYPES) == names


def test_struct_sizes_match_the_header():
    assert ctypes.sizeof(m.XferInfo) == 24          # nccl_net_ofi_xfer_info_t
    assert ctypes.sizeof(m.SchedState) == 32
    assert ctypes.sizeof(m.GinDesc) == 64
    assert ctypes.sizeof(m.GinWire) == 224
    assert ctypes.sizeof(m.GinMr) == 56             # gin_remote_mr is 56 bytes in the reference too
    assert ctypes.sizeof(m.TunerVariant) == 16


def test_gpu_entry_points_fail_loudly_without_a_gpu(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    enodev = -errno.ENODEV
    assert lib.ofi_amd_gpu_init() == enodev
    p = ctypes.c_void_p()
    assert lib.ofi_amd_gpu_mem_alloc(ctypes.byref(p), 64) == enodev
    assert lib.ofi_amd_bounce_scatter(1, 64, 1, 64, 1, 1, 1, 1, None, None) == enodev
    assert lib.ofi_amd_flush_read(1, 1, 1, 1, None) == enodev
    assert lib.ofi_amd_sched_batch(1, 1, 1, 128, 1, 1, None) == enodev
    assert lib.ofi_amd_gin_rings_create(4, 256, ctypes.byref(p)) == enodev
    colls, sizes, nodes, ppn, algos = synthetic.tuner_axes()
    assert lib.ofi_amd_tuner_plan_create(colls.ctypes.data, 3, sizes.ctypes.data, 140,
                                         nodes.ctypes.data, 11, ppn.ctypes.data, 4,
                                         algos.ctypes.data, 3, ctypes.byref(p)) == enodev
    assert lib.ofi_amd_devcopy_register(1, 64, ctypes.byref(p)) == enodev
    assert lib.ofi_amd_net_link_create(4, 8192, 0, 0, 0, None, ctypes.byref(p)) == enodev and not p.value
    ids = (ctypes.c_uint32 * 2)(0, 1)
    assert lib.ofi_amd_devfab_create(4, 64, 2, ids, None, 0, None, ctypes.byref(p)) == enodev and not p.value
    assert lib.ofi_amd_gpu_flush_gpudirect_rdma_writes() == -errno.EPERM   # as the ROCm reference
    assert lib.ofi_amd_gpu_have_gdr_support_attr() == 0


def test_wire_encoders_match_oracle(lib, oracle):
    rng = np.random.default_rng(3)
    for _ in range(3000):
        comm, seq = int(rng.integers(0, 1024)), int(rng.integers(0, 8192))
        nseg, ack, rx = int(rng.integers(0, 16)), int(rng.integers(0, 2)), int(rng.integers(0, 16384))
        assert lib.ofi_amd_gin_imm(comm, seq, nseg, ack) == oracle.oracle_gin_imm(comm, seq, nseg, ack)
        assert lib.ofi_amd_gin_meta_header(comm, seq, nseg, ack) == \
            oracle.oracle_gin_meta_header(comm, seq, nseg, ack)
        assert lib.ofi_amd_gin_ack_msg(comm, rx) == oracle.oracle_gin_ack_msg(comm, rx)


@pytest.mark.parametrize("rails,min_stripe,max_small", [(4, 131072, 64), (4, 4096, 64), (3, 100000, 64),
                                                        (2, 8192, 0), (1, 131072, 64)])
def test_host_scheduler_matches_oracle(lib, oracle, rails, min_stripe, max_small):
    sizes = synthetic.stripe_sizes(rails * 7 + min_stripe, 20000)
    num, xf, ost = _oracle.sched_batch(oracle, sizes, rails, min_stripe, max_small, (1 % rails, 0))
    st = m.SchedState(1 % rails, 0, max_small, min_stripe, rails, 0)
    x = (m.XferInfo * 4)()
    for i, s in enumerate(sizes):
        n = lib.ofi_amd_sched_get_schedule(ctypes.byref(st), int(s), 128, x)
        assert n == num[i]
        for k in range(n):
            assert (x[k].rail_id, x[k].pad0, x[k].pad1, x[k].offset, x[k].msg_size) == (
                int(xf[i, k, 0]) & 0xFFFF, 0, 0, int(xf[i, k, 1]), int(xf[i, k, 2]))
    assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)
    bad = m.SchedState(0, 0, 64, 0, 4, 0)
    assert lib.ofi_amd_sched_get_schedule(ctypes.byref(bad), 100, 128, x) == -errno.EINVAL


@pytest.mark.parametrize("ack_model,agg_mask,signal_op,rails", [(1, 1, 1, 4), (1, 0, 2, 4), (0, 1, 1, 2),
                                                                 (1, 1, 2, 3)])
def test_proxy_derivation_matches_oracle(lib, oracle, ack_model, agg_mask, signal_op, rails):
    """ofi_amd_gin_iput_signal (product host code) against oracle_gin_iput_signal over a seeded
    stream: every field of every wire record, and the whole comm state after each op."""
    omrs = _oracle.default_mrs()
    pmrs = _oracle.default_mrs(m.GinMr)
    oc, pc = _oracle.GinComm(), m.GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(oc), 9, rails, 131072, 64, ack_model)
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(pc), 9, rails, 131072, 64, ack_model) == 0
    od, ow, pw = _oracle.GinDesc(), _oracle.GinWire(), m.GinWire()
    n = 12000 if ack_model else 9000
    for i in range(n):
        oracle.oracle_gin_gen_desc(1234, 6, i, 1, 64 if i % 2000 < 1500 else 3, signal_op, agg_mask,
                                   ctypes.byref(od))
        if i % 97 == 0:
            od.size = 0                                # signal-only / empty ops now and then
        pd = m.GinDesc.from_buffer_copy(bytes(od))
        orc = oracle.oracle_gin_iput_signal(ctypes.byref(oc), omrs, ctypes.byref(od), ctypes.byref(ow))
        prc = lib.ofi_amd_gin_iput_signal(ctypes.byref(pc), pmrs, 3, ctypes.byref(pd), ctypes.byref(pw))
        assert (orc, prc) in ((0, 0), (-11, -errno.EAGAIN))
        assert bytes(ow) == bytes(pw), i
        assert bytes(oc) == bytes(pc), i
    if ack_model == 0:
        assert prc == -errno.EAGAIN                    # window filled at 8192 outstanding
        lib.ofi_amd_gin_apply_ack(ctypes.byref(pc), 100)
        assert pc.tx_tail == 100
        lib.ofi_amd_gin_apply_ack(ctypes.byref(pc), 50)          # older ACK: ignored
        assert pc.tx_tail == 100
        assert lib.ofi_amd_gin_iput_signal(ctypes.byref(pc), pmrs, 3, ctypes.byref(pd), ctypes.byref(pw)) == 0


def test_proxy_derivation_survives_a_communicator_edited_by_hand(lib):
    """ofi_amd_gin_comm_t is the caller's struct.  Fields that comm_init and the derivation never
    produce -- a rail count outside 1..4, a zero stripe size, a pin or a rail cursor beyond the rail
    count, round-robin counters beyond it -- must end in an error or in rails inside the table,
    never in a read past the stripe-count or key tables (the build under AddressSanitizer in
    tests/test_host_sanitizers.py runs the same code)."""
    mrs = _oracle.default_mrs(m.GinMr)
    base = m.GinComm()
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(base), 3, 4, 131072, 64, 1) == 0
    state = bytes(base)
    d_small = m.GinDesc(0, 0, 4096, 8, 0, 1, 0, 0, 0, 0, 1, 2, 1)
    d_big = m.GinDesc(0, 0, 1 << 20, 8, 0, 1, 0, 0, 0, 0, 1, 2, 1)
    d_signal_only = m.GinDesc(0, 0, 0, 8, 0, 1, 1, 0, 0, 0, 1, 2, 2)
    w = m.GinWire()

    def edited(**fields):
        c = m.GinComm.from_buffer_copy(state)
        for k, v in fields.items():
            if k.startswith("sched_"):
                setattr(c.sched, k[6:], v)
            else:
                setattr(c, k, v)
        return c

    for d in (d_small, d_big):
        for fields in ({"sched_num_rails": 8}, {"sched_num_rails": 16}, {"sched_num_rails": 0},
                       {"sched_num_rails": -1}, {"sched_min_stripe_size": 0}):
            c = edited(**fields)
            assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d), ctypes.byref(w)) == \
                -errno.ENOMEM, fields                       # no schedule, as the reference's nullptr schedule
        for fields in ({"pinned_rail_id": 4}, {"pinned_rail_id": 1 << 20}, {"num_rails": 0}, {"num_rails": 9},
                       {"next_rail_id": 4}):
            c = edited(**fields)
            assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d), ctypes.byref(w)) == \
                -errno.EINVAL, fields
            assert bytes(w) == bytes(224)
        # counters beyond the rail count are reduced, not used as indices
        for fields in ({"sched_rr_small_counter": 4}, {"sched_rr_counter": 7}, {"sched_rr_counter": 0xFFFFFFFF},
                       {"sched_rr_small_counter": 1 << 30, "sched_rr_counter": 1 << 31}):
            c = edited(**fields)
            assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d), ctypes.byref(w)) == 0, fields
            assert 1 <= w.num_writes <= 4 and all(w.writes[k].rail < 4 for k in range(w.num_writes))
            assert c.sched.rr_small_counter < 4 and c.sched.rr_counter < 4
    for fields in ({"num_rails": 0}, {"next_rail_id": 9}, {"pinned_rail_id": 5}):
        c = edited(**fields)
        assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d_signal_only),
                                           ctypes.byref(w)) == -errno.EINVAL, fields
    # three rails (the general path from the start): same answers
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(base), 3, 3, 131072, 64, 1) == 0
    state = bytes(base)
    c = edited(sched_rr_counter=5, sched_rr_small_counter=3)
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d_big), ctypes.byref(w)) == 0
    assert all(w.writes[k].rail < 3 for k in range(w.num_writes))
    c = edited(pinned_rail_id=3)
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d_big), ctypes.byref(w)) == -errno.EINVAL


def test_proxy_rejects_bad_arguments(lib):
    c = m.GinComm()
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(c), 1024, 4, 131072, 64, 1) == -errno.EINVAL
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(c), 1, 5, 131072, 64, 1) == -errno.EINVAL
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(c), 1, 4, 0, 64, 1) == -errno.EINVAL
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(c), 1, 4, 131072, 64, 1) == 0
    d = m.GinDesc(0, 0, 8, 0, 0, 1, 7, 0, 0, 0, 1, 2, 2)
    w = m.GinWire()
    mrs = _oracle.default_mrs(m.GinMr)
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d), ctypes.byref(w)) == -errno.EINVAL
    # handles outside the registration table: the record comes from device code and is not trusted
    state = bytes(c)
    for src_mr, dst_mr, sig_mr, sig_op, size, n_mrs, want in [
            (0, 1, 2, 1, 8, 3, 0), (3, 1, 2, 1, 8, 3, -errno.EINVAL), (0, 3, 2, 1, 8, 3, -errno.EINVAL),
            (0, 1, 3, 1, 8, 3, -errno.EINVAL), (0, 1, 0xFFFF, 1, 8, 3, 0), (0, 1, 2, 1, 8, 2, -errno.EINVAL),
            (0, 1, 9, 0, 8, 3, 0),               # no signal: the signal handle is not looked at
            (9, 9, 2, 1, 0, 3, 0),               # no payload: the data handles are not looked at
            (0, 1, 2, 1, 8, 0, -errno.EINVAL)]:
        c2 = m.GinComm.from_buffer_copy(state)
        d = m.GinDesc(0, 0, size, 8, 0, 1, sig_op, 0, 0, src_mr, dst_mr, sig_mr, 2 if sig_op else 1)
        w.imm = 77
        rc = lib.ofi_amd_gin_iput_signal(ctypes.byref(c2), mrs, n_mrs, ctypes.byref(d), ctypes.byref(w))
        assert rc == want, (src_mr, dst_mr, sig_mr, sig_op, size, n_mrs)
        if want != 0:
            assert bytes(w) == bytes(224) and bytes(c2) == state     # nothing derived, state untouched
    assert lib.ofi_amd_gin_iput_signal(None, mrs, 3, ctypes.byref(d), ctypes.byref(w)) == -errno.EINVAL
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), None, 3, ctypes.byref(d), ctypes.byref(w)) == -errno.EINVAL
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, None, ctypes.byref(w)) == -errno.EINVAL
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c), mrs, 3, ctypes.byref(d), None) == -errno.EINVAL


def test_device_put_header_compiles_in_a_user_kernel(tmp_path):
    """include/ofi_amd_gin_device.h is all a user's own kernel needs to initiate puts."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    obj = tmp_path / "user_put_kernel.o"
    proc = subprocess.run([hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-Wall",
                           "-Wno-unknown-warning-option",
                           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                           "-I", os.path.join(ROOT, "include"), "-c",
                           os.path.join(ROOT, "tests", "host", "user_put_kernel.hip"), "-o", str(obj)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    text = "\n".join(l for l in proc.stdout.splitlines()
                     if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    assert proc.returncode == 0, text
    assert obj.stat().st_size > 0


def test_net_entry_points_check_their_arguments_without_a_link(lib):
    """nccl_net_ofi_isend / _irecv / _iflush / _test (src/nccl_ofi_api.cpp:440-567): what they answer
    before any comm is looked at."""
    internal, invalid = 3, 4
    vp = ctypes.c_void_p
    req = vp(1)
    assert lib.ofi_amd_net_isend(None, None, 8, 1, None, None, ctypes.byref(req)) == internal and req.value is None
    data, sizes, tags, mhs = (vp * 1)(), (ctypes.c_size_t * 1)(8), (ctypes.c_int * 1)(1), (vp * 1)()
    assert lib.ofi_amd_net_irecv(None, 1, data, sizes, tags, mhs, None, ctypes.byref(req)) == invalid
    not_a_comm = (ctypes.c_uint64 * 4)()
    assert lib.ofi_amd_net_irecv(not_a_comm, 1, data, sizes, tags, mhs, None, ctypes.byref(req)) == internal
    assert lib.ofi_amd_net_irecv(not_a_comm, 9, data, sizes, tags, mhs, None, ctypes.byref(req)) == invalid
    assert lib.ofi_amd_net_irecv_v5(not_a_comm, 1, data, None, tags, mhs, ctypes.byref(req)) == invalid
    assert lib.ofi_amd_net_iflush(None, 1, data, (ctypes.c_int * 1)(8), mhs, ctypes.byref(req)) == internal
    done = ctypes.c_int()
    assert lib.ofi_amd_net_test(None, ctypes.byref(done), None) == internal
    not_a_request = (ctypes.c_uint64 * 4)()
    assert lib.ofi_amd_net_test(not_a_request, ctypes.byref(done), None) == internal
    assert lib.ofi_amd_net_link_create(0, 8192, 0, 0, 0, None, ctypes.byref(req)) == -errno.EINVAL
    assert lib.ofi_amd_net_link_create(4, 16384, 0, 0, 0, None, ctypes.byref(req)) == -errno.EINVAL
    assert lib.ofi_amd_net_link_create(4, 8192, 0, 0, 257, None, ctypes.byref(req)) == -errno.EINVAL
    assert lib.ofi_amd_net_link_destroy(None) == -errno.EINVAL
    assert lib.ofi_amd_net_link_send_comm(None) is None and lib.ofi_amd_net_link_recv_comm(None) is None
