"""Pins the GIN oracle.  Wire encoders are checked against the reference's own macros and
bit-field structs compiled as-is (oracle/_ref).  The iputSignal state machine has no
wire-level test in the reference and does not build here, so it is checked against the
behaviour the reference documents in its comments (src/rdma/gin/nccl_ofi_gin.cpp:629-651)
and against hand-derived sequence / window / ACK numbers -- parity beyond that is unpinned."""
import ctypes

import numpy as np
import pytest

import _oracle
from _oracle import GinComm, GinDesc, GinWire

AGG = 1
INC, ADD = 1, 2


def new_comm(oracle, comm_id=5, rails=4, ack_model=1):
    c = GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(c), comm_id, rails, 131072, 64, ack_model)
    return c


def put(oracle, c, mrs, size, flags=0, signal_op=0, value=0, sig_off=0, src=0, dst=0):
    d = GinDesc(src, dst, size, sig_off, value, 1, signal_op, flags, 0, 0, 1,
                2 if signal_op else 0xFFFF, 2 if signal_op else 1)
    w = GinWire()
    rc = oracle.oracle_gin_iput_signal(ctypes.byref(c), mrs, ctypes.byref(d), ctypes.byref(w))
    return rc, w


def test_immediate_matches_reference_macros(oracle, ref):
    rng = np.random.default_rng(1)
    for _ in range(5000):
        comm, seq = int(rng.integers(0, 1024)), int(rng.integers(0, 8192))
        nseg, ack = int(rng.integers(0, 16)), int(rng.integers(0, 2))
        imm = oracle.oracle_gin_imm(comm, seq, nseg, ack)
        assert imm == ref.ref_gin_imm(comm, seq, nseg, ack)
        out = [ctypes.c_uint32() for _ in range(4)]
        ref.ref_gin_imm_decode(imm, *[ctypes.byref(x) for x in out])
        assert [x.value for x in out] == [comm, seq, nseg, ack]
        assert imm & 1 == 0           # bit 0 reserved, nccl_ofi_gin_types.h:48


def test_metadata_and_ack_match_reference_bitfields(oracle, ref):
    rng = np.random.default_rng(2)
    for _ in range(5000):
        comm, seq = int(rng.integers(0, 1024)), int(rng.integers(0, 8192))
        nseg, ack = int(rng.integers(0, 16)), int(rng.integers(0, 2))
        base, off, val = (int(x) for x in rng.integers(0, 1 << 62, 3))
        buf = np.zeros(4, dtype=np.uint64)
        ref.ref_gin_meta(comm, seq, nseg, ack, base, off, val, _oracle.ptr(buf))
        assert int(buf[0]) == oracle.oracle_gin_meta_header(comm, seq, nseg, ack)
        assert [int(x) for x in buf[1:]] == [base, off, val]
        rx = int(rng.integers(0, 1 << 14))
        assert oracle.oracle_gin_ack_msg(comm, rx) == ref.ref_gin_ack(comm, rx)
    # message type sits in the two lowest bits (static_asserts, nccl_ofi_gin_types.h:187-204)
    assert oracle.oracle_gin_meta_header(1023, 8191, 15, 1) & 3 == 0
    assert oracle.oracle_gin_ack_msg(1023, (1 << 14) - 1) & 3 == 1


def test_protocol_constants(ref):
    want = {0: 8191, 1: 16383, 2: 8192, 3: 64, 4: 16, 5: 4096, 6: 1024, 7: 4}
    for k, v in want.items():
        assert ref.ref_gin_const(k) == v


def test_sequence_numbers_and_segment_counts(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    sizes = [8, 63, 64, 131072, 131073, 262144, 262145, 393216, 393217, 1 << 20]
    stripes = [1, 1, 1, 1, 2, 2, 2, 2, 4, 4]      # 4 rails, 128 KiB minimum stripe
    for i, (s, n) in enumerate(zip(sizes, stripes)):
        sig = INC if i % 3 == 2 else 0
        rc, w = put(oracle, c, mrs, s, signal_op=sig)
        assert rc == 0 and w.seq == i and w.num_writes == n
        assert w.nseg == n + (1 if sig else 0)
        assert w.imm == oracle.oracle_gin_imm(5, i, w.nseg, 0)
        assert w.has_meta == (1 if sig else 0)
        assert sum(w.writes[k].len for k in range(n)) == s
        for k in range(n):
            assert w.writes[k].src == mrs[0].local_base + sum(w.writes[j].len for j in range(k))
            assert w.writes[k].dest == mrs[1].remote_address_offset + sum(w.writes[j].len for j in range(k))
            assert w.writes[k].key == mrs[1].key[w.writes[k].rail]
    assert c.tx_head == len(sizes)


def test_sequence_wraps_at_13_bits_cursor_at_14(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle, ack_model=1)
    seqs = []
    for i in range(20000):
        rc, w = put(oracle, c, mrs, 256)
        assert rc == 0
        seqs.append(w.seq)
    assert seqs == [i % 8192 for i in range(20000)]
    assert c.tx_head == 20000 % 16384


def test_metadata_signal_values(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    rc, w = put(oracle, c, mrs, 1024, signal_op=INC, value=77, sig_off=40)
    assert list(w.meta)[1:] == [mrs[2].remote_address, 40, 1]      # INC sends 1
    rc, w = put(oracle, c, mrs, 1024, signal_op=ADD, value=77, sig_off=48)
    assert list(w.meta)[1:] == [mrs[2].remote_address, 48, 77]     # ADD sends the value
    assert w.meta[0] == oracle.oracle_gin_meta_header(5, 1, 2, 0)
    rc, w = put(oracle, c, mrs, 1024, signal_op=3)
    assert rc == -22                                               # only 0 / INC / ADD
    assert c.tx_head == 2                                          # rejected op consumed nothing


def test_signal_first_write_defers_doorbell_to_metadata_send(oracle):
    # "FI_MORE ... for the first stripe of a put+signal (the metadata send that follows flushes it)"
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    rc, w = put(oracle, c, mrs, 1 << 20, signal_op=INC)
    assert [w.writes[k].more for k in range(4)] == [1, 0, 0, 0]
    assert w.meta_more == 0 and w.meta_rail == w.writes[0].rail


def test_pin_batch_and_flush_by_non_aggregate_op(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    rails = []
    for _ in range(5):                      # aggregating single-stripe ops: all defer, same rail
        rc, w = put(oracle, c, mrs, 4096, flags=AGG)
        assert w.writes[0].more == 1
        rails.append(w.writes[0].rail)
    assert len(set(rails)) == 1 and c.pinned_rail_id == rails[0] and c.pinned_rail_run == 5
    rc, w = put(oracle, c, mrs, 4096, flags=0)      # batch end: rings, on the pinned rail
    assert w.writes[0].rail == rails[0] and w.writes[0].more == 0
    assert c.pinned_rail_id == -1 and c.pinned_rail_run == 0
    rc, w = put(oracle, c, mrs, 4096, flags=0)      # no pin: scheduler's round robin resumes
    # the scheduler advanced once per op (7 ops so far on the large counter, start 0)
    assert w.writes[0].rail == 6 % 4


def test_pin_rotates_every_16_ops(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    more, rails = [], []
    for _ in range(40):
        rc, w = put(oracle, c, mrs, 512, flags=AGG)
        more.append(w.writes[0].more)
        rails.append(w.writes[0].rail)
    # 15 deferred + 1 ringing op per batch of GIN_REQS_PER_DOORBELL
    assert more == ([1] * 15 + [0]) * 2 + [1] * 8
    assert len(set(rails[:16])) == 1 and len(set(rails[16:32])) == 1
    # batch k starts on the rail the scheduler hands its first op: op index 16k (mod 4 rails)
    assert rails[0] == 0 and rails[16] == 16 % 4 and rails[32] == 32 % 4


def test_striped_op_rings_the_pinned_rail(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    rc, w = put(oracle, c, mrs, 4096, flags=AGG)          # opens a pin on rail 0
    assert c.pinned_rail_id == 0
    rc, w = put(oracle, c, mrs, 200000, flags=AGG)        # 2 stripes: scheduler gives rails 1,2
    assert w.num_writes == 2
    assert [w.writes[k].rail for k in range(2)] == [0, 2]  # stripe 0 redirected onto the pin
    assert [w.writes[k].more for k in range(2)] == [0, 0]  # striped ops never defer
    assert c.pinned_rail_id == -1
    rc, w = put(oracle, c, mrs, 4096, flags=AGG)          # pin on rail 3 (scheduler: 0,1-2,3)
    assert c.pinned_rail_id == 3
    rc, w = put(oracle, c, mrs, 1 << 20, flags=AGG)       # 4 stripes touch every rail: no redirect
    assert sorted(w.writes[k].rail for k in range(4)) == [0, 1, 2, 3]
    assert w.writes[0].rail == 0


def test_signal_only_uses_pin_or_round_robin(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle)
    got = []
    for _ in range(5):
        rc, w = put(oracle, c, mrs, 0, signal_op=INC)
        assert w.num_writes == 0 and w.nseg == 1 and w.has_meta == 1
        got.append(w.meta_rail)
    assert got == [0, 1, 2, 3, 0]                          # get_next_rail round robin
    rc, w = put(oracle, c, mrs, 4096, flags=AGG)           # open a pin
    pin = c.pinned_rail_id
    rc, w = put(oracle, c, mrs, 0, signal_op=INC, flags=AGG)
    assert w.meta_rail == pin and w.meta_more == 1         # rides and keeps the pin


def test_window_blocks_at_8192_without_acks(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle, ack_model=0)
    first_ack = None
    for i in range(8192):
        rc, w = put(oracle, c, mrs, 128)
        assert rc == 0
        if w.ack_req and first_ack is None:
            first_ack = i
    # threshold 4096 outstanding, then every op counts: the 65th op above it asks
    assert first_ack == 4096 + 64
    rc, w = put(oracle, c, mrs, 128)
    assert rc == -11 and c.tx_head == 8192                 # window full: would block


def test_ack_hysteresis_with_immediate_acks(oracle):
    mrs = _oracle.default_mrs()
    c = new_comm(oracle, ack_model=1)
    asked = []
    for i in range(20000):
        rc, w = put(oracle, c, mrs, 128)
        assert rc == 0
        if w.ack_req:
            asked.append(i)
            assert (w.imm >> 28) & 1 == 1
    # op 4160 asks; its ACK empties the window; 4096 more ops refill it, 64 more pass the gate
    assert asked == [4160, 4160 + 1 + 4096 + 64, 4160 + 2 * (1 + 4096 + 64), 4160 + 3 * (1 + 4096 + 64)]


def test_generator_fields(oracle):
    d = GinDesc()
    sizes = []
    for i in range(4096):
        oracle.oracle_gin_gen_desc(99, 3, i, 1, 64, INC, 1, ctypes.byref(d))
        assert 8 <= d.size < (1 << 20) and d.src_off % 8 == 0 and d.dst_off % 8 == 0
        assert d.src_off + d.size <= (1 << 30) and d.dst_off + d.size <= (1 << 30)
        assert d.context == 3 and d.rank == 1 and d.opt_flags in (0, 1)
        if i % 64 == 63:
            assert (d.signal_op, d.kind, d.sig_mr) == (INC, 2, 2)
            assert d.signal_off == 8 * ((i // 64) % 512)
        else:
            assert (d.signal_op, d.kind, d.sig_mr, d.signal_off) == (0, 1, 0xFFFF, 0)
        sizes.append(d.size)
    octaves = np.bincount(np.log2(np.array(sizes)).astype(int), minlength=20)[3:20]
    assert octaves.min() > 150          # every octave 2^3..2^19 is populated (mean 241)
    assert ctypes.sizeof(GinDesc) == 64 and ctypes.sizeof(GinWire) == 224
