"""GPU parity: GIN descriptor production into pinned-host rings drained by the host proxy,
through the C ABI, against the CPU oracle (descriptor stream and derived wire records
bit-exact per context), plus the ring protocol on the real pinned rings."""
import ctypes
import errno
import threading

import numpy as np
import pytest
import torch

import _gpu
import _oracle
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

SEED = 20240607


def make_rings(lib, nctx, cap):
    r = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rings_create(nctx, cap, ctypes.byref(r)) == 0
    return r


def oracle_stream(oracle, nctx, ops, signal_every, signal_op, agg_mask, peer=1):
    out = np.zeros((nctx, ops, 8), dtype=np.uint64)
    d = _oracle.GinDesc()
    for c in range(nctx):
        for i in range(ops):
            oracle.oracle_gin_gen_desc(SEED, c, i, peer, signal_every, signal_op, agg_mask, ctypes.byref(d))
            out[c, i] = np.frombuffer(bytes(d), dtype=np.uint64)
    return out


def produce_and_drain(lib, rings, nctx, ops, mode, signal_every=64, signal_op=1, agg_mask=1,
                      comms=None, mrs=None, want_wire=False, timeout_ms=10000):
    descs = (m.GinDesc * (nctx * ops))() if mode == 1 else None
    wires = (m.GinWire * (nctx * ops))() if want_wire else None
    stats = m.GinProxyStats()
    assert lib.ofi_amd_gin_produce_seeded(rings, SEED, ops, 1, signal_every, signal_op, agg_mask, 0,
                                          _gpu.stream()) == 0
    rc = lib.ofi_amd_gin_proxy_drain(rings, ops, mode, ctypes.cast(descs, ctypes.c_void_p) if descs else None,
                                     ctypes.cast(comms, ctypes.c_void_p) if comms else None,
                                     ctypes.cast(mrs, ctypes.c_void_p) if mrs else None, len(mrs) if mrs else 0,
                                     ctypes.cast(wires, ctypes.c_void_p) if wires else None,
                                     timeout_ms, ctypes.byref(stats))
    _gpu.sync()
    return rc, stats, descs, wires


@pytest.mark.parametrize("nctx,cap,ops", [(1, 256, 1), (1, 256, 255), (3, 256, 257), (4, 256, 5000),
                                          (8, 4096, 20000), (64, 1024, 3001)])
def test_descriptor_stream_bit_exact(lib, oracle, gpu, nctx, cap, ops):
    rings = make_rings(lib, nctx, cap)
    rc, stats, descs, _ = produce_and_drain(lib, rings, nctx, ops, mode=1)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    assert stats.descriptors == nctx * ops and stats.signals == nctx * (ops // 64)
    got = np.frombuffer(descs, dtype=np.uint64).reshape(nctx, ops, 8)
    want = oracle_stream(oracle, nctx, ops, 64, 1, 1)
    assert np.array_equal(got, want)
    # the checksum the proxy folds equals the oracle's over the same stream
    assert stats.checksum == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 0, 4, 131072,
                                                                64, 1, None)
    assert lib.ofi_amd_gin_rings_destroy(rings) == 0


def test_second_launch_continues_ring_positions(lib, oracle, gpu):
    """Cursors persist across launches: a second batch lands behind the first (positions keep
    counting past the capacity, slots wrap)."""
    nctx, cap, ops = 2, 256, 1000
    rings = make_rings(lib, nctx, cap)
    for _ in range(3):
        rc, stats, descs, _ = produce_and_drain(lib, rings, nctx, ops, mode=1)
        assert rc == 0
        got = np.frombuffer(descs, dtype=np.uint64).reshape(nctx, ops, 8)
        assert np.array_equal(got, oracle_stream(oracle, nctx, ops, 64, 1, 1))
    seqs, recs = ctypes.c_void_p(), ctypes.c_void_p()
    n, c = ctypes.c_uint32(), ctypes.c_uint32()
    assert lib.ofi_amd_gin_rings_view(rings, ctypes.byref(recs), ctypes.byref(seqs), ctypes.byref(n),
                                      ctypes.byref(c)) == 0
    assert (n.value, c.value) == (nctx, cap)
    seq = np.ctypeslib.as_array(ctypes.cast(seqs, ctypes.POINTER(ctypes.c_uint32)),
                                shape=(nctx * cap,)).reshape(nctx, cap)
    # every slot has been freed for its next lap: sequence == next position that maps to it
    for s in range(cap):
        nxt = s + ((3000 - s + cap - 1) // cap) * cap
        assert seq[0, s] == nxt and seq[1, s] == nxt
    lib.ofi_amd_gin_rings_destroy(rings)


@pytest.mark.parametrize("signal_every,signal_op,agg_mask", [(64, 1, 1), (3, 2, 1), (0, 0, 0)])
def test_wire_records_bit_exact(lib, oracle, gpu, signal_every, signal_op, agg_mask):
    """Proxy mode 3: sequence numbers, segment counts, immediate data, stripes, doorbell flags and
    metadata messages derived from the GPU-produced stream equal the oracle's iputSignal."""
    nctx, cap, ops = 6, 512, 12000
    rings = make_rings(lib, nctx, cap)
    comms = (m.GinComm * nctx)()
    for c in range(nctx):
        assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[c]), c, 4, 131072, 64, 1) == 0
    pmrs, omrs = _oracle.default_mrs(m.GinMr), _oracle.default_mrs()
    rc, stats, _, wires = produce_and_drain(lib, rings, nctx, ops, mode=3, signal_every=signal_every,
                                            signal_op=signal_op, agg_mask=agg_mask, comms=comms, mrs=pmrs,
                                            want_wire=True)
    assert rc == 0
    got = np.frombuffer(wires, dtype=np.uint8).reshape(nctx, ops, 224)
    d, w = _oracle.GinDesc(), _oracle.GinWire()
    total_writes = 0
    for c in range(nctx):
        oc = _oracle.GinComm()
        oracle.oracle_gin_comm_init(ctypes.byref(oc), c, 4, 131072, 64, 1)
        for i in range(ops):
            oracle.oracle_gin_gen_desc(SEED, c, i, 1, signal_every, signal_op, agg_mask, ctypes.byref(d))
            assert oracle.oracle_gin_iput_signal(ctypes.byref(oc), omrs, ctypes.byref(d), ctypes.byref(w)) == 0
            assert bytes(w) == got[c, i].tobytes(), (c, i)
            total_writes += w.num_writes
        assert bytes(oc) == bytes(comms[c])
    assert stats.writes == total_writes
    assert stats.checksum == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, signal_every, signal_op,
                                                                agg_mask, 1, 4, 131072, 64, 1, omrs)
    lib.ofi_amd_gin_rings_destroy(rings)


def test_proxy_mode_two_derives_without_folding_the_wire_records(lib, oracle, gpu):
    """Mode 2 is mode 3 without the check: the same wire records and comm state, the checksum of
    the descriptor stream alone."""
    nctx, cap, ops = 5, 512, 7000
    pmrs = _oracle.default_mrs(m.GinMr)
    out = []
    for mode in (2, 3):
        rings = make_rings(lib, nctx, cap)
        comms = (m.GinComm * nctx)()
        for c in range(nctx):
            assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[c]), c, 4, 131072, 64, 1) == 0
        rc, stats, _, wires = produce_and_drain(lib, rings, nctx, ops, mode=mode, comms=comms, mrs=pmrs,
                                                want_wire=True)
        assert rc == 0
        out.append((bytes(wires), bytes(comms), stats.writes, stats.checksum))
        lib.ofi_amd_gin_rings_destroy(rings)
    assert out[0][:3] == out[1][:3]
    assert out[0][3] == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 0, 4, 131072, 64, 1, None)
    assert out[1][3] == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 1, 4, 131072, 64, 1,
                                                          _oracle.default_mrs())


def test_proxy_derives_gets_among_puts_like_the_oracle(lib, oracle, gpu):
    """A table in which every third descriptor is a get goes through the device-side put, the ring
    and the proxy's derivation (mode 2); every wire record and the final comm state equal what
    the oracle derives from the same descriptors one by one."""
    ops, cap = 3000, 512
    rng = np.random.default_rng(99)
    table = np.zeros((1, ops, 8), dtype=np.uint64)
    for i in range(ops):
        size = int(2 ** rng.uniform(0, 21))
        if i % 3 == 2:      # get: remote handle 2, local handle 0
            table[0, i] = [int(rng.integers(0, 1 << 30)), int(rng.integers(0, 1 << 30)), size, 0, 0, 1, 0,
                           2 | (0 << 16) | (0xFFFF << 32) | (3 << 48)]
        else:
            sop = 1 if i % 7 == 0 else 0
            table[0, i] = [int(rng.integers(0, 1 << 30)), int(rng.integers(0, 1 << 30)), size, 8 * (i % 16) if sop else 0,
                           0, 1 | (sop << 32), int(rng.integers(0, 2)),
                           0 | (1 << 16) | ((2 if sop else 0xFFFF) << 32) | ((2 if sop else 1) << 48)]
    d_table = _gpu.to_dev(table)
    rings = make_rings(lib, 1, cap)
    comms = (m.GinComm * 1)()
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[0]), 9, 4, 131072, 64, 1) == 0
    pmrs, omrs = _oracle.default_mrs(m.GinMr), _oracle.default_mrs()
    wires = (m.GinWire * ops)()
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 1, 0, _gpu.stream()) == 0
    stats = m.GinProxyStats()
    rc = lib.ofi_amd_gin_proxy_drain(rings, ops, 2, None, ctypes.cast(comms, ctypes.c_void_p),
                                     ctypes.cast(pmrs, ctypes.c_void_p), 3, ctypes.cast(wires, ctypes.c_void_p),
                                     5000, ctypes.byref(stats))
    _gpu.sync()
    assert rc == 0 and stats.descriptors == ops
    oc = _oracle.GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(oc), 9, 4, 131072, 64, 1)
    n_reads = 0
    for i in range(ops):
        d = _oracle.GinDesc.from_buffer_copy(table[0, i].tobytes())
        w = _oracle.GinWire()
        fn = oracle.oracle_gin_iget if d.kind == 3 else oracle.oracle_gin_iput_signal
        assert fn(ctypes.byref(oc), omrs, ctypes.byref(d), ctypes.byref(w)) == 0
        assert bytes(w) == bytes(wires[i]), i
        n_reads += w.num_writes if d.kind == 3 else 0
    assert bytes(oc) == bytes(comms[0]) and comms[0].tx_head == ops - ops // 3
    assert n_reads > ops // 3
    lib.ofi_amd_gin_rings_destroy(rings)


def test_proxy_stops_at_a_descriptor_with_a_handle_outside_the_table(lib, gpu):
    """The handle indices of a record are written by device code; the proxy checks them against the
    registration table it was given and ends the drain with -EINVAL instead of reading past it."""
    ops, cap = 200, 256
    table = np.zeros((1, ops, 8), dtype=np.uint64)
    table[0, :, 2] = 4096                                        # size
    table[0, :, 5] = 1                                           # rank 1, no signal
    table[0, :, 7] = (1 << 16) | (0xFFFF << 32) | (1 << 48)      # src 0, dst 1, no signal handle, kind 1
    table[0, 150, 7] = 7 | (1 << 16) | (0xFFFF << 32) | (1 << 48)    # source handle 7 of a table of 3
    d_table = _gpu.to_dev(table)
    for n_mrs, want_rc, want_done in ((3, -errno.EINVAL, 150), (8, 0, ops)):
        rings = make_rings(lib, 1, cap)
        comms = (m.GinComm * 1)()
        assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[0]), 1, 4, 131072, 64, 1) == 0
        mrs = (m.GinMr * 8)()
        assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 1, 0, _gpu.stream()) == 0
        _gpu.sync()                                              # 200 records fit the ring: the producer is done
        stats = m.GinProxyStats()
        rc = lib.ofi_amd_gin_proxy_drain(rings, ops, 2, None, ctypes.cast(comms, ctypes.c_void_p),
                                         ctypes.cast(mrs, ctypes.c_void_p), n_mrs, None, 2000, ctypes.byref(stats))
        assert rc == want_rc and comms[0].tx_head == want_done
        lib.ofi_amd_gin_rings_destroy(rings)


def test_proxy_thread_count_does_not_change_the_result(lib, oracle, gpu):
    """Several proxy threads, each owning a range of contexts: wire records, per-context comm
    state and the checksum equal the single-thread run (and so the oracle's)."""
    nctx, cap, ops = 13, 512, 6000
    omrs, pmrs = _oracle.default_mrs(), _oracle.default_mrs(m.GinMr)
    want_ck = oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 5, 2, 1, 1, 4, 131072, 64, 1, omrs)
    results = []
    for threads in (1, 3, 4, 32):
        rings = make_rings(lib, nctx, cap)
        comms = (m.GinComm * nctx)()
        for c in range(nctx):
            assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[c]), c, 4, 131072, 64, 1) == 0
        wires = (m.GinWire * (nctx * ops))()
        stats = m.GinProxyStats()
        assert lib.ofi_amd_gin_produce_seeded(rings, SEED, ops, 1, 5, 2, 1, 0, _gpu.stream()) == 0
        rc = lib.ofi_amd_gin_proxy_drain_mt(rings, ops, 3, None, ctypes.cast(comms, ctypes.c_void_p),
                                            ctypes.cast(pmrs, ctypes.c_void_p), 3,
                                            ctypes.cast(wires, ctypes.c_void_p), 10000, threads,
                                            ctypes.byref(stats))
        _gpu.sync()
        assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
        assert stats.descriptors == nctx * ops and stats.checksum == want_ck
        results.append((bytes(wires), bytes(comms), stats.writes, stats.signals))
        lib.ofi_amd_gin_rings_destroy(rings)
    assert all(r == results[0] for r in results[1:])
    rings = make_rings(lib, 2, 256)
    assert lib.ofi_amd_gin_proxy_drain_mt(rings, 0, 0, None, None, None, 0, None, 10, 0, None) == -22
    assert lib.ofi_amd_gin_proxy_drain_mt(rings, 0, 0, None, None, None, 0, None, 10, 65, None) == -22
    lib.ofi_amd_gin_rings_destroy(rings)


def drain_descs(lib, rings, nctx, ops, timeout_ms=10000):
    descs = (m.GinDesc * (nctx * ops))()
    stats = m.GinProxyStats()
    rc = lib.ofi_amd_gin_proxy_drain(rings, ops, 1, ctypes.cast(descs, ctypes.c_void_p), None, None, 0, None,
                                     timeout_ms, ctypes.byref(stats))
    _gpu.sync()
    return rc, stats, np.frombuffer(descs, dtype=np.uint64).reshape(nctx, ops, 8)


def test_device_put_single_wave_keeps_table_order(lib, oracle, gpu):
    """One producing wavefront per context through the device-side put: the ring order is the
    table order, so the drained stream and its checksum equal the oracle's."""
    nctx, cap, ops = 5, 256, 3001
    table = oracle_stream(oracle, nctx, ops, 64, 1, 1)
    d_table = _gpu.to_dev(table)
    rings = make_rings(lib, nctx, cap)
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 1, 0, _gpu.stream()) == 0
    rc, stats, got = drain_descs(lib, rings, nctx, ops)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    assert np.array_equal(got, table)
    assert stats.checksum == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 0, 4, 131072,
                                                                64, 1, None)
    # a second launch on the same rings (seeded generator this time) continues at the cursor
    rc, stats, _d, _w = produce_and_drain(lib, rings, nctx, 500, mode=0)
    assert rc == 0 and stats.descriptors == nctx * 500
    # and the device-side put again behind it: cursor and free-slot horizon carried over
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 1, 0, _gpu.stream()) == 0
    rc, stats, got = drain_descs(lib, rings, nctx, ops)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    assert np.array_equal(got, table)
    lib.ofi_amd_gin_rings_destroy(rings)


@pytest.mark.parametrize("waves,cap,ops", [(2, 256, 5000), (7, 256, 10001), (16, 1024, 20000),
                                           (64, 4096, 70000)])
def test_device_put_many_producers_per_ring(lib, gpu, waves, cap, ops):
    """Several wavefronts put into one ring at once: nothing lost or duplicated, every
    64-descriptor group lands in consecutive slots in lane order, and each producer's groups
    appear in the order it put them (the multi-producer guarantees of the reference ring)."""
    nctx = 6
    rng = np.random.default_rng(waves)
    table = rng.integers(0, 1 << 63, (nctx, ops, 8), dtype=np.uint64)
    table[:, :, 0] = np.arange(ops, dtype=np.uint64)[None, :]          # op index
    table[:, :, 1] = np.arange(nctx, dtype=np.uint64)[:, None]         # context
    d_table = _gpu.to_dev(table)
    rings = make_rings(lib, nctx, cap)
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, waves, 0, _gpu.stream()) == 0
    rc, stats, got = drain_descs(lib, rings, nctx, ops)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0 and stats.descriptors == nctx * ops
    for c in range(nctx):
        idx = got[c, :, 0].astype(np.int64)
        assert np.array_equal(np.sort(idx), np.arange(ops))                       # no loss, no duplicate
        assert np.array_equal(got[c], table[c][idx])                              # records intact
        groups = idx // 64
        starts = np.flatnonzero(np.diff(np.concatenate([[-1], groups])) != 0)
        seen = groups[starts]
        assert len(seen) == (ops + 63) // 64                                      # each group in one piece
        for s, g in zip(starts, seen):
            n = min(64, ops - g * 64)
            assert np.array_equal(idx[s:s + n], np.arange(g * 64, g * 64 + n))    # in lane order
        for w in range(waves):
            mine = seen[seen % waves == w]
            assert np.array_equal(mine, np.sort(mine))                            # per-producer FIFO
    lib.ofi_amd_gin_rings_destroy(rings)


def test_device_put_gives_up_on_a_ring_nobody_drains(lib, gpu):
    nctx, cap, ops = 2, 256, 1000
    table = np.zeros((nctx, ops, 8), dtype=np.uint64)
    d_table = _gpu.to_dev(table)
    rings = make_rings(lib, nctx, cap)
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 3, 200, _gpu.stream()) == 0
    _gpu.sync()                                 # every wave leaves after its bounded wait
    assert lib.ofi_amd_gin_producer_status(rings) == -110
    view = m.GinDevRing()
    assert lib.ofi_amd_gin_rings_device_view(rings, 1, ctypes.byref(view)) == 0
    assert view.capacity == cap and view.context == 1 and view.records and view.reserve
    assert lib.ofi_amd_gin_rings_device_view(rings, 2, ctypes.byref(view)) == -22
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 0, 0, _gpu.stream()) == -22
    assert lib.ofi_amd_gin_produce_table(rings, None, ops, 1, 0, _gpu.stream()) == -22
    lib.ofi_amd_gin_rings_destroy(rings)


def test_configured_shape_checksum(lib, oracle, gpu):
    """256 contexts, 4096-entry rings, put-signal every 64th op; 20,000 ops per context here
    (the benchmark runs the full 1,000,000).  Checked through the order-sensitive checksum."""
    nctx, cap, ops = 256, 4096, 20000
    rings = make_rings(lib, nctx, cap)
    rc, stats, _, _ = produce_and_drain(lib, rings, nctx, ops, mode=0)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    assert stats.descriptors == nctx * ops and stats.signals == nctx * (ops // 64)
    assert stats.checksum == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 0, 4, 131072,
                                                                64, 1, None)
    lib.ofi_amd_gin_rings_destroy(rings)


def test_configured_shape_full_size(lib, oracle, gpu):
    """The configured run in full: 256 contexts x 1,000,000 put ops (a put-signal every 64th)
    into 4096-entry rings drained by one proxy thread; the order-sensitive checksum of all
    256,000,000 descriptors against the oracle's."""
    nctx, cap, ops = 256, 4096, 1_000_000
    rings = make_rings(lib, nctx, cap)
    rc, stats, _, _ = produce_and_drain(lib, rings, nctx, ops, mode=0)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    assert stats.descriptors == nctx * ops and stats.signals == nctx * (ops // 64)
    assert stats.checksum == oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 0, 4, 131072,
                                                                64, 1, None)
    lib.ofi_amd_gin_rings_destroy(rings)


def test_configured_shape_full_size_derived_stream(lib, oracle, gpu):
    """The same configured run with the proxy's full work per descriptor: every one of the
    256,000,000 puts goes through the iputSignal derivation (sequence number, immediate data,
    stripes, metadata), and every 224-byte wire record is folded, in order, into the checksum that
    the oracle computes over its own derivation of the same stream.  One proxy thread, as the
    configuration says; the oracle needs some fifteen seconds on one core."""
    nctx, cap, ops = 256, 4096, 1_000_000
    omrs, pmrs = _oracle.default_mrs(), _oracle.default_mrs(m.GinMr)
    rings = make_rings(lib, nctx, cap)
    comms = (m.GinComm * nctx)()
    for c in range(nctx):
        assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[c]), c % 1024, 4, 131072, 64, 1) == 0
    rc, stats, _, _ = produce_and_drain(lib, rings, nctx, ops, mode=3, comms=comms, mrs=pmrs, timeout_ms=30000)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    assert stats.descriptors == nctx * ops and stats.signals == nctx * (ops // 64)
    want = oracle.oracle_gin_stream_checksum(SEED, nctx, ops, 1, 64, 1, 1, 1, 4, 131072, 64, 1, omrs)
    assert stats.checksum == want
    lib.ofi_amd_gin_rings_destroy(rings)


def test_producer_gives_up_when_nobody_drains(lib, gpu):
    """Failure path forced from the host: more ops than slots, no consumer, a tiny spin limit.
    Every wave reaches its exit, the kernel ends, the status word reports the timeout."""
    rings = make_rings(lib, 2, 256)
    assert lib.ofi_amd_gin_produce_seeded(rings, SEED, 1000, 1, 64, 1, 1, 50, _gpu.stream()) == 0
    _gpu.sync()
    assert lib.ofi_amd_gin_producer_status(rings) == -errno.ETIMEDOUT
    stats = m.GinProxyStats()
    # the first lap (256 per ring) was published before the producers ran out of slots
    rc = lib.ofi_amd_gin_proxy_drain(rings, 256, 0, None, None, None, 0, None, 2000, ctypes.byref(stats))
    assert rc == 0 and stats.descriptors == 512
    rc = lib.ofi_amd_gin_proxy_drain(rings, 1, 0, None, None, None, 0, None, 200, ctypes.byref(stats))
    assert rc == -errno.ETIMEDOUT                    # nothing more will come
    lib.ofi_amd_gin_rings_destroy(rings)


def test_host_push_pop_ring_behaviour(lib, gpu):
    """The cases of the reference's tests/unit/mpsc_ring.cpp:16-97 on a pinned ring, through the
    host-side push/pop of the same protocol."""
    rings = make_rings(lib, 1, 256)
    d = m.GinDesc()
    assert lib.ofi_amd_gin_ring_pop(rings, 0, ctypes.byref(d)) == 0            # empty
    for i in range(256):
        assert lib.ofi_amd_gin_ring_push(rings, 0, ctypes.byref(m.GinDesc(src_off=i))) == 1
    assert lib.ofi_amd_gin_ring_push(rings, 0, ctypes.byref(m.GinDesc(src_off=999))) == 0   # all slots used
    assert lib.ofi_amd_gin_ring_pop(rings, 0, ctypes.byref(d)) == 1 and d.src_off == 0
    assert lib.ofi_amd_gin_ring_push(rings, 0, ctypes.byref(m.GinDesc(src_off=256))) == 1   # one freed, one fits
    assert lib.ofi_amd_gin_ring_push(rings, 0, ctypes.byref(m.GinDesc(src_off=999))) == 0
    for i in range(1, 257):
        assert lib.ofi_amd_gin_ring_pop(rings, 0, ctypes.byref(d)) == 1 and d.src_off == i   # FIFO
    assert lib.ofi_amd_gin_ring_pop(rings, 0, ctypes.byref(d)) == 0
    for i in range(1000):                                                        # wrap-around
        assert lib.ofi_amd_gin_ring_push(rings, 0, ctypes.byref(m.GinDesc(dst_off=i))) == 1
        assert lib.ofi_amd_gin_ring_pop(rings, 0, ctypes.byref(d)) == 1 and d.dst_off == i
        assert lib.ofi_amd_gin_ring_pop(rings, 0, ctypes.byref(d)) == 0
    assert lib.ofi_amd_gin_ring_push(rings, 1, ctypes.byref(d)) == -errno.EINVAL
    lib.ofi_amd_gin_rings_destroy(rings)


def test_rings_recover_from_a_producer_timeout(lib, oracle, gpu):
    """A time-out forced from the host (no consumer, a tiny spin limit: every wave leaves after its
    bounded wait), then ofi_amd_gin_rings_reset, then bit-exact streams on the same rings -- from
    the seeded generator and from several waves per ring through the general device put.  The
    rings restart at the consumer's position, which is not 0 for the ring that had been drained
    in part."""
    nctx, cap = 3, 256
    rings = make_rings(lib, nctx, cap)
    assert lib.ofi_amd_gin_produce_seeded(rings, SEED, 1000, 1, 64, 1, 1, 50, _gpu.stream()) == 0
    _gpu.sync()
    assert lib.ofi_amd_gin_producer_status(rings) == -errno.ETIMEDOUT
    # pop 100 records of ring 1 by hand: its consumer position moves, the other rings' do not
    d = m.GinDesc()
    for _ in range(100):
        assert lib.ofi_amd_gin_ring_pop(rings, 1, ctypes.byref(d)) == 1
    dropped = ctypes.c_uint64()
    assert lib.ofi_amd_gin_rings_reset(rings, 7, None) == -22
    assert lib.ofi_amd_gin_rings_reset(rings, 0, ctypes.byref(dropped)) == 0 and dropped.value == 256
    assert lib.ofi_amd_gin_producer_status(rings) == -errno.ETIMEDOUT      # one ring alone does not clear it
    assert lib.ofi_amd_gin_rings_reset(rings, 0xFFFFFFFF, ctypes.byref(dropped)) == 0
    assert dropped.value == 156 + 256                                      # ring 0 was already clean
    assert lib.ofi_amd_gin_producer_status(rings) == 0
    assert lib.ofi_amd_gin_ring_pop(rings, 1, ctypes.byref(d)) == 0        # nothing left in the rings

    ops = 5000
    rc, stats, descs, _ = produce_and_drain(lib, rings, nctx, ops, mode=1)
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    got = np.frombuffer(descs, dtype=np.uint64).reshape(nctx, ops, 8)
    assert np.array_equal(got, oracle_stream(oracle, nctx, ops, 64, 1, 1))
    # the general device put on the same rings: one wave per ring keeps the table order
    rng = np.random.default_rng(4)
    table = rng.integers(0, 1 << 62, (nctx, 3000, 8), dtype=np.uint64)
    d_table = _gpu.to_dev(table)
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), 3000, 1, 0, _gpu.stream()) == 0
    rc, _stats, got = drain_descs(lib, rings, nctx, 3000)
    assert rc == 0 and np.array_equal(got, table)
    # a second time-out and reset on the same rings, then host producers
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), 3000, 3, 50, _gpu.stream()) == 0
    _gpu.sync()
    assert lib.ofi_amd_gin_producer_status(rings) == -errno.ETIMEDOUT
    assert lib.ofi_amd_gin_rings_reset(rings, 0xFFFFFFFF, None) == 0
    one = m.GinDesc(1, 2, 3, 4, 5, 6, 0, 0, 2, 0, 1, 0xFFFF, 1)
    assert lib.ofi_amd_gin_ring_push(rings, 2, ctypes.byref(one)) == 1
    assert lib.ofi_amd_gin_ring_pop(rings, 2, ctypes.byref(d)) == 1 and bytes(d) == bytes(one)
    assert lib.ofi_amd_gin_ring_pop(rings, 2, ctypes.byref(d)) == 0
    lib.ofi_amd_gin_rings_destroy(rings)


def test_host_producers_threaded(lib, gpu):
    """Four CPU producer threads on one ring, the proxy loop as consumer (mpsc_ring.cpp:134-189):
    per-producer FIFO, no loss, no duplicate."""
    per, producers = 20000, 4
    rings = make_rings(lib, 1, 1024)

    def produce(p):
        i = 0
        d = m.GinDesc(context=p)
        while i < per:
            d.src_off = i
            if lib.ofi_amd_gin_ring_push(rings, 0, ctypes.byref(d)) == 1:
                i += 1

    threads = [threading.Thread(target=produce, args=(p,)) for p in range(producers)]
    for t in threads:
        t.start()
    out = (m.GinDesc * (per * producers))()
    stats = m.GinProxyStats()
    rc = lib.ofi_amd_gin_proxy_drain(rings, per * producers, 1, ctypes.cast(out, ctypes.c_void_p), None, None, 0,
                                     None, 20000, ctypes.byref(stats))
    for t in threads:
        t.join()
    assert rc == 0
    words = np.frombuffer(out, dtype=np.uint64).reshape(-1, 8)
    who = (words[:, 6] >> np.uint64(32)).astype(np.int64)
    for p in range(producers):
        assert np.array_equal(words[who == p, 0], np.arange(per, dtype=np.uint64))
    lib.ofi_amd_gin_rings_destroy(rings)


def test_bad_arguments(lib, gpu):
    r = ctypes.c_void_p()
    for nctx, cap in [(0, 256), (1, 128), (1, 300), (70000, 256)]:
        assert lib.ofi_amd_gin_rings_create(nctx, cap, ctypes.byref(r)) == -errno.EINVAL
    rings = make_rings(lib, 1, 256)
    assert lib.ofi_amd_gin_produce_seeded(rings, 1, 10, 1, 64, 3, 1, 0, None) == -errno.EINVAL
    assert lib.ofi_amd_gin_proxy_drain(rings, 1, 1, None, None, None, 0, None, 10, None) == -errno.EINVAL
    assert lib.ofi_amd_gin_proxy_drain(rings, 1, 2, None, None, None, 0, None, 10, None) == -errno.EINVAL
    lib.ofi_amd_gin_rings_destroy(rings)
