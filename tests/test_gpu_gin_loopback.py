"""The GIN path end to end on one GPU, in process: device-side puts -> rings -> host proxy ->
wire records -> (loop-back "network": RDMA writes become device copies, completions and
metadata go to the receiver out of order, ACKs return) -> signal counters in HBM.

What the reference checks with two processes and a NIC (tests/functional/rma.cpp: payload
bytes and signal counters at the target) is checked here bit for bit against a plain numpy
replay of the same operations; the wire-level bookkeeping must also close: every op
retired, every signal delivered once, the sender's window never stuck."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

SIG_BASE = 0x7F5500000000
N_SLOTS = 64


def build_ops(rng, nctx, ops, src_bytes, max_size):
    """table[ctx][i] of 8 u64 words (ofi_amd_gin_desc_t) with disjoint destinations"""
    table = np.zeros((nctx, ops, 8), dtype=np.uint64)
    dst_pos = 0
    replay = []
    for c in range(nctx):
        for i in range(ops):
            kind = rng.random()
            if kind < 0.08:
                size = 0                                           # signal only
            elif kind < 0.6:
                size = int(rng.integers(1, 4096))
            else:
                size = int(2 ** rng.uniform(3, np.log2(max_size)))
            src_off = int(rng.integers(0, src_bytes - size))
            dst_off = dst_pos + int(rng.integers(0, 24))           # arbitrary alignment
            dst_pos = dst_off + size + int(rng.integers(0, 8))
            signal = size == 0 or (i % 5) == 4
            sop = (1 if rng.random() < 0.5 else 2) if signal else 0
            sval = int(rng.integers(1, 1 << 40)) if sop == 2 else 0
            slot = int(rng.integers(0, N_SLOTS))
            flags = int(rng.integers(0, 2))                        # doorbell aggregation hint
            table[c, i] = [src_off, dst_off, size, 8 * slot if sop else 0, sval,
                           1 | (sop << 32), flags | (c << 32),
                           0 | (1 << 16) | ((2 if sop else 0xFFFF) << 32) | ((2 if sop else 1) << 48)]
            replay.append((src_off, dst_off, size, sop, sval, slot))
    return table, replay, dst_pos + 64


@pytest.mark.parametrize("nctx,ops,waves,reorder,batch,max_size,sq_depth", [
    (1, 300, 1, 0, 64, 70_000, 0),
    (2, 1200, 2, 16, 64, 70_000, -1),     # the copies on the producers' own stream: they start when the producers end
    (4, 1500, 3, 37, 512, 300_000, 0),
    (3, 6000, 2, 500, 4096, 40_000, 0),   # more than 4096 ops per context in flight at times: ACKs matter
    (4, 6000, 2, 64, 1024, 600_000, 8),   # send queues of 8 entries per rail, a progress call every 16 ops
    (2, 3000, 1, 0, 256, 300_000, 1),     # one entry per rail: most posts between two progress calls are refused
])
def test_puts_and_signals_arrive_bit_exact(lib, gpu, nctx, ops, waves, reorder, batch, max_size, sq_depth):
    rng = np.random.default_rng(nctx * 1000 + ops)
    src_bytes = 32 << 20
    src = rng.integers(0, 256, src_bytes, dtype=np.uint8)
    table, replay, dst_bytes = build_ops(rng, nctx, ops, src_bytes, max_size)
    d_src = _gpu.to_dev(src)
    d_dst = torch.full((dst_bytes,), 0xEE, dtype=torch.uint8, device="cuda")
    start = rng.integers(0, 1 << 63, N_SLOTS, dtype=np.uint64)
    d_cnt = _gpu.to_dev(start)
    d_table = _gpu.to_dev(table)

    mrs = (m.GinMr * 3)()
    mrs[0].local_base = d_src.data_ptr()                       # source MR: local address
    mrs[1].remote_address_offset = d_dst.data_ptr()            # target MR: where writes land
    mrs[2].remote_address = SIG_BASE                           # signal MR: the address the peer knows
    for i in range(3):
        for r in range(4):
            mrs[i].key[r] = 0x100 * (i + 1) + r
    comms = (m.GinComm * nctx)()
    for c in range(nctx):
        assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[c]), 100 + c, 4, 131072, 64, 0) == 0
    regions = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, 8 * N_SLOTS, d_cnt.data_ptr()))
    rings = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rings_create(nctx, 1024, ctypes.byref(rings)) == 0

    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, waves, 0, _gpu.stream()) == 0
    stats = m.GinLoopbackStats()
    # the copies and signal updates go on their own stream: the producer kernel occupies the first
    side = torch.cuda.Stream()
    # sq_depth -1: the run's launches go on the stream the producers run on, which is what two streams that
    # share a hardware queue amount to.  No launch starts before the producers have finished, and they finish
    # only when the run has drained their rings: the run adds table sets instead of waiting for a sentinel.
    same_stream = sq_depth < 0
    sq_depth = max(sq_depth, 0)
    rc = lib.ofi_amd_gin_loopback_run(rings, ops, ctypes.cast(comms, ctypes.c_void_p),
                                      ctypes.cast(mrs, ctypes.c_void_p), len(mrs), regions, 1, reorder, batch,
                                      sq_depth, 16 if sq_depth else 1, 20000,
                                      _gpu.stream() if same_stream else ctypes.c_void_p(side.cuda_stream),
                                      ctypes.byref(stats))
    torch.cuda.synchronize()
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0
    if same_stream:
        assert stats.table_sets_added > 0

    # payload: a plain replay of the puts on the host
    want = np.full(dst_bytes, 0xEE, dtype=np.uint8)
    counters = [int(x) for x in start]
    n_signals = 0
    for src_off, dst_off, size, sop, sval, slot in replay:
        want[dst_off:dst_off + size] = src[src_off:src_off + size]
        if sop:
            counters[slot] = (counters[slot] + (1 if sop == 1 else sval)) % (1 << 64)
            n_signals += 1
    assert np.array_equal(d_dst.cpu().numpy(), want)
    assert [int(x) for x in _gpu.to_host(d_cnt, np.uint64)] == counters

    # bookkeeping closes
    total = nctx * ops
    assert stats.descriptors == total and stats.signals == n_signals
    assert stats.bytes == sum(r[2] for r in replay)
    assert stats.writes >= sum(1 for r in replay if r[2]) and stats.copy_entries >= stats.writes
    assert 0 < stats.work_items <= n_signals          # same-slot neighbours may have been folded
    for c in range(nctx):
        assert comms[c].tx_head == ops % 16384
        outstanding = (comms[c].tx_head - comms[c].tx_tail) & 0x3FFF
        assert outstanding < 8192
        if ops > 4096 + 64:
            assert outstanding < ops                  # ACKs did come back
    if ops > 4096 + 64:
        assert stats.acks > 0
    # every post completed on the initiator: one per RDMA write, metadata message and ACK
    assert stats.tx_completions == stats.writes + stats.signals + stats.acks
    if sq_depth:
        # bounded send queues: posts were refused, queued and posted again by progress calls, and
        # everything above still holds
        assert stats.posts_refused > (2000 if sq_depth == 8 else 3000), stats.posts_refused
        assert stats.post_retries >= stats.posts_refused and stats.pending_max > 1
    else:
        assert stats.posts_refused == 0 and stats.post_retries == 0
    assert _gpu.fetch_async_errors(lib) == 0
    lib.ofi_amd_gin_rings_destroy(rings)


def test_gets_land_bit_exact_beside_puts(lib, gpu):
    """Every fourth operation is a get (iget, src/rdma/gin/nccl_ofi_gin.cpp:879-939): its reads come
    back as copies from the peer's registration into a local landing buffer.  Gets use the same
    scheduler as the puts, but no sequence number: the window counts the puts only, the receiver
    hears of the puts only, and every read completes on the initiator."""
    rng = np.random.default_rng(4242)
    nctx, ops = 3, 2000
    src_bytes = 16 << 20
    src = rng.integers(0, 256, src_bytes, dtype=np.uint8)
    remote = rng.integers(0, 256, src_bytes, dtype=np.uint8)      # what the gets read
    table, replay, dst_bytes = build_ops(rng, nctx, ops, src_bytes, 300_000)
    land_pos, gets, want_reads = 0, [], 0
    for c in range(nctx):
        for i in range(3, ops, 4):
            size = int(2 ** rng.uniform(0, 19.5)) if rng.random() < 0.9 else 0
            remote_off = int(rng.integers(0, src_bytes - size))
            local_off = land_pos + int(rng.integers(0, 24))
            land_pos = local_off + size + int(rng.integers(0, 8))
            # remote handle 3, local handle 4, kind 3
            table[c, i] = [remote_off, local_off, size, 0, 0, 1, (c << 32), 3 | (4 << 16) | (0xFFFF << 32) | (3 << 48)]
            replay[c * ops + i] = None
            gets.append((remote_off, local_off, size))
            want_reads += 1 if size <= 131072 else (2 if size <= 393216 else 4)
    d_src, d_remote = _gpu.to_dev(src), _gpu.to_dev(remote)
    d_dst = torch.full((dst_bytes,), 0xEE, dtype=torch.uint8, device="cuda")
    d_land = torch.full((land_pos + 64,), 0xDD, dtype=torch.uint8, device="cuda")
    start = rng.integers(0, 1 << 63, N_SLOTS, dtype=np.uint64)
    d_cnt = _gpu.to_dev(start)
    d_table = _gpu.to_dev(table)

    mrs = (m.GinMr * 5)()
    mrs[0].local_base = d_src.data_ptr()
    mrs[1].remote_address_offset = d_dst.data_ptr()
    mrs[2].remote_address = SIG_BASE
    mrs[3].remote_address_offset = d_remote.data_ptr()            # the peer's memory the gets read
    mrs[4].local_base = d_land.data_ptr()                          # where they land
    for i in range(5):
        for r in range(4):
            mrs[i].key[r] = 0x100 * (i + 1) + r
    comms = (m.GinComm * nctx)()
    for c in range(nctx):
        assert lib.ofi_amd_gin_comm_init(ctypes.byref(comms[c]), 100 + c, 4, 131072, 64, 0) == 0
    regions = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, 8 * N_SLOTS, d_cnt.data_ptr()))
    rings = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rings_create(nctx, 1024, ctypes.byref(rings)) == 0
    assert lib.ofi_amd_gin_produce_table(rings, d_table.data_ptr(), ops, 2, 0, _gpu.stream()) == 0
    stats = m.GinLoopbackStats()
    side = torch.cuda.Stream()
    rc = lib.ofi_amd_gin_loopback_run(rings, ops, ctypes.cast(comms, ctypes.c_void_p),
                                      ctypes.cast(mrs, ctypes.c_void_p), len(mrs), regions, 1, 50, 512, 8, 16,
                                      20000, ctypes.c_void_p(side.cuda_stream), ctypes.byref(stats))
    torch.cuda.synchronize()
    assert rc == 0 and lib.ofi_amd_gin_producer_status(rings) == 0

    want = np.full(dst_bytes, 0xEE, dtype=np.uint8)
    counters = [int(x) for x in start]
    n_signals = n_puts = 0
    for r in replay:
        if r is None:
            continue
        src_off, dst_off, size, sop, sval, slot = r
        n_puts += 1
        want[dst_off:dst_off + size] = src[src_off:src_off + size]
        if sop:
            counters[slot] = (counters[slot] + (1 if sop == 1 else sval)) % (1 << 64)
            n_signals += 1
    want_land = np.full(land_pos + 64, 0xDD, dtype=np.uint8)
    for remote_off, local_off, size in gets:
        want_land[local_off:local_off + size] = remote[remote_off:remote_off + size]
    assert np.array_equal(d_dst.cpu().numpy(), want)
    assert np.array_equal(d_land.cpu().numpy(), want_land)
    assert [int(x) for x in _gpu.to_host(d_cnt, np.uint64)] == counters

    assert stats.descriptors == nctx * ops and stats.signals == n_signals
    assert stats.reads == want_reads and stats.flush_reads == 4     # the fence behind the gets: one read per rail
    assert stats.bytes == sum(r[2] for r in replay if r) + sum(g[2] for g in gets)
    for c in range(nctx):
        assert comms[c].tx_head == n_puts // nctx                 # the puts only
    assert stats.tx_completions == stats.writes + stats.signals + stats.acks + stats.reads + stats.flush_reads
    assert stats.posts_refused > 0
    assert _gpu.fetch_async_errors(lib) == 0
    lib.ofi_amd_gin_rings_destroy(rings)


def test_copy_table_matches_a_host_replay(lib, gpu):
    """The loop-back's data mover by itself: address triples at any alignment and length."""
    rng = np.random.default_rng(5)
    n = 3000
    src = rng.integers(0, 256, 8 << 20, dtype=np.uint8)
    lens = np.concatenate([rng.integers(0, 300, n // 2), (2 ** rng.uniform(3, 16.5, n - n // 2)).astype(np.int64)])
    lens = lens.astype(np.uint32)
    src_off = rng.integers(0, len(src) - int(lens.max()), n).astype(np.uint64)
    gaps = rng.integers(0, 20, n).astype(np.uint64)
    dst_off = (np.cumsum(lens.astype(np.uint64) + gaps) - lens.astype(np.uint64)).astype(np.uint64)
    total = int(dst_off[-1] + lens[-1]) + 32
    d_src = _gpu.to_dev(src)
    d_dst = torch.full((total,), 0x77, dtype=torch.uint8, device="cuda")
    a_src = _gpu.to_dev(src_off + np.uint64(d_src.data_ptr()))
    a_dst = _gpu.to_dev(dst_off + np.uint64(d_dst.data_ptr()))
    d_len = _gpu.to_dev(lens)
    assert lib.ofi_amd_copy_table(a_src.data_ptr(), a_dst.data_ptr(), d_len.data_ptr(), n, _gpu.stream()) == 0
    _gpu.sync()
    want = np.full(total, 0x77, dtype=np.uint8)
    for s, d, l in zip(src_off, dst_off, lens):
        want[int(d):int(d) + int(l)] = src[int(s):int(s) + int(l)]
    assert np.array_equal(d_dst.cpu().numpy(), want)
    assert lib.ofi_amd_copy_table(None, a_dst.data_ptr(), d_len.data_ptr(), 1, _gpu.stream()) == -22
    assert lib.ofi_amd_copy_table(a_src.data_ptr(), a_dst.data_ptr(), d_len.data_ptr(), 0, _gpu.stream()) == 0


def test_copy_table_in_pieces_matches_a_host_replay(lib, gpu):
    """The same table through the launch that gives every 8 KiB of an entry its own wavefront: a few
    long entries (up to 5 MiB) among many short and empty ones, any alignment; lengths at and
    round the 8 KiB piece size; a maximum that is not a multiple of the piece size; an entry longer
    than the stated maximum is copied up to it and reported."""
    rng = np.random.default_rng(7)
    edge = [0, 1, 63, 64, 65, 8191, 8192, 8193, 16383, 16384, 16385, 3 * 8192 + 100]
    lens = np.concatenate([rng.integers(0, 300, 400), (2 ** rng.uniform(3, 22.3, 200)).astype(np.int64),
                           np.array(edge * 3)]).astype(np.uint32)
    n = len(lens)
    src = rng.integers(0, 256, 32 << 20, dtype=np.uint8)
    src_off = rng.integers(0, len(src) - int(lens.max()), n).astype(np.uint64)
    gaps = rng.integers(0, 70, n).astype(np.uint64)
    dst_off = (np.cumsum(lens.astype(np.uint64) + gaps) - lens.astype(np.uint64)).astype(np.uint64)
    total = int(dst_off[-1] + lens[-1]) + 128
    d_src = _gpu.to_dev(src)
    a_src = _gpu.to_dev(src_off + np.uint64(d_src.data_ptr()))
    d_len = _gpu.to_dev(lens)
    want = np.full(total, 0x77, dtype=np.uint8)
    for s, d, l in zip(src_off, dst_off, lens):
        want[int(d):int(d) + int(l)] = src[int(s):int(s) + int(l)]
    for max_len in (int(lens.max()), int(lens.max()) + 12345, 0xFFFFFFFF // 64):
        d_dst = torch.full((total,), 0x77, dtype=torch.uint8, device="cuda")
        a_dst = _gpu.to_dev(dst_off + np.uint64(d_dst.data_ptr()))
        assert lib.ofi_amd_copy_table_pieces(a_src.data_ptr(), a_dst.data_ptr(), d_len.data_ptr(), n, max_len,
                                             _gpu.stream()) == 0
        _gpu.sync()
        assert np.array_equal(d_dst.cpu().numpy(), want), max_len
        assert _gpu.fetch_async_errors(lib) == 0
    # a stated maximum that is not a multiple of the 8 KiB piece: longer entries stop at exactly that
    # many bytes (also those that would still fit the last piece) and bit 3 is set; 0 copies nothing
    for max_len in (20000, 8192, 100, 0):
        d_dst = torch.full((total,), 0x77, dtype=torch.uint8, device="cuda")
        a_dst = _gpu.to_dev(dst_off + np.uint64(d_dst.data_ptr()))
        assert lib.ofi_amd_copy_table_pieces(a_src.data_ptr(), a_dst.data_ptr(), d_len.data_ptr(), n, max_len,
                                             _gpu.stream()) == 0
        _gpu.sync()
        cut = np.full(total, 0x77, dtype=np.uint8)
        for s, d, l in zip(src_off, dst_off, lens):
            l = min(int(l), max_len)
            cut[int(d):int(d) + l] = src[int(s):int(s) + l]
        assert np.array_equal(d_dst.cpu().numpy(), cut), max_len
        assert _gpu.fetch_async_errors(lib) == 8
    # every entry within the bound although longer than the bound rounded down to pieces: no report
    short = np.minimum(lens, 20000).astype(np.uint32)
    d_short = _gpu.to_dev(short)
    d_dst = torch.full((total,), 0x77, dtype=torch.uint8, device="cuda")
    a_dst = _gpu.to_dev(dst_off + np.uint64(d_dst.data_ptr()))
    assert lib.ofi_amd_copy_table_pieces(a_src.data_ptr(), a_dst.data_ptr(), d_short.data_ptr(), n, 20000,
                                         _gpu.stream()) == 0
    _gpu.sync()
    assert _gpu.fetch_async_errors(lib) == 0
    assert lib.ofi_amd_copy_table_pieces(None, a_dst.data_ptr(), d_len.data_ptr(), 1, 64, _gpu.stream()) == -22
    assert lib.ofi_amd_copy_table_pieces(a_src.data_ptr(), a_dst.data_ptr(), d_len.data_ptr(), 0, 64, _gpu.stream()) == 0
    assert lib.ofi_amd_copy_table_pieces(a_src.data_ptr(), a_dst.data_ptr(), d_len.data_ptr(), 1 << 20, 0xFFFFFFFF,
                                         _gpu.stream()) == -7   # 2^20 entries x 2^19 pieces: split the table


def test_bad_arguments(lib, gpu):
    rings = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rings_create(1, 256, ctypes.byref(rings)) == 0
    comms = (m.GinComm * 1)()
    mrs = (m.GinMr * 3)()
    regions = (m.GinSignalRegion * 1)()
    stats = m.GinLoopbackStats()
    args = (ctypes.cast(comms, ctypes.c_void_p), ctypes.cast(mrs, ctypes.c_void_p), 3, regions)
    assert lib.ofi_amd_gin_loopback_run(None, 1, *args, 1, 0, 64, 0, 1, 10, None, ctypes.byref(stats)) == -22
    assert lib.ofi_amd_gin_loopback_run(rings, 1, *args, 0, 0, 64, 0, 1, 10, None, ctypes.byref(stats)) == -22
    assert lib.ofi_amd_gin_loopback_run(rings, 1, *args, 1, 0, 0, 0, 1, 10, None, ctypes.byref(stats)) == -22
    assert lib.ofi_amd_gin_loopback_run(rings, 1, *args, 1, 5000, 64, 0, 1, 10, None, ctypes.byref(stats)) == -22
    lib.ofi_amd_gin_rings_destroy(rings)
