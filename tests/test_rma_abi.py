"""The data-path members of ncclRma_v15_t (rma_v15.h:43-56) as this library exports them
(include/ofi_amd_rma_abi.h), driven the way the reference's tests/functional/rma.cpp:212-375 drives
the plugin: 64 puts and 64 put-signals to a peer without a progress call in between, then
"test the oldest request, progress if it is not done" until none is left; the target sees the
signal count reach 64.  Two ranks in one process: the initiator posts into the library's
in-process fabric, the test plays the wire and the target's receiver.  Runs on the CPU.

What is checked: the posts equal the oracle's derivation of the same argument stream (rail,
addresses, lengths, keys, immediate data, metadata words), requests complete exactly once,
return codes follow nccl_net_ofi_retval_translate, and the scheduler and the doorbell pin are
shared by all ranks of a context while sequence numbers are per rank."""
import ctypes

import numpy as np
import pytest

import _oracle
import aws_ofi_nccl_amd as m

ncclSuccess, ncclSystemError, ncclInternalError = 0, 2, 3
WRITE, META, ACK, READ = 1, 2, 3, 4
SIGNAL_INC, SIGNAL_ADD = 1, 2
AGGREGATE = 1                       # ncclRmaOptFlagsAggregateRequests
NRANKS = 3


def mr_arrays(i):
    """Registration i as every rank sees it: the addresses of tests/_oracle.default_mrs, shifted per rank."""
    addr = np.array([0x7E0000000000 + (i << 32) + (r << 24) for r in range(NRANKS)], dtype=np.uint64)
    off = addr.copy() if i != 1 else np.array([r << 24 for r in range(NRANKS)], dtype=np.uint64)
    keys = np.array([[0x1000 * (i + 1) + 0x100 * r + k for k in range(4)] for r in range(NRANKS)], dtype=np.uint64)
    return 0x7F0000000000 + (i << 32), addr, off, keys


class Initiator:
    def __init__(self, lib, rails=4, sq_depth=512, pool=65536, wait_ms=50):
        self.lib = lib
        self.fab = ctypes.c_void_p()
        assert lib.ofi_amd_loopfab_create(rails, sq_depth, ctypes.byref(self.fab)) == 0
        self.ops = m.GinFabricOps()
        assert lib.ofi_amd_loopfab_ops(self.fab, ctypes.byref(self.ops)) == 0
        self.ctx = ctypes.c_void_p()
        assert lib.ofi_amd_rma_ctx_create(NRANKS, rails, 131072, 64, ctypes.byref(self.ops), pool, wait_ms,
                                          ctypes.byref(self.ctx)) == 0
        self.mrs, self.tables = [], []
        for i in range(3):
            base, addr, off, keys = mr_arrays(i)
            h = ctypes.c_void_p()
            assert lib.ofi_amd_rma_mr_create(self.ctx, base, addr.ctypes.data, off.ctypes.data, keys.ctypes.data,
                                             ctypes.byref(h)) == 0
            self.mrs.append(h)
            self.tables.append((base, addr, off, keys))
        self.posts = (m.GinPost * 64)()

    def oracle_table(self, rank):
        """The same registrations as the oracle's three-entry table for one target rank."""
        t = (_oracle.GinMr * 3)()
        for i, (base, addr, off, keys) in enumerate(self.tables):
            t[i].local_base, t[i].remote_address, t[i].remote_address_offset = base, int(addr[rank]), int(off[rank])
            for k in range(4):
                t[i].key[k] = int(keys[rank][k])
        return t

    def wire(self):
        """Everything the fabric has transmitted since the last call, in transmission order."""
        out = []
        while True:
            n = self.lib.ofi_amd_loopfab_take_transmitted(self.fab, self.posts, 64)
            for i in range(n):
                p = self.posts[i]
                out.append((p.kind, p.rail, p.peer, p.imm, p.src, p.len, p.dest, p.key, tuple(p.msg)))
            if n < 64:
                return out

    def close(self):
        for h in self.mrs:
            assert self.lib.ofi_amd_rma_mr_destroy(h) == 0
        assert self.lib.ofi_amd_rma_ctx_destroy(self.ctx) == 0
        assert self.lib.ofi_amd_loopfab_destroy(self.fab) == 0


def expected_posts(oracle, oc, table, desc_fields):
    """The oracle's derivation of one operation as the posts it stands for: writes in stripe order,
    then the metadata message."""
    d = _oracle.GinDesc(*desc_fields)
    w = _oracle.GinWire()
    assert oracle.oracle_gin_iput_signal(ctypes.byref(oc), table, ctypes.byref(d), ctypes.byref(w)) == 0
    posts = [(WRITE, w.writes[k].rail, w.imm, w.writes[k].src, w.writes[k].len, w.writes[k].dest, w.writes[k].key)
             for k in range(w.num_writes)]
    if w.has_meta:
        posts.append((META, w.meta_rail, tuple(w.meta)))
    return posts


@pytest.mark.parametrize("size,stripes", [(5000, 1), (4 << 20, 4)])
def test_sixty_four_puts_and_sixty_four_put_signals_then_poll(lib, oracle, size, stripes):
    """size 5000 is the reference test's SEND_SIZE (tests/functional/functional_test.h:30): one write
    per operation; 4 MiB takes a stripe on each of the four rails."""
    ini = Initiator(lib)
    rank = 1
    oc = _oracle.GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(oc), rank, 4, 131072, 64, 0)
    table = ini.oracle_table(rank)
    rx = ctypes.c_void_p()
    ids = (ctypes.c_uint32 * 1)(rank)
    assert lib.ofi_amd_gin_rx_create(1, ids, ctypes.byref(rx)) == 0
    requests, want = [], []
    for i in range(64):
        req = ctypes.c_void_p()
        assert lib.ofi_amd_rma_iput(ini.ctx, 0, 0, ini.mrs[0], size, 0, ini.mrs[1], rank, 0, ctypes.byref(req)) == 0
        assert req.value
        requests.append(req)
        want += expected_posts(oracle, oc, table, (0, 0, size, 0, 0, rank, 0, 0, 0, 0, 1, 0xFFFF, 1))
    for i in range(64):
        req = ctypes.c_void_p()
        assert lib.ofi_amd_rma_iputSignal(ini.ctx, 0, 0, ini.mrs[0], size, 0, ini.mrs[1], rank, 8, ini.mrs[2], 1,
                                          SIGNAL_INC, True, 0, ctypes.byref(req)) == 0
        requests.append(req)
        want += expected_posts(oracle, oc, table, (0, 0, size, 8, 1, rank, SIGNAL_INC, 0, 0, 0, 1, 2, 2))
    assert len(set(r.value for r in requests)) == 128     # every open request has its own handle
    # nothing completes before the first progress call
    done = ctypes.c_int(-1)
    assert lib.ofi_amd_rma_test(ini.ctx, requests[0], ctypes.byref(done)) == 0 and done.value == 0
    # the wire: what left the initiator equals the oracle's records, operation by operation per rail
    got = ini.wire()
    by_rail = lambda posts, pick: [[pick(p) for p in posts if p[1] == r] for r in range(4)]
    assert by_rail(got, lambda p: (p[0], p[1], p[3], p[4], p[5], p[6], p[7]) if p[0] == WRITE else (p[0], p[1], p[8])) == \
        by_rail(want, lambda p: p)
    assert sum(1 for p in got if p[0] == WRITE) == 128 * stripes and sum(1 for p in got if p[0] == META) == 64
    # the target: completions in the order they were transmitted; its ACKs go back to the initiator
    acks = (m.GinAck * 64)()
    work = (m.GinSignalWork * 256)()
    delivered = 0
    for p in got:
        if p[0] == WRITE:
            assert lib.ofi_amd_gin_rx_write_completion(rx, 0, p[3]) == 0
        else:
            meta = (ctypes.c_uint64 * 4)(*p[8])
            assert lib.ofi_amd_gin_rx_metadata(rx, 0, meta) == 0
        for k in range(lib.ofi_amd_gin_rx_take_acks(rx, acks, 64)):
            assert lib.ofi_amd_rma_ack_received(ini.ctx, rank, acks[k].msg) == 0
    n_work = lib.ofi_amd_gin_rx_take_work(rx, work, 256)
    for k in range(n_work):
        assert work[k].base == int(ini.tables[2][1][rank]) and work[k].offset == 8
        delivered += work[k].value
    assert delivered == 64                                # "signal_buff reaches the designated signal value"
    # poll_request_completion (tests/functional/rma.cpp:12-26): test the oldest, progress if not done
    polls = 0
    while requests:
        assert lib.ofi_amd_rma_test(ini.ctx, requests[0], ctypes.byref(done)) == 0
        if done.value:
            finished = requests.pop(0)
            # a completed request is back in the pool: testing it again is an error, not a second "done"
            assert lib.ofi_amd_rma_test(ini.ctx, finished, ctypes.byref(done)) == ncclInternalError
        else:
            assert lib.ofi_amd_rma_rmaProgress(ini.ctx) == 0
        polls += 1
        assert polls < 10000
    st = m.GinTxStats()
    assert lib.ofi_amd_rma_tx_stats(ini.ctx, ctypes.byref(st)) == 0
    assert st.requests == 0 and st.completions == 128 * stripes + 64 and st.posts == st.completions
    peer = lib.ofi_amd_rma_peer_state(ini.ctx, rank).contents
    assert peer.tx_head == oc.tx_head == 128 and peer.tx_tail == oc.tx_tail
    assert peer.consecutive_puts_without_ack == oc.consecutive_puts_without_ack
    lib.ofi_amd_gin_rx_destroy(rx)
    ini.close()


def test_scheduler_and_pin_are_one_for_all_ranks_sequence_numbers_per_rank(lib):
    """Small puts take one rail each from the endpoint's round-robin counter, whichever rank they go
    to (the reference has one scheduler per endpoint, src/rdma/gin/nccl_ofi_gin.cpp:590); the
    sequence number in the immediate data counts per target rank (rank_comms[dst_rank], :587)."""
    ini = Initiator(lib)
    rails, seqs = [], {1: [], 2: []}
    for i in range(12):
        rank = 1 + i % 2
        req = ctypes.c_void_p()
        assert lib.ofi_amd_rma_iput(ini.ctx, 0, 64 * i, ini.mrs[0], 32, 64 * i, ini.mrs[1], rank, 0,
                                    ctypes.byref(req)) == 0
    for p in ini.wire():
        assert p[0] == WRITE and p[5] == 32
        rails.append(p[1])
        seqs[p[2]].append((p[3] >> 11) & 0x1FFF)
        # the key is the target rank's for the rail taken, the destination its address offset + dstOff
        assert p[7] == 0x2000 + 0x100 * p[2] + p[1]
        assert p[6] == (p[2] << 24) + 64 * (len(rails) - 1)
        assert (p[3] >> 1) & 0x3FF == p[2]                  # comm id of the peer's state = its rank
    assert rails == [0, 1, 2, 3] * 3
    assert seqs == {1: list(range(6)), 2: list(range(6))}
    # an aggregated run pins one rail across ranks: 15 deferred writes and the 16th rings
    for i in range(16):
        req = ctypes.c_void_p()
        assert lib.ofi_amd_rma_iput(ini.ctx, 0, 0, ini.mrs[0], 32, 0, ini.mrs[1], 1 + i % 2, AGGREGATE,
                                    ctypes.byref(req)) == 0
        sent = ini.wire()
        assert (len(sent) == 16 and len(set(p[1] for p in sent)) == 1) if i == 15 else sent == []
    shared = lib.ofi_amd_rma_peer_state(ini.ctx, 0xFFFFFFFF).contents
    assert shared.pinned_rail_id == -1 and shared.sched.rr_small_counter == (12 + 16) % 4
    ini.close()


def test_get_posts_reads_and_flush_waits_for_the_sentinel(lib):
    ini = Initiator(lib)
    req = ctypes.c_void_p()
    size = 300000                                           # 3 stripes asked, 2 taken with 4 rails (131072-byte minimum)
    assert lib.ofi_amd_rma_iget(ini.ctx, 0, 4096, ini.mrs[1], size, 128, ini.mrs[0], 2, 0, ctypes.byref(req)) == 0
    reads = ini.wire()
    assert [p[0] for p in reads] == [READ, READ] and sum(p[5] for p in reads) == size
    base_local, remote_off = ini.tables[0][0], int(ini.tables[1][2][2])
    at = 0
    for p in reads:
        assert p[4] == base_local + 128 + at and p[6] == remote_off + 4096 + at     # local landing, remote source
        assert p[7] == 0x2000 + 0x200 + p[1] and p[3] == 0
        at += p[5]
    # a get takes no sequence number and no room in the window
    assert lib.ofi_amd_rma_peer_state(ini.ctx, 2).contents.tx_head == 0
    done = ctypes.c_int()
    assert lib.ofi_amd_rma_rmaProgress(ini.ctx) == 0
    assert lib.ofi_amd_rma_test(ini.ctx, req, ctypes.byref(done)) == 0 and done.value == 1
    # iflush: refused until its buffers are known; then one 64-byte read per rail, done by sentinel
    assert lib.ofi_amd_rma_iflush(ini.ctx, 0, None, 0, ctypes.byref(req)) == ncclInternalError
    slots = np.zeros(4 * 8, dtype=np.uint64)
    sentinel = 0xDEADBEEFDEADBEEF
    assert lib.ofi_amd_rma_set_flush_buffers(ini.ctx, slots.ctypes.data, 0x7F4400000000, sentinel) == 0
    slots[:] = 7
    assert lib.ofi_amd_rma_iflush(ini.ctx, 0, ini.mrs[0], 1, ctypes.byref(req)) == 0
    assert not slots[::8].any()                             # the slots are cleared before the reads go out
    reads = ini.wire()
    assert [(p[0], p[1], p[5], p[6]) for p in reads] == [(READ, r, 64, 0x7F4400000000) for r in range(4)]
    assert [p[4] for p in reads] == [slots.ctypes.data + 64 * r for r in range(4)]
    assert lib.ofi_amd_rma_rmaProgress(ini.ctx) == 0       # the reads' own completions do not finish the flush
    assert lib.ofi_amd_rma_test(ini.ctx, req, ctypes.byref(done)) == 0 and done.value == 0
    slots[0::8][:3] = sentinel
    assert lib.ofi_amd_rma_test(ini.ctx, req, ctypes.byref(done)) == 0 and done.value == 0
    slots[24] = sentinel
    assert lib.ofi_amd_rma_test(ini.ctx, req, ctypes.byref(done)) == 0 and done.value == 1
    ini.close()


def test_return_codes_follow_the_reference_translation(lib):
    ini = Initiator(lib, pool=40000, wait_ms=30)
    req = ctypes.c_void_p(1)
    put = lambda rank, size=8, src=0, dst=1: lib.ofi_amd_rma_iput(
        ini.ctx, 0, 0, ini.mrs[src] if src is not None else None, size, 0,
        ini.mrs[dst] if dst is not None else None, rank, 0, ctypes.byref(req))
    # -EINVAL -> ncclInternalError ("invalid arguments to plugin calls should return ncclInternalError")
    assert put(NRANKS) == ncclInternalError and req.value is None
    assert put(1, src=None) == ncclInternalError and put(1, dst=None) == ncclInternalError
    assert lib.ofi_amd_rma_iput(None, 0, 0, ini.mrs[0], 8, 0, ini.mrs[1], 1, 0, ctypes.byref(req)) == ncclInternalError
    assert lib.ofi_amd_rma_iputSignal(ini.ctx, 0, 0, ini.mrs[0], 8, 0, ini.mrs[1], 1, 0, ini.mrs[2], 1, 3, True, 0,
                                      ctypes.byref(req)) == ncclInternalError          # no such signal op
    assert lib.ofi_amd_rma_rmaProgress(None) == ncclInternalError
    done = ctypes.c_int()
    bogus = ctypes.c_int32(5)
    assert lib.ofi_amd_rma_test(ini.ctx, ctypes.byref(bogus), ctypes.byref(done)) == ncclInternalError
    # a handle of another context is refused
    other = Initiator(lib)
    assert lib.ofi_amd_rma_iput(ini.ctx, 0, 0, other.mrs[0], 8, 0, ini.mrs[1], 1, 0, ctypes.byref(req)) == \
        ncclInternalError
    other.close()
    # a signal-only operation needs no data registrations (size 0), as in the reference
    assert lib.ofi_amd_rma_iputSignal(ini.ctx, 0, 0, None, 0, 0, None, 1, 16, ini.mrs[2], 5, SIGNAL_ADD, True, 0,
                                      ctypes.byref(req)) == 0
    sent = ini.wire()
    assert len(sent) == 1 and sent[0][0] == META and sent[0][8][2:] == (16, 5)
    # the window towards one rank holds 8192 operations; with no ACK coming back the next put
    # gives up after window_wait_ms of progress calls: any other errno -> ncclSystemError
    for i in range(8191):
        assert put(1) == 0
        if i % 256 == 0:
            ini.wire()
            assert lib.ofi_amd_rma_rmaProgress(ini.ctx) == 0
    assert put(1) == ncclSystemError and req.value is None
    assert put(2) == 0                                      # another rank's window is its own
    # an ACK for half of them makes room again
    assert lib.ofi_amd_rma_ack_received(ini.ctx, 1, int(lib.ofi_amd_gin_ack_msg(1, 4096))) == 0
    assert put(1) == 0
    assert lib.ofi_amd_rma_peer_state(ini.ctx, 1).contents.tx_tail == 4096
    ini.close()


def test_a_full_window_opens_when_the_ack_arrives_inside_a_progress_call(lib):
    """await_tx_window (src/rdma/gin/nccl_ofi_gin.cpp:518-537): a put towards a rank whose window is
    full keeps calling progress; the ACK that makes room is a receive completion handled inside that
    progress call (handle_ack_completion, :1843-1869).  Here the CQ callback plays it: on its third
    call during the wait it hands the ACK to ofi_amd_rma_ack_received, and the put that was waiting
    goes through with the next sequence number (its post queues up behind those the full send
    queues have refused so far)."""
    ini = Initiator.__new__(Initiator)
    ini.lib = lib
    ini.fab = ctypes.c_void_p()
    assert lib.ofi_amd_loopfab_create(4, 512, ctypes.byref(ini.fab)) == 0
    inner = m.GinFabricOps()
    assert lib.ofi_amd_loopfab_ops(ini.fab, ctypes.byref(inner)) == 0
    state = {"armed": False, "calls": 0, "ctx": None}

    def cq_read(fabric, rail, contexts, cap):
        if state["armed"]:
            state["calls"] += 1
            if state["calls"] == 3:
                state["armed"] = False
                assert lib.ofi_amd_rma_ack_received(state["ctx"], 1, int(lib.ofi_amd_gin_ack_msg(1, 100))) == 0
        return inner.cq_read(fabric, rail, contexts, cap)

    ini.ops = m.GinFabricOps(inner.post, m.FABRIC_CQ_READ_FN(cq_read), inner.fabric)
    ini.ctx = ctypes.c_void_p()
    assert lib.ofi_amd_rma_ctx_create(NRANKS, 4, 131072, 64, ctypes.byref(ini.ops), 40000, 5000,
                                      ctypes.byref(ini.ctx)) == 0
    state["ctx"] = ini.ctx
    ini.mrs, ini.tables, ini.posts = [], [], (m.GinPost * 64)()
    for i in range(3):
        base, addr, off, keys = mr_arrays(i)
        h = ctypes.c_void_p()
        assert lib.ofi_amd_rma_mr_create(ini.ctx, base, addr.ctypes.data, off.ctypes.data, keys.ctypes.data,
                                         ctypes.byref(h)) == 0
        ini.mrs.append(h)
    req = ctypes.c_void_p()
    put = lambda: lib.ofi_amd_rma_iput(ini.ctx, 0, 0, ini.mrs[0], 8, 0, ini.mrs[1], 1, 0, ctypes.byref(req))
    for i in range(8192):
        assert put() == 0
        if i % 256 == 0:
            ini.wire()
            assert lib.ofi_amd_rma_rmaProgress(ini.ctx) == 0
    ini.wire()
    state["armed"] = True
    assert put() == ncclSuccess and req.value         # waited through two progress calls, then went
    assert state["calls"] >= 3 and not state["armed"]
    peer = lib.ofi_amd_rma_peer_state(ini.ctx, 1).contents
    assert peer.tx_tail == 100 and peer.tx_head == 8193
    ini.close()


def test_the_older_op_tables_spell_the_same_operations(lib):
    """ncclRma_v14_t, ncclGin_v13_t and ncclGin_v11_t (rma_v14.h:49-57, gin_v13.h:48-57, net_v11.h:222-227)
    carry no optFlags, v13 and v11 no isStrongSignal, v11 no context number: the reference's wrappers
    forward optFlags 0 (src/rdma/gin/nccl_ofi_gin_api.cpp:505-564, 651-663).  Two contexts are given the
    same operations, one through the v15 entry points with optFlags 0, one through the older spellings:
    the posts on the wire are the same, and so is the state towards the peer."""
    a, b = Initiator(lib), Initiator(lib)
    req = ctypes.c_void_p()
    sizes = [0, 8, 5000, 200000, 4 << 20]
    for k, size in enumerate(sizes * 3):
        which = k // len(sizes)
        common = (0, ) if which < 2 else ()
        if size:
            assert lib.ofi_amd_rma_iput(a.ctx, 0, 16, a.mrs[0], size, 32, a.mrs[1], 1, 0, ctypes.byref(req)) == 0
            fn = lib.ofi_amd_rma_iput_v14 if which < 2 else lib.ofi_amd_gin_iput_v11
            assert fn(b.ctx, *common, 16, b.mrs[0], size, 32, b.mrs[1], 1, ctypes.byref(req)) == 0 and req.value
            assert lib.ofi_amd_rma_iget(a.ctx, 0, 16, a.mrs[1], size, 32, a.mrs[0], 1, 0, ctypes.byref(req)) == 0
            assert lib.ofi_amd_rma_iget_v14(b.ctx, 0, 16, b.mrs[1], size, 32, b.mrs[0], 1, ctypes.byref(req)) == 0
        assert lib.ofi_amd_rma_iputSignal(a.ctx, 0, 16, a.mrs[0], size, 32, a.mrs[1], 1, 8 * k, a.mrs[2], 3 + k,
                                          SIGNAL_ADD, True, 0, ctypes.byref(req)) == 0
        if which == 0:
            rc = lib.ofi_amd_rma_iputSignal_v14(b.ctx, 0, 16, b.mrs[0], size, 32, b.mrs[1], 1, 8 * k, b.mrs[2], 3 + k,
                                                SIGNAL_ADD, False, ctypes.byref(req))
        elif which == 1:
            rc = lib.ofi_amd_gin_iputSignal_v13(b.ctx, 0, 16, b.mrs[0], size, 32, b.mrs[1], 1, 8 * k, b.mrs[2], 3 + k,
                                                SIGNAL_ADD, ctypes.byref(req))
        else:
            rc = lib.ofi_amd_gin_iputSignal_v11(b.ctx, 16, b.mrs[0], size, 32, b.mrs[1], 1, 8 * k, b.mrs[2], 3 + k,
                                                SIGNAL_ADD, ctypes.byref(req))
        assert rc == 0 and req.value
        assert a.wire() == b.wire()
    pa, pb = lib.ofi_amd_rma_peer_state(a.ctx, 1).contents, lib.ofi_amd_rma_peer_state(b.ctx, 1).contents
    assert bytes(pa) == bytes(pb) and pa.tx_head == 15 + 12
    # the same argument checks behind every spelling
    assert lib.ofi_amd_gin_iput_v11(b.ctx, 0, b.mrs[0], 8, 0, b.mrs[1], NRANKS, ctypes.byref(req)) == ncclInternalError
    assert req.value is None
    assert lib.ofi_amd_gin_iputSignal_v13(b.ctx, 0, 0, b.mrs[0], 8, 0, b.mrs[1], 1, 0, b.mrs[2], 1, 3,
                                          ctypes.byref(req)) == ncclInternalError
    a.close()
    b.close()


def test_a_full_request_pool_refuses_the_operation_before_it_takes_a_sequence_number(lib):
    """A pool of 16 entries holds two puts of one stripe and their metadata messages' worth of room
    less than a third needs (an operation asks for 2 + rails entries up front).  The refused call must
    leave the peer's next sequence number where it was -- a number used up without a post would stall
    the target's in-order retire -- and succeed once completions have given entries back."""
    ini = Initiator(lib, pool=16, wait_ms=30)
    req = ctypes.c_void_p()
    put = lambda: lib.ofi_amd_rma_iputSignal(ini.ctx, 0, 0, ini.mrs[0], 5000, 0, ini.mrs[1], 1, 8, ini.mrs[2], 1,
                                             SIGNAL_INC, True, 0, ctypes.byref(req))
    reqs = []
    while True:
        before = lib.ofi_amd_rma_peer_state(ini.ctx, 1).contents.tx_head
        rc = put()
        if rc != 0:
            break
        reqs.append(ctypes.c_void_p(req.value))
        assert len(reqs) < 16
    assert rc == ncclSystemError and req.value is None and len(reqs) >= 2       # -ENOMEM
    assert lib.ofi_amd_rma_peer_state(ini.ctx, 1).contents.tx_head == before
    # the wire takes the posts, their completions free the entries at the next progress call
    sent = ini.wire()
    assert len(sent) == 2 * len(reqs)
    done = ctypes.c_int()
    for r in reqs:
        for _ in range(100):
            assert lib.ofi_amd_rma_test(ini.ctx, r, ctypes.byref(done)) == 0
            if done.value:
                break
            assert lib.ofi_amd_rma_rmaProgress(ini.ctx) == 0
        assert done.value
    assert put() == 0 and req.value
    assert lib.ofi_amd_rma_peer_state(ini.ctx, 1).contents.tx_head == before + 1
    ini.wire()
    ini.close()
