"""GIN receiver side: reassembly, in-order retire with same-slot folding, ACKs, and the
signal counter update.

The reference's own tests for this path are functional and check end values only
(tests/functional/rma.cpp: 64 put-signals leave the counter at 64;
rma_multiseg_signal.cpp: each of two slots reaches its count), so the work-item and ACK
streams are pinned here by those end values for arbitrary arrival orders, by hand-derived
arrival orders whose folding follows from the retire rules
(src/rdma/gin/nccl_ofi_gin.cpp:1622-1790), and by invariants of in-order delivery.  The
product's host receiver must then agree with the oracle event for event."""
import ctypes

import numpy as np
import pytest

import _gin_rx as G
import _oracle
from _oracle import GinAck, GinSignalWork

SIG_BASE = 0x7F0000000000
c_u32 = ctypes.c_uint32


def oracle_rx(oracle, n_peers=1, comm_ids=None):
    ids = (c_u32 * n_peers)(*(comm_ids or [7 + p for p in range(n_peers)]))
    rx = oracle.oracle_gin_rx_create(n_peers, ids)
    assert rx
    return rx


def oracle_api(oracle):
    return (oracle.oracle_gin_rx_write, oracle.oracle_gin_rx_metadata)


def run_oracle(oracle, events, peer=0, n_peers=1):
    rx = oracle_rx(oracle, n_peers)
    G.feed(oracle_api(oracle), rx, peer, events)
    work = G.take_all(oracle.oracle_gin_rx_take_work, rx, GinSignalWork)
    acks = G.take_all(oracle.oracle_gin_rx_take_acks, rx, GinAck)
    cons, nxt = c_u32(), c_u32()
    oracle.oracle_gin_rx_cursors(rx, peer, ctypes.byref(cons), ctypes.byref(nxt))
    oracle.oracle_gin_rx_destroy(rx)
    return work, acks, cons.value, nxt.value


def signals(n, slot=0, size=4096):
    return [(size, G.INC, 0, 8 * slot)] * n


# ---- end values the reference's functional tests check ----

@pytest.mark.parametrize("lookahead", [0, 1, 7, 63])
def test_sixty_four_put_signals_leave_sixty_four(oracle, lookahead):
    wire = G.sender_ops(oracle, signals(64, size=42))
    ev = G.reorder(G.events_of(wire), np.random.default_rng(lookahead), lookahead)
    work, _acks, cons, nxt = run_oracle(oracle, ev)
    assert int(G.slot_sums(work, 4, SIG_BASE)[0]) == 64
    assert cons == 64 and nxt == 64
    assert sum(w[5] for w in work) == 64


def test_two_slots_each_reach_their_count(oracle):
    # multi-rail payloads (4 segments + metadata) to two different slots, interleaved
    ops = []
    for i in range(32):
        ops.append((1 << 20, G.INC, 0, 0))
        ops.append((1 << 20, G.INC, 0, 8 * 300))
    wire = G.sender_ops(oracle, ops)
    assert all(nw == 4 for _imm, nw, _m, _a, _s in wire)
    ev = G.reorder(G.events_of(wire), np.random.default_rng(3), 9)
    work, _acks, cons, _nxt = run_oracle(oracle, ev)
    sums = G.slot_sums(work, 512, SIG_BASE)
    assert int(sums[0]) == 32 and int(sums[300]) == 32 and int(sums.sum()) == 64
    assert cons == 64


# ---- arrival orders whose outcome follows from the retire rules ----

def test_in_order_arrival_never_folds(oracle):
    wire = G.sender_ops(oracle, signals(20))
    work, _a, _c, _n = run_oracle(oracle, G.events_of(wire))
    assert [w[5] for w in work] == [1] * 20
    assert [w[4] for w in work] == list(range(20))


def test_reversed_arrival_folds_the_whole_run(oracle):
    wire = G.sender_ops(oracle, signals(20))
    ev = G.events_of(wire)
    by_op = [[e for e in ev if e[0] == k] for k in range(20)]
    rev = [e for k in reversed(range(20)) for e in by_op[k]]
    work, _a, cons, _n = run_oracle(oracle, rev)
    assert len(work) == 1
    base, off, val, peer, gate, run = work[0]
    assert (base, off, val, peer, gate, run) == (SIG_BASE, 0, 20, 0, 19, 20)
    assert cons == 20


def test_fold_stops_where_the_slot_changes(oracle):
    # slots A A B A A A, delivered last-first: runs [A x2] [B] [A x3]
    ops = [(256, G.ADD, 5, 0), (256, G.ADD, 6, 0), (256, G.ADD, 7, 8), (256, G.ADD, 1, 0),
           (256, G.ADD, 2, 0), (256, G.ADD, 3, 0)]
    wire = G.sender_ops(oracle, ops)
    ev = G.events_of(wire)
    rev = [e for k in reversed(range(6)) for e in ev if e[0] == k]
    work, _a, _c, _n = run_oracle(oracle, rev)
    assert [(w[1], w[2], w[4], w[5]) for w in work] == [(0, 11, 1, 2), (8, 7, 2, 1), (0, 6, 5, 3)]


def test_plain_put_between_signals_breaks_the_run(oracle):
    ops = [(256, G.INC, 0, 0), (256, 0, 0, 0), (256, G.INC, 0, 0)]
    wire = G.sender_ops(oracle, ops)
    assert wire[1][2] is None
    ev = G.events_of(wire)
    rev = [e for k in reversed(range(3)) for e in ev if e[0] == k]
    work, _a, cons, nxt = run_oracle(oracle, rev)
    assert [(w[2], w[4], w[5]) for w in work] == [(1, 0, 1), (1, 2, 1)]
    assert cons == 3 and nxt == 3


def test_nothing_is_delivered_past_a_missing_segment(oracle):
    wire = G.sender_ops(oracle, [(1 << 20, G.INC, 0, 0)] + signals(5))
    ev = G.events_of(wire)
    held = ev[0]                       # one payload segment of op 0 is late
    work, _a, cons, _n = run_oracle(oracle, ev[1:])
    assert work == [] and cons == 0
    work, _a, cons, _n = run_oracle(oracle, ev[1:] + [held])
    assert sum(w[5] for w in work) == 6 and cons == 6
    assert work[0][5] == 6             # all six were ready: one folded delivery


def test_signal_only_and_add_values(oracle):
    ops = [(0, G.ADD, 1 << 63, 16), (0, G.ADD, 1 << 63, 16), (0, G.ADD, 9, 16)]
    wire = G.sender_ops(oracle, ops)
    assert all(nw == 0 and m is not None for _i, nw, m, _a, _s in wire)
    work, _a, _c, _n = run_oracle(oracle, G.events_of(wire))
    assert int(G.slot_sums(work, 4, SIG_BASE)[2]) == 9      # 2^63 + 2^63 wraps to 0


# ---- invariants under random traffic ----

def random_ops(rng, n, slots=8):
    ops = []
    for _ in range(n):
        size = int(2 ** rng.uniform(0, 21)) if rng.random() < 0.9 else 0
        kind = rng.random()
        if kind < 0.45 or size == 0:
            sop = G.INC if rng.random() < 0.5 else G.ADD
            ops.append((size, sop, int(rng.integers(0, 1 << 40)), 8 * int(rng.integers(0, slots))))
        else:
            ops.append((size, 0, 0, 0))
    return ops


@pytest.mark.parametrize("seed,lookahead", [(1, 0), (2, 3), (3, 40), (4, 700)])
def test_in_order_delivery_invariants(oracle, seed, lookahead):
    rng = np.random.default_rng(seed)
    ops = random_ops(rng, 6000)
    wire = G.sender_ops(oracle, ops)
    ev = G.reorder(G.events_of(wire), rng, lookahead)
    work, acks, cons, nxt = run_oracle(oracle, ev)
    assert cons == len(ops) and nxt == len(ops) % 8192
    sig_seqs = [s for (_i, _nw, m, _a, s) in wire if m is not None]
    covered = []
    for base, off, val, _peer, gate, run in work:
        covered += [(gate - run + 1 + j) % 8192 for j in range(run)]
    # every signal op delivered exactly once, in sequence order (a run may not skip a put)
    assert covered == sig_seqs
    # the end state equals a straight per-slot sum over the ops
    want = np.zeros(8, dtype=np.uint64)
    for size, sop, val, off in ops:
        if sop:
            want[off // 8] += np.uint64(1 if sop == G.INC else val)
    assert np.array_equal(G.slot_sums(work, 8, SIG_BASE), want)
    # folded values are sums of their ops
    k = 0
    values = [1 if sop == G.INC else val for (_s, sop, val, _o) in ops if sop]
    for _b, _o, val, _p, _g, run in work:
        assert val == sum(values[k:k + run]) % (1 << 64)
        k += run


def test_ack_carries_the_cursor_and_decodes_with_reference_bitfields(oracle, ref):
    # past 4096 outstanding the sender asks for an ACK every 65th op (model 0: no ACK arrives)
    ops = signals(4400, size=8)
    wire = G.sender_ops(oracle, ops, ack_model=0)
    asked = [k for k, w in enumerate(wire) if w[3]]
    assert asked and asked[0] == 4096 + 64
    work, acks, cons, _n = run_oracle(oracle, G.events_of(wire))
    assert [a[1] for a in acks] == [k + 1 for k in asked]     # in-order arrival: one ACK per ask
    for peer, rx_consumed, msg in acks:
        assert msg == ref.ref_gin_ack(7, rx_consumed)
        assert msg == oracle.oracle_gin_ack_msg(7, rx_consumed)


# ---- ACK emission cadence, worked out by hand from retire_completed_peer_iput_ops ----
#
# src/rdma/gin/nccl_ofi_gin.cpp:1622-1790: one retire call walks every op that is complete and next
# in sequence, ORs their ack-request bits, advances rx_consumed (a 14-bit cursor) once per op, and
# at its end (maybe_send_ack, :1608-1620) sends at most ONE standalone ACK carrying the cursor as it
# stands then -- not one per asking op, and not the cursor at the asking op.  A retire call happens
# only when an arriving completion makes its own op complete (:1843-1846, :1913-1921).
# Events below are built from literal wire words: imm = ack << 28 | nseg << 24 | seq << 11 | comm << 1
# (include/rdma/gin/nccl_ofi_gin_types.h:55-79), so seq 3 / one segment / comm 5 / ack is
# 0x1000000 | 0x1800 | 0xA | 0x10000000 = 0x1100180A.

def _imm(seq, nseg=1, ack=0, comm=5):
    return (ack << 28) | (nseg << 24) | (seq << 11) | (comm << 1)


def _meta(seq, nseg, ack, base, off, val, comm=5):
    # header bit-field (:128-159): type 2 bits = 0, comm 10 bits, seq 13 bits, segment count 4 bits, ack 1 bit
    return [(comm << 2) | (seq << 12) | (nseg << 25) | (ack << 29), base, off, val]


class _Rx:
    """The oracle's or the product's receiver behind one set of calls."""

    def __init__(self, which, oracle, lib):
        self.product = which == "product"
        if self.product:
            import aws_ofi_nccl_amd as m
            self.lib, self.pre, self.Ack, self.Work = lib, "ofi_amd_gin_rx_", m.GinAck, m.GinSignalWork
            self.api = (lib.ofi_amd_gin_rx_write_completion, lib.ofi_amd_gin_rx_metadata)
        else:
            self.lib, self.pre, self.Ack, self.Work = oracle, "oracle_gin_rx_", GinAck, GinSignalWork
            self.api = oracle_api(oracle)

    def call(self, name):
        return getattr(self.lib, self.pre + name)

    def create(self, comm_ids):
        ids = (c_u32 * len(comm_ids))(*comm_ids)
        if self.product:
            rx = ctypes.c_void_p()
            assert self.lib.ofi_amd_gin_rx_create(len(comm_ids), ids, ctypes.byref(rx)) == 0
            return rx
        return self.lib.oracle_gin_rx_create(len(comm_ids), ids)


@pytest.fixture(params=["oracle", "product"])
def rxside(request, oracle, lib):
    return _Rx(request.param, oracle, lib)


def _run_events(side, events, comm_ids=(7,), peer=0):
    rx = side.create(list(comm_ids))
    acks_after = []
    buf = (side.Ack * 16)()
    for ev in events:
        G.feed(side.api, rx, peer, [ev])
        n = side.call("take_acks")(rx, buf, 16)
        acks_after.append([(buf[i].peer, buf[i].rx_consumed, buf[i].msg) for i in range(n)])
    work = G.take_all(side.call("take_work"), rx, side.Work)
    cons, nxt = c_u32(), c_u32()
    side.call("cursors")(rx, peer, ctypes.byref(cons), ctypes.byref(nxt))
    side.call("destroy")(rx)
    return acks_after, work, cons.value, nxt.value


def _ack_word(comm, rx_consumed):
    # gin_ack_msg_t (:170-181): type 2 bits = 1, comm 10 bits, rx_consumed 14 bits
    return 1 | (comm << 2) | (rx_consumed << 12)


def test_hand_built_wire_words_agree_with_the_pinned_encoders(oracle):
    assert _imm(3, 1, 1) == 0x1100180A == oracle.oracle_gin_imm(5, 3, 1, 1)
    assert _meta(3, 2, 1, 0, 0, 0)[0] == oracle.oracle_gin_meta_header(5, 3, 2, 1)
    assert _ack_word(7, 6) == 0x601D == oracle.oracle_gin_ack_msg(7, 6)


def test_ack_cadence_in_order_one_ack_per_asking_op(rxside):
    # six one-segment puts, seq 1 and 4 ask: each arrival retires exactly its own op
    ev = [(k, "w", _imm(k, ack=int(k in (1, 4)))) for k in range(6)]
    acks, work, cons, nxt = _run_events(rxside, ev)
    assert acks == [[], [(0, 2, _ack_word(7, 2))], [], [], [(0, 5, _ack_word(7, 5))], []]
    assert work == [] and (cons, nxt) == (6, 6)


def test_ack_cadence_reversed_arrival_one_ack_for_the_whole_walk(rxside):
    # same ops, arriving 5, 4, 3, 2, 1, 0: nothing can retire before seq 0 is there; that arrival
    # walks all six in one call -> a single ACK with the cursor after the walk (6, not 2 or 5)
    ev = [(k, "w", _imm(k, ack=int(k in (1, 4)))) for k in reversed(range(6))]
    acks, _work, cons, _nxt = _run_events(rxside, ev)
    assert acks == [[], [], [], [], [], [(0, 6, _ack_word(7, 6))]]
    assert cons == 6


def test_ack_cadence_pairwise_swapped(rxside):
    # arrival 1, 0, 3, 2, 5, 4; asks on 1 and 4.  Walks: {0, 1} -> ACK 2; {2, 3} -> none; {4, 5} -> ACK 6
    ev = [(k, "w", _imm(k, ack=int(k in (1, 4)))) for k in (1, 0, 3, 2, 5, 4)]
    acks, _work, _cons, _nxt = _run_events(rxside, ev)
    assert acks == [[], [(0, 2, _ack_word(7, 2))], [], [], [], [(0, 6, _ack_word(7, 6))]]


def test_ack_cursor_is_the_end_of_the_walk_not_the_asking_op(rxside):
    # arrival 2, 1, 0 with only seq 0 asking: one ACK, cursor 3
    ev = [(k, "w", _imm(k, ack=int(k == 0))) for k in (2, 1, 0)]
    acks, _work, _cons, _nxt = _run_events(rxside, ev)
    assert acks == [[], [], [(0, 3, _ack_word(7, 3))]]


def test_ack_request_is_honoured_from_either_submission_path(rxside):
    """:1817-1828 and :1893-1900: the bit may come with the write's immediate data or with the
    metadata header; the op asks if either did.  Two-segment put-signals (one write + metadata)."""
    base = SIG_BASE
    for imm_ack, meta_ack in ((1, 0), (0, 1), (1, 1), (0, 0)):
        for order in ("wm", "mw"):
            w = (0, "w", _imm(0, nseg=2, ack=imm_ack))
            mm = (0, "m", _meta(0, 2, meta_ack, base, 8, 1))
            ev = [w, mm] if order == "wm" else [mm, w]
            acks, work, cons, _nxt = _run_events(rxside, ev)
            want = [(0, 1, _ack_word(7, 1))] if (imm_ack or meta_ack) else []
            assert acks == [[], want], (imm_ack, meta_ack, order)
            assert [(x[1], x[2], x[4], x[5]) for x in work] == [(8, 1, 0, 1)] and cons == 1


def test_ack_with_a_folded_run(rxside):
    # three put-signals to one slot arrive last-first, the middle one asks: one work item of run
    # length 3 (gate = seq 2) and one ACK with cursor 3
    ev = []
    for k in (2, 1, 0):
        ev.append((k, "w", _imm(k, nseg=2, ack=int(k == 1))))
        ev.append((k, "m", _meta(k, 2, 0, SIG_BASE, 16, 1)))
    acks, work, cons, nxt = _run_events(rxside, ev)
    assert acks[:-1] == [[]] * 5 and acks[-1] == [(0, 3, _ack_word(7, 3))]
    assert work == [(SIG_BASE, 16, 3, 0, 2, 3)] and (cons, nxt) == (3, 3)


def test_ack_cursor_is_fourteen_bits_while_sequence_numbers_are_thirteen(rxside):
    """rx_consumed counts modulo 16,384 (gin_cursor_inc, include/rdma/gin/nccl_ofi_gin.h:155-158),
    sequence numbers modulo 8,192 (GIN_IMM_SEQ_MASK).  16,386 in-order puts; op 16,383 asks: the
    cursor it reports is (16,383 + 1) mod 16,384 = 0; op 16,385 asks: 2.  Op k travels as seq k mod 8,192."""
    total = 16386
    ev = [(k, "w", _imm(k & 0x1FFF, ack=int(k in (8191, 16383, 16385)))) for k in range(total)]
    acks, _work, cons, nxt = _run_events(rxside, ev)
    said = [(k, a) for k, a in enumerate(acks) if a]
    assert said == [(8191, [(0, 8192, _ack_word(7, 8192))]), (16383, [(0, 0, _ack_word(7, 0))]),
                    (16385, [(0, 2, _ack_word(7, 2))])]
    assert (cons, nxt) == (2, 2)


def test_ack_names_the_comm_id_the_peer_expects(rxside):
    # two peers with their own comm ids; completions of peer 1 only: its ACK carries id 33
    ev = [(0, "w", _imm(0, ack=1))]
    acks, _w, _c, _n = _run_events(rxside, ev, comm_ids=(21, 33), peer=1)
    assert acks == [[(1, 1, _ack_word(33, 1))]]


def test_closed_loop_never_stalls(oracle):
    """Sender and receiver wired back to back for four trips round the 13-bit sequence
    space: the ACKs the receiver produces keep the sender's window open."""
    rx = oracle_rx(oracle, 1, [5])
    api = oracle_api(oracle)
    rng = np.random.default_rng(11)
    ackbuf = (GinAck * 64)()
    workbuf = (GinSignalWork * 4096)()
    c = _oracle.GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(c), 5, 4, 131072, 64, 0)
    mrs = G.make_mrs(SIG_BASE)
    total = 4 * 8192 + 123
    pending, n_acks, max_out, delivered = [], 0, 0, 0
    for k in range(total):
        d = _oracle.GinDesc(0, 0, 8, 0, 0, 1, G.INC, 0, 0, 0, 1, 2, 2)
        w = _oracle.GinWire()
        rc = oracle.oracle_gin_iput_signal(ctypes.byref(c), mrs, ctypes.byref(d), ctypes.byref(w))
        assert rc == 0, "window closed at op %d" % k
        pending.append((int(w.imm), int(w.num_writes), [int(x) for x in w.meta], int(w.ack_req),
                        int(w.seq)))
        max_out = max(max_out, (c.tx_head - c.tx_tail) & 0x3FFF)
        if len(pending) < 5000 and k != total - 1:
            continue
        # the receiver lags: it sees a burst, out of order within the burst
        G.feed(api, rx, 0, G.reorder(G.events_of(pending), rng, 50))
        pending = []
        for i in range(oracle.oracle_gin_rx_take_acks(rx, ackbuf, 64)):
            oracle.oracle_gin_apply_ack(ctypes.byref(c), ackbuf[i].rx_consumed)
            n_acks += 1
        n = oracle.oracle_gin_rx_take_work(rx, workbuf, 4096)
        while n:
            delivered += sum(workbuf[i].run_len for i in range(n))
            n = oracle.oracle_gin_rx_take_work(rx, workbuf, 4096)
    assert delivered == total
    assert n_acks > 0 and 4096 < max_out <= 8192
    cons, nxt = c_u32(), c_u32()
    oracle.oracle_gin_rx_cursors(rx, 0, ctypes.byref(cons), ctypes.byref(nxt))
    assert cons.value == total % 16384 and nxt.value == total % 8192
    oracle.oracle_gin_rx_destroy(rx)


# ---- the counter update ----

def test_batch_apply_matches_a_plain_scatter_add(oracle):
    rng = np.random.default_rng(5)
    n, slots = 64, 16
    bases = (ctypes.c_uint64 * 2)(SIG_BASE, SIG_BASE + (1 << 30))
    sizes = (ctypes.c_uint64 * 2)(8 * slots, 8 * slots)
    c0 = rng.integers(0, 1 << 63, slots, dtype=np.uint64)
    c1 = rng.integers(0, 1 << 63, slots, dtype=np.uint64)
    want = [c0.copy(), c1.copy()]
    batch = (GinSignalWork * n)()
    for i in range(n):
        r = int(rng.integers(0, 2))
        s = int(rng.integers(0, slots if i % 2 else 3))
        v = int(rng.integers(0, 1 << 64, dtype=np.uint64))
        batch[i] = GinSignalWork(bases[r], 8 * s, v, 0, i, 1)
        want[r][s] = np.uint64((int(want[r][s]) + v) % (1 << 64))
    ptrs = (ctypes.c_void_p * 2)(c0.ctypes.data, c1.ctypes.data)
    rmw = oracle.oracle_gin_signal_apply(batch, n, bases, sizes, ptrs, 2)
    distinct = len({(batch[i].base, batch[i].offset) for i in range(n)})
    assert rmw == distinct               # one read-modify-write per slot touched
    assert np.array_equal(c0, want[0]) and np.array_equal(c1, want[1])


def test_batch_apply_rejects_unknown_region_and_misaligned_offset(oracle):
    bases = (ctypes.c_uint64 * 1)(SIG_BASE)
    sizes = (ctypes.c_uint64 * 1)(64)
    c0 = np.zeros(8, dtype=np.uint64)
    ptrs = (ctypes.c_void_p * 1)(c0.ctypes.data)
    for bad in (GinSignalWork(SIG_BASE + 8, 0, 1, 0, 0, 1), GinSignalWork(SIG_BASE, 64, 1, 0, 0, 1),
                GinSignalWork(SIG_BASE, 4, 1, 0, 0, 1)):
        batch = (GinSignalWork * 1)(bad)
        assert oracle.oracle_gin_signal_apply(batch, 1, bases, sizes, ptrs, 1) == -22
    assert not c0.any()


def test_batch_apply_finds_the_segment_of_a_window_backed_by_several_allocations(oracle):
    """ensure_signal_seg (src/rdma/gin/nccl_ofi_gin.cpp:1038-1122, 1156-1166): the window is found by its
    base, the segment by the counter's address.  Worked by hand: a window of two segments (32 and 16
    bytes, contiguous) followed by an unrelated region 1000 bytes further on."""
    bases = (ctypes.c_uint64 * 3)(SIG_BASE, SIG_BASE + 32, SIG_BASE + 1000)
    sizes = (ctypes.c_uint64 * 3)(32, 16, 64)
    c = [np.zeros(4, dtype=np.uint64), np.zeros(2, dtype=np.uint64), np.zeros(8, dtype=np.uint64)]
    ptrs = (ctypes.c_void_p * 3)(*[x.ctypes.data for x in c])

    def apply(base, offset, value):
        batch = (GinSignalWork * 1)(GinSignalWork(base, offset, value, 0, 0, 1))
        return oracle.oracle_gin_signal_apply(batch, 1, bases, sizes, ptrs, 3)

    assert apply(SIG_BASE, 0, 1) == 1 and apply(SIG_BASE, 24, 2) == 1       # segment 0, first and last counter
    assert apply(SIG_BASE, 32, 3) == 1 and apply(SIG_BASE, 40, 4) == 1      # segment 1 through the window's base
    assert apply(SIG_BASE + 32, 8, 5) == 1                                  # ... and through its own
    assert apply(SIG_BASE, 48, 9) == -22                                    # past the window's last segment
    assert apply(SIG_BASE, 1000, 9) == -22                                  # the next region is not contiguous
    assert apply(SIG_BASE + 32, 16, 9) == -22                               # past segment 1 from its own base
    assert apply(SIG_BASE, 36, 9) == -22                                    # misaligned, in segment 1
    assert apply(SIG_BASE + 1000, 56, 6) == 1 and apply(SIG_BASE + 1000, 64, 9) == -22
    assert c[0].tolist() == [1, 0, 0, 2] and c[1].tolist() == [3, 9, 0][:2] and c[2].tolist() == [0] * 7 + [6]


# ---- the product's host receiver against the oracle ----

def product_api(lib):
    return (lib.ofi_amd_gin_rx_write_completion, lib.ofi_amd_gin_rx_metadata)


@pytest.mark.parametrize("seed,lookahead,ack_model", [(21, 0, 1), (22, 5, 1), (23, 90, 0),
                                                      (24, 2000, 0)])
def test_product_receiver_matches_oracle(lib, oracle, seed, lookahead, ack_model):
    import aws_ofi_nccl_amd as m
    rng = np.random.default_rng(seed)
    n_peers = 3
    ids = (c_u32 * n_peers)(11, 12, 1023)
    orx = oracle.oracle_gin_rx_create(n_peers, ids)
    prx = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rx_create(n_peers, ids, ctypes.byref(prx)) == 0
    for peer in range(n_peers):
        ops = random_ops(rng, 8000 if ack_model == 0 else 3000, slots=4)
        wire = G.sender_ops(oracle, ops, comm_id=int(ids[peer]), ack_model=ack_model)
        ev = G.reorder(G.events_of(wire), rng, lookahead)
        G.feed(oracle_api(oracle), orx, peer, ev)
        G.feed(product_api(lib), prx, peer, ev)
        oc, on, pc, pn = c_u32(), c_u32(), c_u32(), c_u32()
        oracle.oracle_gin_rx_cursors(orx, peer, ctypes.byref(oc), ctypes.byref(on))
        assert lib.ofi_amd_gin_rx_cursors(prx, peer, ctypes.byref(pc), ctypes.byref(pn)) == 0
        assert (oc.value, on.value) == (pc.value, pn.value) == (len(ops) % 16384, len(ops) % 8192)
    ow = G.take_all(oracle.oracle_gin_rx_take_work, orx, GinSignalWork)
    pw = G.take_all(lib.ofi_amd_gin_rx_take_work, prx, m.GinSignalWork)
    oa = G.take_all(oracle.oracle_gin_rx_take_acks, orx, GinAck)
    pa = G.take_all(lib.ofi_amd_gin_rx_take_acks, prx, m.GinAck)
    assert len(ow) > 1000 and ow == pw
    assert oa == pa
    if ack_model == 0:
        assert len(oa) > 0
    oracle.oracle_gin_rx_destroy(orx)
    assert lib.ofi_amd_gin_rx_destroy(prx) == 0


def test_product_apply_ack_matches_oracle(lib, oracle):
    import aws_ofi_nccl_amd as m
    rng = np.random.default_rng(31)
    oc, pc = _oracle.GinComm(), m.GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(oc), 3, 4, 131072, 64, 0)
    assert lib.ofi_amd_gin_comm_init(ctypes.byref(pc), 3, 4, 131072, 64, 0) == 0
    for _ in range(20000):
        head = int(rng.integers(0, 1 << 14))
        tail = (head - int(rng.integers(0, 8193))) & 0x3FFF
        for c in (oc, pc):
            c.tx_head, c.tx_tail = head, tail
            c.last_ack_requested_seq = (head - 1) & 0x3FFF
            c.has_pending_ack_request = 1
        wire = int(rng.integers(0, 1 << 14))
        oracle.oracle_gin_apply_ack(ctypes.byref(oc), wire)
        lib.ofi_amd_gin_apply_ack(ctypes.byref(pc), wire)
        assert (oc.tx_tail, oc.has_pending_ack_request) == (pc.tx_tail, pc.has_pending_ack_request)
        moved = (wire - tail) & 0x3FFF
        assert oc.tx_tail == (wire if 0 < moved <= 8192 else tail)


def test_product_receiver_bad_arguments(lib):
    prx = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rx_create(0, None, ctypes.byref(prx)) == -22
    assert lib.ofi_amd_gin_rx_create(1, None, None) == -22
    assert lib.ofi_amd_gin_rx_create(2, None, ctypes.byref(prx)) == 0
    assert lib.ofi_amd_gin_rx_write_completion(prx, 2, 0) == -22
    ack_as_meta = (ctypes.c_uint64 * 4)(1, 0, 0, 0)          # msg_type 1 is an ACK, not metadata
    assert lib.ofi_amd_gin_rx_metadata(prx, 0, ack_as_meta) == -22
    assert lib.ofi_amd_gin_rx_destroy(prx) == 0
    assert lib.ofi_amd_gin_rx_destroy(None) == -22
