"""RDMA-protocol wire formats and eager ordering rules, oracle and product side by side.

The known answers are those of the reference's tests/unit/ctrl_msg.cpp (tag matching :36-107,
ready bit :109-142, full groups :144-183, sorted insert :197-316, chain decisions :323-396,
wrap regression :408-446) plus the static_asserts of include/nccl_ofi_rdma.h.  Every case
runs against the oracle (pinning it) and against the product's host code (parity)."""
import ctypes

import numpy as np
import pytest

import _oracle
import aws_ofi_nccl_amd as m


class Side:
    """Uniform access to the oracle_* / ofi_amd_* flavour of the same functions."""

    def __init__(self, lib, prefix, mod):
        self.lib, self.prefix, self.mod = lib, prefix, mod

    def __getattr__(self, name):
        return getattr(self.lib, self.prefix + name)

    def rxq_create(self):
        if self.prefix == "oracle_":
            return self.lib.oracle_eager_rxq_create()
        q = ctypes.c_void_p()
        assert self.lib.ofi_amd_eager_rxq_create(ctypes.byref(q)) == 0
        return q


@pytest.fixture(params=["oracle", "product"])
def side(request, oracle, lib):
    return Side(oracle, "oracle_", _oracle) if request.param == "oracle" else Side(lib, "ofi_amd_", m)


def entry(side, seq=0, off=0, prev=0, tag=0, msg_seq=0, recv_len=0, cookie=0):
    return side.mod.EagerEntry(off, prev, seq, msg_seq, 0, tag, recv_len, cookie)


def peek(side, q):
    buf = (side.mod.EagerEntry * 64)()
    n = side.eager_rxq_peek(q, buf, 64)
    return [(buf[i].eager_seq, buf[i].eager_offset, buf[i].tag) for i in range(n)]


def drain(side, q, cap=64):
    buf = (side.mod.EagerEntry * cap)()
    n = side.eager_rxq_drain(q, buf, cap)
    return [(buf[i].eager_seq, buf[i].eager_offset, buf[i].tag, buf[i].cookie) for i in range(n)]


# ---- layouts ----

def test_struct_layouts():
    for mod in (_oracle, m):
        assert ctypes.sizeof(mod.EagerHdr) == 8                  # include/nccl_ofi_rdma.h:227
        assert ctypes.sizeof(mod.CtrlEntry) == 64                # :268
        assert ctypes.sizeof(mod.CtrlMsg) == 512                 # :291
        assert mod.CtrlEntry.msg_seq_num.offset == 62            # the ready bit closes the line
        assert mod.CtrlEntry.buff_len.offset == 40 and mod.CtrlEntry.tag.offset == 44
        assert mod.CtrlEntry.num_recvs.offset == 48 and mod.CtrlEntry.recv_idx.offset == 50
        assert mod.EagerHdr.eager_seq.offset == 2 and mod.EagerHdr.tag.offset == 4


def test_immediate_data_layout(side):
    # | 4-bit segment count | 3-bit recv_idx | 15-bit comm ID | 10-bit msg_seq_num |
    assert side.rdma_imm(0, 0x3FF, 0, 0) == 0x3FF
    assert side.rdma_imm(0x7FFF, 0, 0, 0) == 0x7FFF << 10
    assert side.rdma_imm(0, 0, 7, 0) == 7 << 25
    assert side.rdma_imm(0, 0, 0, 15) == 15 << 28
    rng = np.random.default_rng(1)
    out = [ctypes.c_uint32() for _ in range(4)]
    for _ in range(2000):
        comm, seq = int(rng.integers(0, 1 << 15)), int(rng.integers(0, 1 << 10))
        ridx, nseg = int(rng.integers(0, 8)), int(rng.integers(0, 16))
        imm = side.rdma_imm(comm, seq, ridx, nseg)
        side.rdma_imm_decode(imm, *[ctypes.byref(x) for x in out])
        assert [x.value for x in out] == [comm, seq, ridx, nseg]


# ---- control message ----

def test_tag_matching(side):
    ctrl = side.mod.CtrlMsg()
    ctrl.entries[0].num_recvs = 4
    for i in range(4):
        ctrl.entries[i].tag = 10 + i
        ctrl.entries[i].buff_len = 1000 * (i + 1)
        ctrl.entries[i].buff_offset = 0x1000 * (i + 1)
    for i in range(4):
        k = side.ctrl_msg_find_tag(ctypes.byref(ctrl), 10 + i)
        assert k == i and ctrl.entries[k].buff_len == 1000 * (i + 1)
    assert side.ctrl_msg_find_tag(ctypes.byref(ctrl), 99) == -1
    ctrl.entries[4].tag = 99                      # in memory, but beyond num_recvs
    assert side.ctrl_msg_find_tag(ctypes.byref(ctrl), 99) == -1
    ctrl.entries[0].num_recvs = 5
    assert side.ctrl_msg_find_tag(ctypes.byref(ctrl), 99) == 4
    ctrl.entries[0].num_recvs = 1
    assert side.ctrl_msg_find_tag(ctypes.byref(ctrl), 10) == 0
    assert side.ctrl_msg_find_tag(ctypes.byref(ctrl), 11) == -1


def fill(side, mailbox, seq, tags, rails=4, opt=0):
    n = len(tags)
    offs = (ctypes.c_uint64 * n)(*[i * 4096 for i in range(n)])
    sizes = (ctypes.c_uint32 * n)(*[4096] * n)
    tg = (ctypes.c_int * n)(*tags)
    keys = (ctypes.c_uint64 * (n * rails))(*[100 + i for i in range(n * rails)])
    return side.ctrl_msg_fill(mailbox, seq, n, offs, sizes, tg, keys, rails, opt)


def test_ready_bit_and_mailbox(side):
    mailbox = (side.mod.CtrlMsg * 256)()
    assert side.ctrl_msg_ready(mailbox, 1, 0, 1) == 0          # zeroed mailbox: seq 1 not there
    assert fill(side, mailbox, 42, [7]) == 0
    assert side.ctrl_mailbox_slot(42) == 42 and mailbox[42].entries[0].msg_seq_num == 42
    assert side.ctrl_msg_ready(mailbox, 42, 0, 1) == 1
    assert side.ctrl_msg_ready(mailbox, 42, 7, 0) == 1 and side.ctrl_msg_ready(mailbox, 42, 8, 0) == 0
    # wrap-around: 1029 lives in slot 1029 % 256 = 5 with ready value 1029 & 0x3FF = 5
    assert fill(side, mailbox, 1029, [3]) == 0
    assert side.ctrl_mailbox_slot(1029) == 5 and mailbox[5].entries[0].msg_seq_num == 5
    assert side.ctrl_msg_ready(mailbox, 1029, 0, 1) == 1
    assert side.ctrl_msg_ready(mailbox, 1030, 0, 1) == 0
    # slot 5 is shared by seq 5, 261, 517, 773: only the one that was written is ready
    assert side.ctrl_msg_ready(mailbox, 261, 0, 1) == 0 and side.ctrl_msg_ready(mailbox, 5, 0, 1) == 1


def test_full_group_and_used_entries(side):
    mailbox = (side.mod.CtrlMsg * 256)()
    assert fill(side, mailbox, 300, list(range(8)), rails=4, opt=1) == 0
    msg = mailbox[300 % 256]
    assert msg.entries[0].num_recvs == 8 and msg.entries[0].flags == 1
    for i in range(8):
        k = side.ctrl_msg_find_tag(ctypes.byref(msg), i)
        assert k == i and msg.entries[k].buff_offset == i * 4096 and msg.entries[k].recv_idx == i
        assert [msg.entries[k].mr_key[r] for r in range(4)] == [100 + i * 4 + r for r in range(4)]
        assert msg.entries[k].msg_seq_num == 300
    # a group is ready only when every entry carries the ready value
    msg.entries[5].msg_seq_num = 0
    assert side.ctrl_msg_ready(mailbox, 300, 0, 1) == 0
    msg.entries[5].msg_seq_num = 300
    assert side.ctrl_msg_ready(mailbox, 300, 3, 0) == 1
    msg.entries[3].entry_used = 1                  # consumed entries no longer match
    assert side.ctrl_msg_ready(mailbox, 300, 3, 0) == 0
    assert fill(side, mailbox, 1, [], 4) == -22 and fill(side, mailbox, 1, [0] * 9, 4) == -22
    assert fill(side, mailbox, 1, [0], 5) == -22


# ---- sequence ordering ----

def test_sequence_comparisons(side):
    assert side.seq_before(1, 2) == 1 and side.seq_before(2, 1) == 0 and side.seq_before(5, 5) == 0
    assert side.seq_before(1023, 0) == 1 and side.seq_before(0, 1023) == 0      # 10-bit wrap
    assert side.seq_before(0, 512) == 1 and side.seq_before(0, 513) == 0        # half the space
    assert side.eager_seq_before(65535, 0) == 1 and side.eager_seq_before(0, 65535) == 0
    assert side.eager_seq_before(0, 32767) == 1 and side.eager_seq_before(0, 32768) == 1
    assert side.eager_seq_before(0, 32769) == 0 and side.eager_seq_before(7, 7) == 0


def test_sorted_insert_known_answers(side):
    def run(items):
        q = side.rxq_create()
        for seq, off, tag in items:
            assert side.eager_rxq_insert(q, ctypes.byref(entry(side, seq, off, tag=tag))) == 0
        got = peek(side, q)
        side.eager_rxq_destroy(q)
        return got

    inorder = [(1, 0, 0), (1, 1, 0), (2, 0, 0)]
    assert run(inorder) == inorder                                   # test 1
    assert run(list(reversed(inorder))) == inorder                   # test 2
    assert [o for _s, o, _t in run([(1, 3, 0), (1, 1, 0), (1, 2, 0), (1, 0, 0)])] == [0, 1, 2, 3]  # 3
    assert [s for s, _o, _t in run([(1, 0, 0), (65535, 0, 0), (0, 0, 0)])] == [65535, 0, 1]        # 4
    assert run([(5, 2, 0)]) == [(5, 2, 0)]                           # test 5
    assert run([(3, 1, 10), (3, 1, 20)]) == [(3, 1, 10), (3, 1, 20)]  # test 6: equal keys keep arrival order
    assert [(s, o) for s, o, _t in run([(2, 1, 0), (1, 0, 0), (2, 0, 0), (1, 1, 0)])] == \
        [(1, 0), (1, 1), (2, 0), (2, 1)]                             # test 7


def test_chain_decisions_known_answers(side):
    can = lambda hp, ls, lo, **kw: side.eager_entry_can_process(hp, ls, lo, ctypes.byref(entry(side, **kw)))
    assert can(0, 0, 0, seq=0, off=0) == 1              # first batch starts at eager_seq 0
    assert can(0, 0, 0, seq=5, off=0) == 0
    assert can(0, 0, 0, seq=0, off=1) == 0
    assert can(1, 5, 2, seq=5, off=3) == 1              # continuation
    assert can(1, 5, 2, seq=5, off=4) == 0              # gap
    assert can(1, 5, 2, seq=6, off=3) == 0              # other batch's offset>0
    assert can(1, 5, 2, seq=6, off=0, prev=3) == 1      # boundary
    assert can(1, 5, 2, seq=6, off=0, prev=1) == 0      # previous batch not complete
    assert can(1, 5, 2, seq=7, off=0, prev=3) == 0      # skips a batch
    assert can(1, 65535, 1, seq=0, off=0, prev=2) == 1  # wrap at the boundary
    assert can(1, 5, 0, seq=6, off=0, prev=0) == 0      # prev_batch_count 0 never matches


def test_wrap_collision_regression(side):
    q = side.rxq_create()
    # bring the chain to (eager_seq 65535, offset 0): 65536 single-entry batches
    for s in range(65536):
        assert side.eager_rxq_insert(q, ctypes.byref(entry(side, s, 0, prev=1 if s else 0))) == 0
        assert len(drain(side, q)) == 1
    # new batch after the wrap: its offset 1 arrives before its offset 0
    assert side.eager_rxq_insert(q, ctypes.byref(entry(side, 0, 1, cookie=11))) == 0
    assert drain(side, q) == [] and side.eager_rxq_pending(q) == 1
    assert side.eager_rxq_insert(q, ctypes.byref(entry(side, 0, 0, prev=1, cookie=10))) == 0
    assert [c for _s, _o, _t, c in drain(side, q)] == [10, 11]
    side.eager_rxq_destroy(q)


# ---- sender numbering by hand ----

def test_sender_numbering_three_batches_by_hand(side):
    """send(), src/nccl_ofi_rdma.cpp:5783-5806, with the batch close of :5594-5598 / :5863-5866,
    from a fresh send comm (all four fields zero, :6324-6326).  Worked out on paper:
      batch 1, three eager sends (tags 10, 11, -2): the first finds eager_offset_next == 0 and takes
        eager_seq 0; offsets 0, 1, 2; prev_batch_count 0 (nothing before)
      msg_seq_num advances: prev_eager_batch_count = 3, eager_offset_next = 0
      msg_seq_num advances again with no eager send in between (rendezvous traffic): no change
      batch 2, one send (tag 20): eager_seq 1, offset 0, prev_batch_count 3
      advance: prev = 1
      batch 3, two sends (tags 30, 31): eager_seq 2, offsets 0 and 1; BOTH carry prev_batch_count 1
        (the field is copied from the comm on every send, the receiver only reads it at offset 0)
    Header bytes, little-endian {u8 offset, u8 prev, u16 seq, i32 tag}
    (include/nccl_ofi_rdma.h:217-226)."""
    tx = side.mod.EagerTx()
    side.eager_tx_init(ctypes.byref(tx))

    def send(tag):
        h = side.mod.EagerHdr()
        side.eager_tx_assign(ctypes.byref(tx), tag, ctypes.byref(h))
        return bytes(h)

    assert send(10) == bytes([0, 0, 0, 0, 10, 0, 0, 0])
    assert send(11) == bytes([1, 0, 0, 0, 11, 0, 0, 0])
    assert send(-2) == bytes([2, 0, 0, 0, 0xFE, 0xFF, 0xFF, 0xFF])
    side.eager_tx_advance(ctypes.byref(tx))
    assert (tx.eager_seq_next, tx.cur_eager_seq, tx.eager_offset_next, tx.prev_eager_batch_count) == (1, 0, 0, 3)
    side.eager_tx_advance(ctypes.byref(tx))
    assert (tx.eager_seq_next, tx.cur_eager_seq, tx.eager_offset_next, tx.prev_eager_batch_count) == (1, 0, 0, 3)
    assert send(20) == bytes([0, 3, 1, 0, 20, 0, 0, 0])
    side.eager_tx_advance(ctypes.byref(tx))
    assert send(30) == bytes([0, 1, 2, 0, 30, 0, 0, 0])
    assert send(31) == bytes([1, 1, 2, 0, 31, 0, 0, 0])
    assert (tx.eager_seq_next, tx.cur_eager_seq, tx.eager_offset_next, tx.prev_eager_batch_count) == (3, 2, 2, 1)
    # a batch is only closed by an advance: without one the next send continues batch 3
    assert send(32) == bytes([2, 1, 2, 0, 32, 0, 0, 0])


def test_sender_numbering_wraps_at_sixteen_bits(side):
    """eager_seq_next is a uint16 that wraps naturally (:5792): batch number 65,536 is numbered
    0 again, batch 65,537 (two sends) announces the single send of the batch before it."""
    tx = side.mod.EagerTx()
    side.eager_tx_init(ctypes.byref(tx))
    h = side.mod.EagerHdr()
    for batch in range(65536):
        side.eager_tx_assign(ctypes.byref(tx), 7, ctypes.byref(h))
        assert h.eager_seq == batch
        side.eager_tx_advance(ctypes.byref(tx))
    assert bytes(h) == bytes([0, 1, 0xFF, 0xFF, 7, 0, 0, 0])       # batch 65,535
    side.eager_tx_assign(ctypes.byref(tx), 8, ctypes.byref(h))
    assert bytes(h) == bytes([0, 1, 0, 0, 8, 0, 0, 0])
    side.eager_tx_assign(ctypes.byref(tx), 9, ctypes.byref(h))
    assert bytes(h) == bytes([1, 1, 0, 0, 9, 0, 0, 0])


# ---- sender numbering -> network reordering -> receiver chain ----

@pytest.mark.parametrize("seed", [1, 2, 3])
def test_sender_headers_drain_in_send_order(side, seed):
    rng = np.random.default_rng(seed)
    tx = side.mod.EagerTx()
    side.eager_tx_init(ctypes.byref(tx))
    sent = []
    for _batch in range(400):
        for _k in range(int(rng.integers(1, 9))):
            h = side.mod.EagerHdr()
            side.eager_tx_assign(ctypes.byref(tx), int(rng.integers(0, 1000)), ctypes.byref(h))
            sent.append((h.eager_seq, h.eager_offset, h.prev_batch_count, h.tag))
        side.eager_tx_advance(ctypes.byref(tx))
        if rng.random() < 0.3:
            side.eager_tx_advance(ctypes.byref(tx))       # rendezvous traffic in between: no effect
    # batches are numbered 0, 1, 2, ... with offsets 0..k-1, and announce their predecessor's size
    sizes = {}
    for s, o, _p, _t in sent:
        sizes[s] = max(sizes.get(s, 0), o + 1)
    assert sorted(sizes) == list(range(400))
    for s, o, p, _t in sent:
        if o == 0 and s > 0:
            assert p == sizes[s - 1]
    # the network delivers within a window of 32 in-flight messages in any order
    q = side.rxq_create()
    got, i = [], 0
    while i < len(sent):
        window = list(range(i, min(i + 32, len(sent))))
        rng.shuffle(window)
        for j in window:
            s, o, p, t = sent[j]
            assert side.eager_rxq_insert(q, ctypes.byref(entry(side, s, o, prev=p, tag=t, cookie=j))) == 0
            got += [c for _s, _o, _t, c in drain(side, q, cap=5)]
        i += 32
    got += [c for _s, _o, _t, c in drain(side, q)]
    assert got == list(range(len(sent)))
    assert side.eager_rxq_pending(q) == 0
    side.eager_rxq_destroy(q)


def test_eager_eligibility(side):
    # size + 8-byte header must fit the eager send size (8192 by default: 8184 payload bytes)
    assert side.eager_fits(8184, 8192) == 1 and side.eager_fits(8185, 8192) == 0
    assert side.eager_fits(0, 8192) == 1 and side.eager_fits(0, 7) == 0
    assert side.eager_fits(100, -1) == 0           # eager disabled


def test_product_matches_oracle_on_random_chains(lib, oracle):
    rng = np.random.default_rng(9)
    for _ in range(20000):
        hp, ls, lo = int(rng.integers(0, 2)), int(rng.integers(0, 1 << 16)), int(rng.integers(0, 256))
        near = lambda x, m_: int((x + rng.integers(-2, 3)) % m_)
        seq, off, prev = near(ls, 1 << 16), near(lo, 256), near(lo, 256)
        a = oracle.oracle_eager_entry_can_process(hp, ls, lo, ctypes.byref(_oracle.EagerEntry(off, prev, seq)))
        b = lib.ofi_amd_eager_entry_can_process(hp, ls, lo, ctypes.byref(m.EagerEntry(off, prev, seq)))
        assert a == b
        x, y = int(rng.integers(0, 1 << 16)), near(ls, 1 << 16)
        assert oracle.oracle_seq_before(x, y) == lib.ofi_amd_seq_before(x, y)
        assert oracle.oracle_eager_seq_before(x, y) == lib.ofi_amd_eager_seq_before(x, y)


# ---- sentinel flush: host-side completion test ----

def test_flush_completion_looks_at_the_first_word_of_every_rail_slot(lib, oracle):
    import numpy as np
    rdma, gin = 0x00000000FFFFFFFF, 0xDEADBEEFDEADBEEF          # include/nccl_ofi_rdma.h:45, gin_reqs.h:274
    for sentinel in (rdma, gin):
        for rails in (1, 2, 3, 4):
            slots = np.zeros(8 * 4, dtype=np.uint64)
            ptr = ctypes.c_void_p(slots.ctypes.data)
            assert lib.ofi_amd_flush_test(ptr, rails, sentinel) == 0 == oracle.oracle_flush_completed(ptr, rails, sentinel)
            buf = np.full(8, sentinel, dtype=np.uint64)
            oracle.oracle_flush_post(ctypes.c_void_p(buf.ctypes.data), ptr, rails)
            assert np.all(slots[:8 * rails] == sentinel) and not slots[8 * rails:].any()
            assert lib.ofi_amd_flush_test(ptr, rails, sentinel) == 1 == oracle.oracle_flush_completed(ptr, rails, sentinel)
            slots[8 * (rails - 1)] = 0                              # last rail's flag not there yet
            assert lib.ofi_amd_flush_test(ptr, rails, sentinel) == 0 == oracle.oracle_flush_completed(ptr, rails, sentinel)
            slots[8 * (rails - 1)] = sentinel
            slots[8 * (rails - 1) + 1] = 0                          # only the first 8 bytes count
            assert lib.ofi_amd_flush_test(ptr, rails, sentinel) == 1 == oracle.oracle_flush_completed(ptr, rails, sentinel)
    slots = np.zeros(32, dtype=np.uint64)
    assert lib.ofi_amd_flush_test(None, 1, rdma) == -22
    assert lib.ofi_amd_flush_test(ctypes.c_void_p(slots.ctypes.data), 0, rdma) == -22
    assert lib.ofi_amd_flush_test(ctypes.c_void_p(slots.ctypes.data), 5, rdma) == -22
