"""Send/receive protocol state machines, oracle and product side by side.

Known answers:
  * message buffer: the scenario of the reference's tests/unit/msgbuff.cpp:42-122 (4 in flight,
    4-bit sequence numbers, four rounds of insert / duplicate / retrieve / complete);
  * who receives what: the scenarios of tests/functional/eager_multirecv.cpp (T5..T25), which
    the reference runs over a fabric between two ranks; here the test is the wire.  Their
    assertion is always the same: the k-th send of a tag lands, whole, in the k-th posted
    (sub-)receive of that tag, and test() reports its size.
Every case runs against the oracle (pinning it) and against the product's host code; the
randomised cases compare the two decision traces step by step.
"""
import ctypes
import random

import pytest

import _sendrecv
from _sendrecv import EAGER, WRITE, Link

EAGER_SIZE = 1024      # tests/functional/eager_multirecv.cpp:16
LARGE_SIZE = 16384     # :18

COMPLETED, INPROGRESS, NOTSTARTED, UNAVAILABLE = 0, 1, 2, 3
SUCCESS, INVALID_IDX, ERROR = 0, 1, 2
REQ, BUFF = 0, 1


@pytest.fixture(params=["oracle", "product"])
def fl(request, oracle, lib):
    return _sendrecv.flavours(oracle, lib)[request.param]


# ------------------------------------------------------------------ message buffer

class MsgBuff:
    def __init__(self, fl, max_inprogress, bits, start):
        self.fl = fl
        if fl.is_oracle:
            self.h = ctypes.c_void_p(fl.fn("msgbuff_create")(max_inprogress, bits, start))
        else:
            self.h = ctypes.c_void_p()
            rc = fl.fn("msgbuff_create")(max_inprogress, bits, start, ctypes.byref(self.h))
            if rc != 0:
                self.h = ctypes.c_void_p()
        self.ok = bool(self.h.value)

    def insert(self, idx, elem, typ=REQ):
        st = ctypes.c_int(-1)
        return self.fl.fn("msgbuff_insert")(self.h, idx, ctypes.c_void_p(elem), typ, ctypes.byref(st)), st.value

    def replace(self, idx, elem, typ=REQ):
        st = ctypes.c_int(-1)
        return self.fl.fn("msgbuff_replace")(self.h, idx, ctypes.c_void_p(elem), typ, ctypes.byref(st)), st.value

    def retrieve(self, idx):
        st, typ, elem = ctypes.c_int(-1), ctypes.c_int(-1), ctypes.c_void_p()
        res = self.fl.fn("msgbuff_retrieve")(self.h, idx, ctypes.byref(elem), ctypes.byref(typ),
                                             ctypes.byref(st))
        return res, st.value, (elem.value, typ.value) if res == SUCCESS else None

    def complete(self, idx):
        st = ctypes.c_int(-1)
        return self.fl.fn("msgbuff_complete")(self.h, idx, ctypes.byref(st)), st.value

    def close(self):
        if self.ok:
            self.fl.fn("msgbuff_destroy")(self.h)


def test_msgbuff_reference_unit_scenario(fl):
    max_inprogress, bits = 4, 4
    field = 1 << bits
    mb = MsgBuff(fl, max_inprogress, bits, 0)
    assert mb.ok
    store = [0x1000 + 8 * i for i in range(max_inprogress)]
    seq, last_completed = 0, field - 1
    for _ in range(4):
        for i in range(max_inprogress):                                   # insert new
            assert mb.insert((seq + i) % field, store[i])[0] == SUCCESS
        assert mb.insert((seq + max_inprogress) % field, 0) == (INVALID_IDX, UNAVAILABLE)   # full
        assert mb.insert((seq + max_inprogress - 1) % field, 0) == (INVALID_IDX, INPROGRESS)  # duplicate
        for i in range(max_inprogress):                                   # retrieve
            assert mb.retrieve((seq + i) % field) == (SUCCESS, INPROGRESS, (store[i], REQ))
        assert mb.retrieve((seq + max_inprogress) % field)[:2] == (INVALID_IDX, NOTSTARTED)
        assert mb.retrieve(last_completed)[:2] == (INVALID_IDX, COMPLETED)
        for i in range(max_inprogress):                                   # complete
            assert mb.complete((seq + i) % field)[0] == SUCCESS
        assert mb.complete((seq + max_inprogress) % field) == (INVALID_IDX, NOTSTARTED)
        assert mb.complete(seq) == (INVALID_IDX, COMPLETED)
        last_completed = (seq + max_inprogress - 1) % field
        seq = (seq + max_inprogress) % field
    mb.close()


def test_msgbuff_rejects_a_window_of_half_the_field_or_more(fl):
    # the constructor's check, src/nccl_ofi_msgbuff.cpp:22-26
    for max_inprogress, bits in ((0, 4), (8, 4), (9, 4), (512, 10)):
        assert not MsgBuff(fl, max_inprogress, bits, 0).ok
    mb = MsgBuff(fl, 7, 4, 0)
    assert mb.ok
    mb.close()


def test_msgbuff_replace_and_out_of_order_completion(fl):
    mb = MsgBuff(fl, 4, 4, 14)                     # the window wraps 14, 15, 0, 1
    assert mb.replace(14, 0x10) == (INVALID_IDX, NOTSTARTED)
    for k, idx in enumerate((14, 15, 0, 1)):
        assert mb.insert(idx, 0x100 + k, BUFF)[0] == SUCCESS
    assert mb.replace(15, 0x999, REQ)[0] == SUCCESS
    assert mb.retrieve(15) == (SUCCESS, INPROGRESS, (0x999, REQ))
    assert mb.retrieve(0) == (SUCCESS, INPROGRESS, (0x102, BUFF))
    assert mb.complete(15)[0] == SUCCESS           # not the oldest: the window does not move
    assert mb.insert(2, 0) == (INVALID_IDX, UNAVAILABLE)
    assert mb.retrieve(15)[:2] == (INVALID_IDX, COMPLETED)
    assert mb.complete(14)[0] == SUCCESS           # now 14 and 15 retire together
    assert mb.insert(2, 0x200)[0] == SUCCESS and mb.insert(3, 0x201)[0] == SUCCESS
    assert mb.insert(4, 0) == (INVALID_IDX, UNAVAILABLE)
    assert mb.retrieve(10)[:2] == (INVALID_IDX, NOTSTARTED)   # far ahead: "not started" for a reader
    mb.close()


def test_msgbuff_insert_ahead_leaves_empty_slots(fl):
    mb = MsgBuff(fl, 4, 4, 0)
    assert mb.insert(2, 0x22)[0] == SUCCESS        # 0 and 1 skipped
    assert mb.retrieve(0)[:2] == (INVALID_IDX, NOTSTARTED)
    assert mb.complete(1) == (INVALID_IDX, NOTSTARTED)
    assert mb.insert(3, 0x23)[0] == SUCCESS
    assert mb.insert(4, 0) == (INVALID_IDX, UNAVAILABLE)      # 0..3 is the whole window
    assert mb.insert(0, 0x20)[0] == SUCCESS        # a skipped number is filled in place
    assert mb.retrieve(0) == (SUCCESS, INPROGRESS, (0x20, REQ))
    assert mb.insert(4, 0) == (INVALID_IDX, UNAVAILABLE)
    assert mb.complete(0)[0] == SUCCESS            # 0 retires; 1 is still empty and holds the window
    assert mb.insert(4, 0x24)[0] == SUCCESS
    assert mb.insert(5, 0) == (INVALID_IDX, UNAVAILABLE)
    mb.close()


def test_msgbuff_random_ops_oracle_and_product_agree(oracle, lib):
    fls = _sendrecv.flavours(oracle, lib)
    rng = random.Random(5)
    for max_inprogress, bits in ((4, 4), (7, 4), (256, 10), (3, 5)):
        field = 1 << bits
        start = rng.randrange(field)
        a, b = MsgBuff(fls["oracle"], max_inprogress, bits, start), MsgBuff(fls["product"], max_inprogress, bits, start)
        head = start
        for step in range(4000):
            op = rng.random()
            idx = (head + rng.randrange(-max_inprogress - 2, max_inprogress + 3)) % field
            if op < 0.35:
                elem = 0x1000 + step * 8
                ra, rb = a.insert(idx, elem, step & 1), b.insert(idx, elem, step & 1)
                if ra[0] == SUCCESS:
                    head = (idx + 1) % field
            elif op < 0.45:
                ra, rb = a.replace(idx, 0x77000 + step), b.replace(idx, 0x77000 + step)
            elif op < 0.7:
                ra, rb = a.retrieve(idx), b.retrieve(idx)
            else:
                ra, rb = a.complete(idx), b.complete(idx)
            assert ra == rb, (max_inprogress, bits, step, idx, ra, rb)
        a.close()
        b.close()


# ------------------------------------------------------- who receives what (T5..T25)

def late_receiver(link, msgs, recvs):
    """Rank 0 posts its sends at once (retrying those told to call again); rank 1 posts its
    receives only after the first round, so whatever can go eager has gone eager."""
    state = {"posted": False, "handles": []}

    def pump():
        if not state["posted"]:
            state["posted"] = True
            for tags, sizes in recvs:
                state["handles"].append(link.recv(tags, sizes))
        link.deliver()
        link.copies()
        for h in range(len(link.sends)):
            link.test_send(h)
    sends = link.post_sends_interleaved(msgs, pump)
    link.run_to_completion()
    return sends, state["handles"]


def early_receiver(link, msgs, recvs):
    handles = [link.recv(tags, sizes) for tags, sizes in recvs]

    def pump():
        link.deliver()
        link.copies()
        for h in range(len(link.sends)):
            link.test_send(h)
    sends = link.post_sends_interleaved(msgs, pump)
    link.run_to_completion()
    return sends, handles


def check_per_tag_order(link, msgs, recvs, sends, handles, check_send_size=True):
    """k-th send of a tag -> k-th posted (sub-)receive of that tag, whole, with sizes reported."""
    slots = {}
    for rh, (tags, sizes) in zip(handles, recvs):
        for sub, (tag, cap) in enumerate(zip(tags, sizes)):
            slots.setdefault(tag, []).append((rh, sub, cap))
    seen = {}
    for (size, tag, label), sh in zip(msgs, sends):
        k = seen.get(tag, 0)
        seen[tag] = k + 1
        rh, sub, cap = slots[tag][k]
        assert link.landed(rh, sub) == [(label, min(size, cap))], (label, tag, link.landed(rh, sub))
        assert link.recvs[rh]["reported"][sub if link.recvs[rh]["n"] > 1 else 0] == size
        if check_send_size:
            assert link.sends[sh]["reported"] == min(size, cap)
    assert all(r["done"] for r in link.recvs) and all(s["done"] for s in link.sends)
    st, rt = link.send_state(), link.recv_state()
    assert st["num_inflight_reqs"] == 0 and st["num_inflight_writes"] == 0 and st["eager_queue_count"] == 0
    assert rt["num_inflight_reqs"] == 0 and rt["eager_pending"] == 0
    assert st["next_msg_seq_num"] == rt["next_msg_seq_num"] == 1 + len(recvs)
    assert st["n_ctrl_received"] == rt["n_ctrl_sent"] == len(recvs)


def kinds(link, sends):
    return [link.sends[h]["kind"] for h in sends]


E, L = EAGER_SIZE, LARGE_SIZE


def test_t5_single_eager_receive_posted_late(fl):
    link = Link(fl)
    msgs, recvs = [(E, 1, "S")], [([1], [E])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER]
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t6_single_receive_posted_first_goes_rendezvous(fl):
    link = Link(fl)
    msgs, recvs = [(E, 1, "S")], [([1], [E])]
    sends, handles = early_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [WRITE]
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t7_four_sequential_eager_messages_form_one_batch(fl):
    link = Link(fl)
    msgs = [(E, 1, "m%d" % i) for i in range(4)]
    recvs = [([1], [E])] * 4
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER] * 4
    hdrs = [t[7] for t in link.trace if t[0] == "send"]
    assert hdrs == [(i, 0, 0, 1) for i in range(4)]            # eager_offset 0..3 of batch 0
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t8_grouped_receive_all_eager(fl):
    link = Link(fl)
    msgs = [(E, 10, "a"), (E, 11, "b"), (E, 12, "c")]
    recvs = [([10, 11, 12], [E, E, E])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER] * 3
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t9_grouped_receive_mixed_eager_and_write(fl):
    link = Link(fl)
    msgs = [(E, 20, "small"), (L, 21, "large")]
    recvs = [([20, 21], [E, L])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER, WRITE]
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t10_grouped_receive_no_eager(fl):
    link = Link(fl)
    msgs = [(L, 30, "x"), (L, 31, "y"), (L, 32, "z")]
    recvs = [([30, 31, 32], [L, L, L])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [WRITE] * 3
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t11_eager_across_single_and_grouped(fl):
    link = Link(fl)
    msgs = [(E, 1, "S"), (E, 40, "T"), (E, 41, "U")]
    recvs = [([1], [E]), ([40, 41], [E, E])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER] * 3
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t12_tag_pushback_across_two_groups(fl):
    link = Link(fl)
    msgs = [(E, 51, "a"), (E, 53, "b"), (E, 50, "c"), (E, 52, "d")]      # B, D, A, C
    recvs = [([51, 53], [E, E]), ([50, 52], [E, E])]
    sends, handles = late_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t13_thirty_two_eager_messages_fill_the_sender_queue(fl):
    link = Link(fl)
    msgs = [(E, 1, "p%d" % i) for i in range(32)]
    recvs = [([1], [E])] * 32
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER] * 32
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_sender_queue_full_refuses_the_thirty_third(fl):
    link = Link(fl)
    for i in range(32):
        assert link.send(E, 1, "p%d" % i) is not None
    assert link.send(E, 1, "p32") is None                       # NCCL_OFI_MAX_EAGER_PENDING reached
    assert link.send_state()["eager_queue_count"] == 32
    link.close()


def test_t14_eager_size_boundary(fl):
    for size, kind in ((8184, EAGER), (8185, None)):
        link = Link(fl)
        h = link.send(size, 1, "b")
        if kind is None:
            assert h is None                                    # 8185 + 8 > 8192: waits for the receive
        else:
            assert link.sends[h]["kind"] == EAGER
        link.close()
    for size in (8184, 8185):
        link = Link(fl)
        msgs, recvs = [(size, 1, "b")], [([1], [size])]
        sends, handles = late_receiver(link, msgs, recvs)
        check_per_tag_order(link, msgs, recvs, sends, handles)
        link.close()


def test_t15_two_groups_every_eager_write_permutation(fl):
    link = Link(fl)
    is_eager = [[True, True, False, False], [True, False, True, False]]     # per group, per tag 60..63
    msgs = [(E if is_eager[g][i] else L, 60 + i, "g%dt%d" % (g, i)) for g in range(2) for i in range(4)]
    recvs = [([60, 61, 62, 63], [E if is_eager[g][i] else L for i in range(4)]) for g in range(2)]
    sends, handles = late_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t16_same_tags_over_four_groups_keep_order(fl):
    link = Link(fl)
    msgs = [(E, 70 + (i & 1), "k%d" % i) for i in range(8)]
    recvs = [([70, 71], [E, E])] * 4
    sends, handles = late_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


INTERLEAVED = [0, 1, 2, 3, 4, 5, 6, 1, 7, 0, 2, 3, 4, 5, 6, 7]   # eager_multirecv.cpp T17/T18


@pytest.mark.parametrize("size", [LARGE_SIZE, EAGER_SIZE])
def test_t17_t18_interleaved_sends_across_two_groups(fl, size):
    link = Link(fl)
    msgs = [(size, t, "i%d" % i) for i, t in enumerate(INTERLEAVED)]
    recvs = [(list(range(8)), [size] * 8)] * 2
    sends, handles = (early_receiver if size == LARGE_SIZE else late_receiver)(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t19_interleaved_mixed_eager_and_write(fl):
    link = Link(fl)
    order = [(0, E), (1, E), (2, L), (1, E), (3, L), (0, E), (2, L), (3, L)]
    msgs = [(s, t, "x%d" % i) for i, (t, s) in enumerate(order)]
    recvs = [([0, 1, 2, 3], [E, E, L, L])] * 2
    sends, handles = late_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t21_three_groups_same_tags_different_sizes(fl):
    link = Link(fl)
    gsz = [E, L, E]
    order = [(0, 0), (0, 1), (1, 0), (2, 0), (1, 1), (2, 1)]               # (group, tag)
    msgs = [(gsz[g], t, "g%dt%d" % (g, t)) for g, t in order]
    recvs = [([0, 1], [gsz[g]] * 2) for g in range(3)]
    sends, handles = late_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t22_heavy_interleaving_all_writes(fl):
    link = Link(fl)
    msgs = [(L, t, "m%dt%d" % (g, t)) for t in range(8) for g in range(2)]
    recvs = [(list(range(8)), [L] * 8)] * 2
    sends, handles = early_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [WRITE] * 16
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t23_eager_batch_spanning_three_groups(fl):
    link = Link(fl)
    stags = [1, 2, 3, 4, 10, 11, 12, 13, 20, 21, 22, 23]
    msgs = [(E, t, chr(ord("A") + i)) for i, t in enumerate(stags)]
    recvs = [(stags[4 * g:4 * g + 4], [E] * 4) for g in range(3)]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER] * 12
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t24_eager_batch_spanning_single_grouped_single_grouped(fl):
    link = Link(fl)
    stags = [1, 50, 51, 1, 60, 61]
    msgs = [(E, t, chr(ord("P") + i)) for i, t in enumerate(stags)]
    recvs = [([1], [E]), ([50, 51], [E, E]), ([1], [E]), ([60, 61], [E, E])]
    sends, handles = late_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_t25_single_receive_control_message_against_a_rotated_queue(fl):
    link = Link(fl)
    msgs = [(E, 30, "A"), (E, 40, "B"), (L, 31, "C"), (L, 20, "D")]
    recvs = [([30, 31], [E, L]), ([20], [L]), ([40], [E])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER, EAGER, WRITE, WRITE]
    check_per_tag_order(link, msgs, recvs, sends, handles)
    assert link.sends[sends[1]]["reported"] == E                # matched to a later control message
    link.close()


# ---------------------------------- grouped receives (tests/functional/grouped_recv.cpp)

@pytest.mark.parametrize("n_recvs", [1, 2, 4, 8])
@pytest.mark.parametrize("runner", ["late", "early"])
def test_grouped_recv_one_tag_growing_sizes(fl, n_recvs, runner):
    # grouped_recv.cpp:158-240: n sends of 1024*(i+1) bytes, one tag, one grouped receive
    link = Link(fl)
    msgs = [(1024 * (i + 1), 1, chr(ord("A") + i)) for i in range(n_recvs)]
    recvs = [([1] * n_recvs, [1024 * (i + 1) for i in range(n_recvs)])]
    sends, handles = (late_receiver if runner == "late" else early_receiver)(link, msgs, recvs)
    # An eager send looks its receive-buffer length up by tag (get_ctrl_msg_buff_len,
    # src/nccl_ofi_rdma.cpp:2183-2196), which finds the group's first entry of that tag: with one
    # tag for all sub-receives the sender reports min(size, first buffer).  The data and the
    # receiver's sizes are right; the reference's test does not read the sender's size.
    check_per_tag_order(link, msgs, recvs, sends, handles, check_send_size=(runner == "early"))
    if runner == "late":
        assert [link.sends[h]["reported"] for h in sends] == [
            1024 if link.sends[h]["kind"] == EAGER else link.sends[h]["size"] for h in sends]
    link.close()


GROUPED_PATTERN = [(8, 20), (3, 1), (8, 10), (4, 1), (1, 1), (8, 10), (7, 1), (5, 1), (8, 4), (2, 1),
                   (1, 1), (8, 4), (7, 1)]          # (sends per receive, receives), grouped_recv.cpp:255-258


def test_grouped_recv_alltoall_pattern(fl):
    """The production alltoall trace shape: phases of grouped receives of 1..8 sub-receives, 256 KiB
    sends into 512 KiB buffers, the receiver keeping a window of receives posted ahead."""
    link = Link(fl)
    msgs, recvs = [], []
    for phase, (per, count) in enumerate(GROUPED_PATTERN):
        for r in range(count):
            recvs.append((list(range(per)), [524288] * per))
            msgs += [(262144, t, "p%dr%dt%d" % (phase, r, t)) for t in range(per)]
    posted = {"n": 0, "handles": []}

    def pump():
        while posted["n"] < len(recvs) and link.recv_state()["num_inflight_reqs"] < 16:
            posted["handles"].append(link.recv(*recvs[posted["n"]]))
            posted["n"] += 1
        link.deliver()
        link.copies()
        for h in range(len(link.sends)):
            link.test_send(h)
        for h in range(len(link.recvs)):
            link.test_recv(h)
    pump()
    sends = link.post_sends_interleaved(msgs, pump, max_rounds=2000)
    link.run_to_completion()
    assert kinds(link, sends) == [WRITE] * len(msgs)
    check_per_tag_order(link, msgs, recvs, sends, posted["handles"])
    link.close()


def test_grouped_recv_multi_tag_send_arrives_before_its_group(fl):
    # grouped_recv.cpp:666-671: receive [tag 8] then receive [tags 0..7]; sends 0, 8, 1, 2, .. 7
    link = Link(fl)
    msgs = [(L, t, "t%d" % t) for t in (0, 8, 1, 2, 3, 4, 5, 6, 7)]
    recvs = [([8], [L]), (list(range(8)), [L] * 8)]
    sends, handles = early_receiver(link, msgs, recvs)
    check_per_tag_order(link, msgs, recvs, sends, handles)
    first = [t for t in link.trace if t[0] == "send"][0]
    assert first[3] == 0                     # tag 0 is told to call again: its group is not at the head
    link.close()


# ------------------------------------------------------------------- further cases

def test_zero_length_messages_complete_without_a_copy(fl):
    link = Link(fl)
    msgs = [(0, 5, "z0"), (E, 5, "d1"), (0, 6, "z2")]
    recvs = [([5], [E]), ([5, 6], [E, E])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER] * 3
    copies = [t for t in link.trace if t[0] == "copy"]
    assert [(c[1], c[6]) for c in copies] == [("z0", 0), ("d1", 1), ("z2", 0)]
    check_per_tag_order(link, msgs, recvs, sends, handles)
    link.close()


def test_receive_buffer_smaller_than_the_message_truncates(fl):
    link = Link(fl)
    msgs, recvs = [(E, 1, "e"), (L, 2, "w")], [([1], [100]), ([2], [5000])]
    sends, handles = late_receiver(link, msgs, recvs)
    assert kinds(link, sends) == [EAGER, WRITE]
    assert link.landed(handles[0]) == [("e", 100)] and link.landed(handles[1]) == [("w", 5000)]
    assert link.sends[sends[0]]["reported"] == 100 and link.sends[sends[1]]["reported"] == 5000
    # an eager message is cut to the receive buffer before the copy (rdma_eager_copy_req::post,
    # src/nccl_ofi_rdma.cpp:2738-2743) and the completion counts the bytes copied (:2936-2937)
    assert link.recvs[handles[0]]["reported"] == [100] and link.recvs[handles[1]]["reported"] == [5000]
    link.close()


def test_eager_arrivals_out_of_order_on_the_wire(fl):
    link = Link(fl)
    for i in range(6):
        assert link.send(E, 1, "m%d" % i) is not None
    link.deliver(order=[3, 1, 5, 0, 2, 4])
    assert link.recv_state()["eager_pending"] == 6
    handles = [link.recv([1], [E]) for _ in range(6)]
    link.run_to_completion()
    for i, h in enumerate(handles):
        assert link.landed(h) == [("m%d" % i, E)]
    link.close()


def test_rendezvous_striping_and_segment_counting(fl):
    link = Link(fl)
    sizes = [64, 4096, 131072, 131073, 400000, 1 << 20, (1 << 22) + 5]
    handles = [link.recv([3], [s]) for s in sizes]
    sends = [link.send(s, 3, "w%d" % i) for i, s in enumerate(sizes)]
    assert None not in sends
    nx = [len(t[10]) for t in link.trace if t[0] == "send"]
    assert nx == [1, 1, 1, 2, 4, 4, 4]
    rng = random.Random(3)
    order = list(range(len(link.wire)))
    rng.shuffle(order)
    link.deliver(order)                               # stripes of different messages interleave
    link.run_to_completion()
    for i, h in enumerate(handles):
        assert link.landed(h) == [("w%d" % i, sizes[i])] and link.recvs[h]["reported"] == [sizes[i]]
    link.close()


def test_receive_completion_optional_needs_only_the_control_message(fl):
    link = Link(fl)
    h = link.recv([9], [L], completion_optional=1)
    assert link.test_recv(h)                          # done once the control message is out
    s = link.send(L, 9, "q")
    assert [t[11] for t in link.trace if t[0] == "send"] == [1]          # no_target_completion
    link.deliver()
    assert link.test_send(s)
    link.close()


def test_receiver_refuses_the_129th_request_and_sender_keeps_sequence(fl):
    link = Link(fl)
    for i in range(128):
        assert isinstance(link.recv([1], [E]), int) and link.recvs[-1]["seq"] == 1 + i
    assert link.recv([1], [E]) == -28                 # -ENOSPC: NCCL_OFI_MAX_REQUESTS in flight
    for i in range(128):
        assert link.send(E, 1, "s%d" % i) is not None
    link.run_to_completion()
    assert link.recv([1], [E]) == 128                 # room again, sequence number 129
    assert link.recvs[-1]["seq"] == 129
    link.close()


def test_sequence_numbers_wrap_at_ten_bits(fl):
    link = Link(fl)
    for i in range(1100):
        size = E if i % 3 else L
        if i % 2:
            h = link.recv([4], [size])
            s = link.send(size, 4, "m%d" % i)
        else:
            s = link.send(size, 4, "m%d" % i)
            if s is None:                                       # large: needs the receive first
                h = link.recv([4], [size])
                s = link.send(size, 4, "m%d" % i)
            else:
                link.deliver()
                h = link.recv([4], [size])
        assert s is not None
        link.run_to_completion()
        assert link.landed(h) == [("m%d" % i, size)]
        assert link.recvs[h]["seq"] == (1 + i) % 1024
    assert link.send_state()["next_msg_seq_num"] == (1 + 1100) % 1024
    link.close()


# ------------------------------------------------- randomised: oracle and product, step by step

def random_program(rng, n_msgs, unique_tags):
    """Sends with random sizes; receives cut from the send order in groups of 1..4, each group
    shuffled, some buffers smaller than their message.  With unique_tags every message has a
    tag of its own, so matching has one answer; without, five tags repeat and messages of one
    tag may overtake each other where the sender's queue has rotated (the reference does the
    same), so only the two flavours' agreement is checked."""
    msgs = []
    for i in range(n_msgs):
        size = rng.choice([0, 8, 100, EAGER_SIZE, 8184, 8185, LARGE_SIZE, 200000, 600000])
        msgs.append((size, 100 + i if unique_tags else rng.randrange(1, 6), "r%d" % i))
    recvs, i = [], 0
    while i < n_msgs:
        n = min(rng.choice([1, 1, 2, 3, 4]), n_msgs - i)
        grp = msgs[i:i + n]
        rng.shuffle(grp)
        recvs.append(([g[1] for g in grp], [g[0] if rng.random() < 0.8 else max(g[0] // 2, 1) for g in grp]))
        i += n
    return msgs, recvs


def run_program(fl, msgs, recvs, seed, max_rounds, strict=True):
    """Random interleaving of send attempts, receive posts, deliveries in random order and
    test() calls; returns (trace, memory, sizes reported, finished)."""
    rng = random.Random(seed)
    link = Link(fl)
    link.strict = strict
    pending_recvs = list(recvs)
    queue = list(range(len(msgs)))
    finished = False
    for _ in range(max_rounds):
        blocked, again = set(), []
        for i in queue:
            size, tag, label = msgs[i]
            if tag in blocked or rng.random() < 0.2:
                again.append(i)
                blocked.add(tag)
                continue
            if link.send(size, tag, label) is None:
                blocked.add(tag)
                again.append(i)
        queue = again
        for _ in range(rng.randrange(0, 3)):
            if pending_recvs and link.recv_state()["num_inflight_reqs"] < 128:
                tags, sizes = pending_recvs.pop(0)
                assert isinstance(link.recv(tags, sizes), int)
        if link.wire and rng.random() < 0.8:
            order = list(range(len(link.wire)))
            rng.shuffle(order)
            link.deliver(order)
        link.copies()
        for h in range(len(link.sends)):
            if rng.random() < 0.7:
                link.test_send(h)
        for h in range(len(link.recvs)):
            if rng.random() < 0.7:
                link.test_recv(h)
        link.trace.append(("state", tuple(sorted(link.send_state().items())),
                           tuple(sorted(link.recv_state().items()))))
        if not (queue or pending_recvs or link.wire or not all(s["done"] for s in link.sends)
                or not all(r["done"] for r in link.recvs)):
            finished = True
            break
    out = (link.trace, {k: [(e[0], e[1]) for e in v] for k, v in link.memory.items()},
           ([s["reported"] for s in link.sends], [r["reported"] for r in link.recvs]), finished)
    link.close()
    return out


def same_decisions(a, b):
    assert len(a[0]) == len(b[0])
    for k, (x, y) in enumerate(zip(a[0], b[0])):
        assert x == y, (k, x, y)
    assert a[1:] == b[1:]


@pytest.mark.parametrize("seed", range(12))
def test_random_programs_with_unique_tags_deliver_everything(oracle, lib, seed):
    fls = _sendrecv.flavours(oracle, lib)
    rng = random.Random(1000 + seed)
    msgs, recvs = random_program(rng, 40 + 10 * seed, unique_tags=True)
    a = run_program(fls["oracle"], msgs, recvs, seed, 400)
    b = run_program(fls["product"], msgs, recvs, seed, 400)
    same_decisions(a, b)
    assert a[3], "did not quiesce"
    # every receive buffer holds exactly its message, cut to the buffer
    memory, size_of = a[1], {m[2]: m[0] for m in msgs}
    assert sum(len(v) for v in memory.values()) == len(msgs)
    caps = {}
    link_dst = 0x10000000
    for tags, sizes in recvs:
        for i, (t, c) in enumerate(zip(tags, sizes)):
            caps[link_dst + 0x100000 * i] = (t, c)
        link_dst += 0x100000 * 8
    for dst, v in memory.items():
        tag, cap = caps[dst]
        assert v == [("r%d" % (tag - 100), min(size_of["r%d" % (tag - 100)], cap))]


@pytest.mark.parametrize("seed", range(12))
def test_random_programs_with_repeating_tags_decide_alike(oracle, lib, seed):
    fls = _sendrecv.flavours(oracle, lib)
    rng = random.Random(2000 + seed)
    msgs, recvs = random_program(rng, 40 + 10 * seed, unique_tags=False)
    same_decisions(run_program(fls["oracle"], msgs, recvs, seed, 150, strict=False),
                   run_program(fls["product"], msgs, recvs, seed, 150, strict=False))
