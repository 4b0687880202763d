"""GIN get (iget, src/rdma/gin/nccl_ofi_gin.cpp:879-939): the derivation of its reads and the
posts below it, oracle and product side by side.

The reference has no wire-level test of iget (tests/functional/rma.cpp checks the bytes that
arrive), so the expected reads are worked out by hand from the reference code: the schedule is
the threshold scheduler's (pinned by the reference's own scheduler known answers), the
addresses are input_address + localOff + offset and address_offset + remoteOff + offset, the
key is the remote registration's for the stripe's rail."""
import ctypes

import numpy as np
import pytest

import _oracle
import aws_ofi_nccl_amd as m
from test_gin_tx import Engine, W, EAGAIN, EIO, EINVAL

R = 4                      # post kind: read
AGG = 1
LOCAL0 = 0x7F0000000000                       # default_mrs(): local_base of handle 0
REMOTE2 = 0x7E0000000000 + (2 << 32)          # remote_address_offset of handle 2
KEY2 = 0x3000                                 # key[rail] of handle 2 = 0x3000 + rail


class Side:
    def __init__(self, which, oracle, lib):
        self.product = which == "product"
        self.mod = m if self.product else _oracle
        self.lib = lib if self.product else oracle
        self.mrs = _oracle.default_mrs(self.mod.GinMr)

    def comm(self, comm_id=5, rails=4, ack_model=1):
        c = self.mod.GinComm()
        if self.product:
            assert self.lib.ofi_amd_gin_comm_init(ctypes.byref(c), comm_id, rails, 131072, 64, ack_model) == 0
        else:
            self.lib.oracle_gin_comm_init(ctypes.byref(c), comm_id, rails, 131072, 64, ack_model)
        return c

    def get(self, c, size, remote_off=0, local_off=0, remote_mr=2, local_mr=0):
        d = self.mod.GinDesc(remote_off, local_off, size, 0, 0, 1, 0, 0, 0, remote_mr, local_mr, 0xFFFF, 3)
        w = self.mod.GinWire()
        if self.product:
            rc = self.lib.ofi_amd_gin_iget(ctypes.byref(c), self.mrs, 3, ctypes.byref(d), ctypes.byref(w))
        else:
            rc = self.lib.oracle_gin_iget(ctypes.byref(c), self.mrs, ctypes.byref(d), ctypes.byref(w))
        return rc, w

    def put(self, c, size, flags=0):
        d = self.mod.GinDesc(0, 0, size, 0, 0, 1, 0, flags, 0, 0, 1, 0xFFFF, 1)
        w = self.mod.GinWire()
        if self.product:
            rc = self.lib.ofi_amd_gin_iput_signal(ctypes.byref(c), self.mrs, 3, ctypes.byref(d), ctypes.byref(w))
        else:
            rc = self.lib.oracle_gin_iput_signal(ctypes.byref(c), self.mrs, ctypes.byref(d), ctypes.byref(w))
        return rc, w


@pytest.fixture(params=["oracle", "product"])
def side(request, oracle, lib):
    return Side(request.param, oracle, lib)


def reads(w):
    return [(w.writes[k].rail, w.writes[k].src, w.writes[k].len, w.writes[k].dest, w.writes[k].key, w.writes[k].more)
            for k in range(w.num_writes)]


def silent(w):
    """nothing in the record is for the target"""
    return (w.seq, w.nseg, w.imm, w.has_meta, w.meta_rail, w.meta_more, w.ack_req, list(w.meta)) == \
        (0, 0, 0, 0, 0, 0, 0, [0, 0, 0, 0])


def test_reads_of_four_gets_by_hand(side):
    """4 rails, 128 KiB minimum stripe, small below 64 B, both counters at 0.
      300,000 B: ceil(300000 / 131072) = 3 stripes wanted, 3 does not divide 4 -> 2.  Start rail =
        rr_counter 0, which moves to 2.  Stripe = ceil(ceil(300000 / 2) / 128) * 128 = 150,016:
        (rail 0, offset 0, 150,016 B), (rail 1, offset 150,016, 149,984 B).
      10 B: small -> one read on rr_small_counter 0, which moves to 1.
      0 B: small -> one read of length 0 on rail 1; rr_small_counter 2.
      1 MiB: 8 wanted, capped to 4 rails; start rail 2: rails 2, 3, 0, 1, 262,144 B each;
        rr_counter (2 + 4) mod 4 = 2."""
    c = side.comm()
    rc, w = side.get(c, 300000, remote_off=4096, local_off=512)
    assert rc == 0 and silent(w)
    assert reads(w) == [(0, LOCAL0 + 512, 150016, REMOTE2 + 4096, KEY2 + 0, 0),
                        (1, LOCAL0 + 512 + 150016, 149984, REMOTE2 + 4096 + 150016, KEY2 + 1, 0)]
    rc, w = side.get(c, 10, remote_off=7, local_off=3)
    assert rc == 0 and silent(w) and reads(w) == [(0, LOCAL0 + 3, 10, REMOTE2 + 7, KEY2 + 0, 0)]
    rc, w = side.get(c, 0)
    assert rc == 0 and silent(w) and reads(w) == [(1, LOCAL0, 0, REMOTE2, KEY2 + 1, 0)]
    rc, w = side.get(c, 1 << 20, remote_off=1 << 21)
    assert rc == 0 and silent(w)
    assert reads(w) == [(rail, LOCAL0 + k * 262144, 262144, REMOTE2 + (1 << 21) + k * 262144, KEY2 + rail, 0)
                        for k, rail in enumerate([2, 3, 0, 1])]
    assert (c.sched.rr_small_counter, c.sched.rr_counter) == (2, 2)
    # a get has no sequence number and takes no room in the window
    assert (c.tx_head, c.tx_tail, c.pinned_rail_id, c.pinned_rail_run, c.consecutive_puts_without_ack) == \
        (0, 0, -1, 0, 0)
    # the unused entries stay zero
    rc, w = side.get(c, 100)
    assert bytes(w.writes[1]) == bytes(40) and bytes(w.writes[3]) == bytes(40)


def test_gets_share_the_scheduler_with_puts_and_nothing_else(side):
    """256 KiB = two stripes.  put: rails 0, 1 (rr_counter -> 2); get: rails 2, 3 (-> 0); put: rails
    0, 1 again.  The puts are operations 0 and 1 of the window."""
    c = side.comm()
    rc, w = side.put(c, 262144)
    assert rc == 0 and [x[0] for x in reads(w)] == [0, 1] and w.seq == 0
    rc, w = side.get(c, 262144)
    assert rc == 0 and [x[0] for x in reads(w)] == [2, 3] and silent(w)
    rc, w = side.put(c, 262144)
    assert rc == 0 and [x[0] for x in reads(w)] == [0, 1] and w.seq == 1
    assert c.tx_head == 2


def test_a_get_neither_rides_nor_closes_an_open_pin(side):
    """put of 8 B with the aggregate hint: small -> rail 0 (rr_small_counter -> 1), doorbell
    deferred, rail 0 pinned with a run of 1.  get of 100 B (not small: 100 >= 64): one read on
    rr_counter's rail 0 -- chosen by the scheduler, not by the pin -- and never FI_MORE; the pin
    stays as it was.  put of 8 B without the hint: rides the pin (rail 0, though rr_small_counter
    says 1), rings the doorbell, closes the pin."""
    c = side.comm()
    rc, w = side.put(c, 8, flags=AGG)
    assert rc == 0 and reads(w)[0][0] == 0 and reads(w)[0][5] == 1
    assert (c.pinned_rail_id, c.pinned_rail_run) == (0, 1)
    rc, w = side.get(c, 100)
    assert rc == 0 and [(x[0], x[5]) for x in reads(w)] == [(0, 0)]
    assert (c.pinned_rail_id, c.pinned_rail_run, c.sched.rr_counter, c.sched.rr_small_counter) == (0, 1, 1, 1)
    rc, w = side.put(c, 8)
    assert rc == 0 and [(x[0], x[5]) for x in reads(w)] == [(0, 0)]
    assert (c.pinned_rail_id, c.pinned_rail_run, c.sched.rr_small_counter) == (-1, 0, 2)


def test_a_full_window_holds_puts_back_but_not_gets(side):
    c = side.comm(ack_model=0)
    c.tx_head, c.tx_tail = 8192 + 5, 5                 # 8,192 operations outstanding
    rc, _ = side.put(c, 8)
    assert rc == EAGAIN
    rc, w = side.get(c, 8)
    assert rc == 0 and w.num_writes == 1
    assert (c.tx_head, c.tx_tail) == (8192 + 5, 5)


def test_random_mix_of_puts_and_gets_matches_the_oracle(oracle, lib):
    rng = np.random.default_rng(11)
    a, b = Side("oracle", oracle, lib), Side("product", oracle, lib)
    for rails in (4, 3, 2, 1):
        ca, cb = a.comm(rails=rails), b.comm(rails=rails)
        for _ in range(5000):
            size = int(2 ** rng.uniform(0, 21)) if rng.random() < 0.9 else int(rng.integers(0, 70))
            if rng.random() < 0.4:
                args = dict(remote_off=int(rng.integers(0, 1 << 30)), local_off=int(rng.integers(0, 1 << 30)),
                            remote_mr=int(rng.integers(0, 3)), local_mr=int(rng.integers(0, 3)))
                (ra, wa), (rb, wb) = a.get(ca, size, **args), b.get(cb, size, **args)
            else:
                flags = int(rng.integers(0, 2))
                (ra, wa), (rb, wb) = a.put(ca, size, flags), b.put(cb, size, flags)
            assert ra == rb == 0
            assert bytes(wa) == bytes(wb)
            assert bytes(ca) == bytes(cb)


def test_product_argument_checks_and_dispatch(lib):
    s = Side("product", None, lib)
    c = s.comm()
    before = bytes(c)
    d = m.GinDesc(0, 0, 1 << 20, 0, 0, 1, 0, 0, 0, 2, 0, 0xFFFF, 3)
    w = m.GinWire()
    w.seq = 77
    assert lib.ofi_amd_gin_iget(None, s.mrs, 3, ctypes.byref(d), ctypes.byref(w)) == EINVAL
    assert lib.ofi_amd_gin_iget(ctypes.byref(c), s.mrs, 3, None, ctypes.byref(w)) == EINVAL
    for bad in (m.GinDesc(0, 0, 8, 0, 0, 1, 0, 0, 0, 3, 0, 0xFFFF, 3),      # remote handle outside the table
                m.GinDesc(0, 0, 8, 0, 0, 1, 0, 0, 0, 2, 9, 0xFFFF, 3),      # local handle outside the table
                m.GinDesc(0, 0, 8, 0, 0, 1, 0, 0, 0, 2, 0, 0xFFFF, 1)):     # a put's descriptor
        w.seq = 77
        assert lib.ofi_amd_gin_iget(ctypes.byref(c), s.mrs, 3, ctypes.byref(bad), ctypes.byref(w)) == EINVAL
        assert bytes(w) == bytes(ctypes.sizeof(w)) and bytes(c) == before
    # by kind: a get goes to iget, anything else to iputSignal
    c1, c2 = s.comm(), s.comm()
    w1, w2 = m.GinWire(), m.GinWire()
    assert lib.ofi_amd_gin_derive(ctypes.byref(c1), s.mrs, 3, ctypes.byref(d), ctypes.byref(w1)) == 0
    assert lib.ofi_amd_gin_iget(ctypes.byref(c2), s.mrs, 3, ctypes.byref(d), ctypes.byref(w2)) == 0
    assert bytes(w1) == bytes(w2) and w1.nseg == 0 and w1.num_writes == 4
    p = m.GinDesc(0, 0, 1 << 20, 0, 0, 1, 0, 0, 0, 0, 1, 0xFFFF, 1)
    assert lib.ofi_amd_gin_derive(ctypes.byref(c1), s.mrs, 3, ctypes.byref(p), ctypes.byref(w1)) == 0
    assert lib.ofi_amd_gin_iput_signal(ctypes.byref(c2), s.mrs, 3, ctypes.byref(p), ctypes.byref(w2)) == 0
    assert bytes(w1) == bytes(w2) and w1.nseg == 4 and bytes(c1) == bytes(c2)


# ---- below the derivation: the reads as posts ----

@pytest.fixture(params=["oracle", "product"])
def which(request):
    return request.param


def get_op(e, rails, peer=0):
    """a get's record with one read per entry of `rails` -> (rc, request handle)"""
    w = e.mod.GinWire()
    w.num_writes = len(rails)
    for k, rail in enumerate(rails):
        w.writes[k].rail = rail
        w.writes[k].src, w.writes[k].len, w.writes[k].dest, w.writes[k].key = 0x9000 + k, 4096, 0xA000 + k, 11
    req = ctypes.c_int32(-7)
    rc = e.fn("iget")(e.tx, peer, ctypes.byref(w), ctypes.byref(req))
    return rc, req.value


def test_a_refused_read_is_queued_and_the_get_completes_when_both_reads_have(which, oracle, lib):
    """Send queues of one entry.  A put's write (entry 1 of operation 0) fills rail 0.  The get is
    operation 2: its read on rail 0 (entry 3) is refused and queued, its read on rail 1 (entry 4)
    is posted; iget still succeeds (:923-924).  The write completes; progress reads it and posts
    entry 3.  The get is done when both reads have completed, and test() then frees it."""
    e = Engine(which, oracle, lib, (1,))
    f = e.fabric
    assert e.op([(0, 0)]) == (0, 0)
    f.take_log()
    assert get_op(e, [0, 1]) == (0, 2)
    assert f.take_log() == [("refused", R, 0, 0, 3), ("post", R, 1, 0, 4)]
    st = e.stats()
    assert (st["posts"], st["refused"], st["pending"], st["requests"]) == (2, 1, 1, 5)
    f.complete(0)
    assert e.progress() == 0
    assert f.take_log() == [("cq_read", 0, 1), ("cq_read", 0, 0), ("cq_read", 1, 0), ("cq_read", 2, 0),
                            ("cq_read", 3, 0), ("post", R, 0, 0, 3)]
    assert e.test(2) == (0, 0)
    f.complete(1)
    assert e.progress() == 0
    assert e.test(2) == (0, 0)                       # the retried read is still out
    f.complete(0)
    assert e.progress() == 0
    assert e.test(2) == (0, 1)
    assert e.test(2)[0] == EINVAL
    assert e.test(0) == (0, 1)
    assert e.stats()["requests"] == 0
    e.close()


def test_a_read_that_fails_for_good_gives_the_get_up(which, oracle, lib):
    """The second post attempt fails with -EIO: iget returns it, the umbrella and the failed read go
    back to the pool, the read that was posted stays out on its own and is freed by its completion."""
    e = Engine(which, oracle, lib, (4, (2, EIO)))
    f = e.fabric
    assert get_op(e, [0, 1, 2]) == (EIO, -1)
    assert f.take_log() == [("post", R, 0, 0, 1), ("failed", R, 1, 0, 2)]
    assert e.stats()["requests"] == 1
    f.complete(0)
    assert e.progress() == 0
    assert e.stats()["requests"] == 0 and e.stats()["completions"] == 1
    # the pool is whole again: the next get is operation 0 with reads 2 and 1 (freed last, taken first)
    f.take_log()
    assert get_op(e, [3])[0] == 0
    e.close()


def test_a_get_needs_room_for_all_its_requests_first(which, oracle, lib):
    e = Engine(which, oracle, lib, (4,), max_requests=4)
    assert get_op(e, [0, 1, 2, 3]) == (-12, -1)       # 1 + 4 entries wanted, 4 there: nothing posted
    assert e.fabric.take_log() == [] and e.stats()["requests"] == 0
    assert get_op(e, [0, 1, 2])[0] == 0
    e.close()


def test_product_rejects_records_that_are_not_a_gets(lib, oracle):
    e = Engine("product", oracle, lib, (4,))
    req = ctypes.c_int32()
    for change in ("nseg", "imm", "has_meta", "none", "rail"):
        w = m.GinWire()
        w.num_writes = 1
        if change == "none":
            w.num_writes = 0
        elif change == "rail":
            w.writes[0].rail = 4
        else:
            setattr(w, change, 1)
        assert lib.ofi_amd_gin_tx_iget(e.tx, 0, ctypes.byref(w), ctypes.byref(req)) == EINVAL
    assert lib.ofi_amd_gin_tx_iget(None, 0, ctypes.byref(m.GinWire()), ctypes.byref(req)) == EINVAL
    assert e.fabric.take_log() == []
    e.close()


def test_reads_through_the_in_process_fabric(lib):
    """The product's own fabric transmits a read like any other post: in post order per rail, with
    its completion readable once the wire has taken it."""
    fab = ctypes.c_void_p()
    assert lib.ofi_amd_loopfab_create(2, 2, ctypes.byref(fab)) == 0
    ops = m.GinFabricOps()
    assert lib.ofi_amd_loopfab_ops(fab, ctypes.byref(ops)) == 0
    tx = ctypes.c_void_p()
    assert lib.ofi_amd_gin_tx_create(2, 4, 4, 16, ctypes.byref(ops), ctypes.byref(tx)) == 0
    w = m.GinWire()
    w.num_writes = 2
    for k in range(2):
        w.writes[k].rail, w.writes[k].src, w.writes[k].len, w.writes[k].dest, w.writes[k].key = k, 100 + k, 64, 200 + k, 5
    req = ctypes.c_int32()
    assert lib.ofi_amd_gin_tx_iget(tx, 3, ctypes.byref(w), ctypes.byref(req)) == 0
    posts = (m.GinPost * 8)()
    assert lib.ofi_amd_loopfab_take_transmitted(fab, posts, 8) == 2
    assert [(p.kind, p.rail, p.peer, p.src, p.len, p.dest, p.key, p.imm) for p in posts[:2]] == \
        [(R, 0, 3, 100, 64, 200, 5, 0), (R, 1, 3, 101, 64, 201, 5, 0)]
    done = ctypes.c_int()
    assert lib.ofi_amd_gin_tx_test(tx, req, ctypes.byref(done)) == 0 and done.value == 0
    assert lib.ofi_amd_gin_tx_progress(tx) == 0
    assert lib.ofi_amd_gin_tx_test(tx, req, ctypes.byref(done)) == 0 and done.value == 1
    lib.ofi_amd_gin_tx_destroy(tx)
    lib.ofi_amd_loopfab_destroy(fab)


# ---- iflush: the fence behind gets ----

SENTINEL = 0xDEADBEEFDEADBEEF
SELF = 0xFFFFFFFF


def test_flush_posts_one_read_per_rail_and_is_done_by_the_sentinel(which, oracle, lib):
    """iflush (src/rdma/gin/nccl_ofi_gin.cpp:941-1003) with send queues of one entry, rail 1 occupied
    by a put's write (entries 0, 1).  The flush is entry 2; its reads are entries 3 (rail 0,
    posted), 4 (rail 1, refused and queued), 5, 6 (rails 2, 3, posted).  The engine has cleared
    the four slots.  The reads' completions free their entries but say nothing to the flush:
    test() is done only when every slot holds the sentinel, whatever the completion queue said."""
    e = Engine(which, oracle, lib, (1,))
    f = e.fabric
    slots = (ctypes.c_uint64 * 32)(*([0x1111] * 32))
    base = ctypes.addressof(slots)
    assert e.op([(1, 0)]) == (0, 0)
    f.take_log()
    req = ctypes.c_int32(-7)
    assert e.fn("iflush")(e.tx, slots, 0xABC000, SENTINEL, ctypes.byref(req)) == 0 and req.value == 2
    assert f.take_log() == [("post", R, 0, 0, 3), ("refused", R, 1, 0, 4), ("post", R, 2, 0, 5), ("post", R, 3, 0, 6)]
    assert [slots[8 * r] for r in range(4)] == [0, 0, 0, 0] and slots[1] == 0x1111
    assert e.stats()["requests"] == 7 and e.stats()["pending"] == 1
    assert e.test(2) == (0, 0)
    # every read that was posted completes; the flush is still not done: no sentinel yet
    for rail in (0, 1, 2, 3):
        f.complete(rail)
    assert e.progress() == 0
    assert [x for x in f.take_log() if x[0] != "cq_read"] == [("post", R, 1, 0, 4)]
    assert e.test(2) == (0, 0)
    assert e.stats()["requests"] == 3                                # the put, the flush and the retried read
    for rail in (0, 2, 3, 1):
        slots[8 * rail] = SENTINEL
        assert e.test(2) == (0, 1 if rail == 1 else 0)
    assert e.test(2)[0] == EINVAL                                   # freed by the test that saw it done
    f.complete(1)
    assert e.progress() == 0 and e.test(0) == (0, 1) and e.stats()["requests"] == 0
    e.close()


def test_flush_read_arguments_and_failure(which, oracle, lib):
    """The reads go to the own rank (loop-back), 64 bytes from the device flush buffer into the
    rail's slot.  A read that fails for good returns the flush request to the pool (:990-993)."""
    seen = []
    e = Engine(which, oracle, lib, (4, (2, EIO)), rails=3)
    real_post = e.fabric.post

    def post(fabric, p):
        c = p.contents
        seen.append((c.kind, c.rail, c.peer, c.src, c.len, c.dest, c.imm))
        return real_post(fabric, p)
    e.fabric._post = e.mod.FABRIC_POST_FN(post)
    e.fabric.ops.post = e.fabric._post
    # the engine copied the callbacks at create: make a new engine on the spying fabric
    e2 = Engine.__new__(Engine)
    e2.__dict__.update(e.__dict__)
    if e.product:
        e2.tx = ctypes.c_void_p()
        assert lib.ofi_amd_gin_tx_create(3, 4, 4, 64, ctypes.byref(e.fabric.ops), ctypes.byref(e2.tx)) == 0
    else:
        e2.tx = ctypes.c_void_p(oracle.oracle_gin_tx_create(3, 4, 4, 64, ctypes.byref(e.fabric.ops)))
    slots = (ctypes.c_uint64 * 24)()
    base = ctypes.addressof(slots)
    req = ctypes.c_int32(-7)
    assert e2.fn("iflush")(e2.tx, slots, 0xABC000, SENTINEL, ctypes.byref(req)) == EIO and req.value == -1
    assert seen == [(R, 0, SELF, base, 64, 0xABC000, 0), (R, 1, SELF, base + 64, 64, 0xABC000, 0)]
    assert e2.stats()["requests"] == 1                              # the read on rail 0 is still out
    e2.close()
    e.close()


def test_product_flush_argument_checks(lib, oracle):
    e = Engine("product", oracle, lib, (4,), max_requests=4)
    slots = (ctypes.c_uint64 * 32)()
    req = ctypes.c_int32()
    assert lib.ofi_amd_gin_tx_iflush(None, slots, 1, SENTINEL, ctypes.byref(req)) == EINVAL
    assert lib.ofi_amd_gin_tx_iflush(e.tx, None, 1, SENTINEL, ctypes.byref(req)) == EINVAL
    assert lib.ofi_amd_gin_tx_iflush(e.tx, ctypes.c_void_p(ctypes.addressof(slots) + 4), 1, SENTINEL,
                                     ctypes.byref(req)) == EINVAL
    assert lib.ofi_amd_gin_tx_iflush(e.tx, slots, 1, SENTINEL, ctypes.byref(req)) == -12   # 1 + 4 entries, 4 there
    assert e.fabric.take_log() == []
    e.close()
