"""The GIN initiator below the wire derivation: request pool, posts, pending retry, bounded CQ
drain (ofi_amd_gin_tx_* against the oracle's restatement of src/rdma/gin/nccl_ofi_gin.cpp:
737-864, 267-315 and src/rdma/gin/nccl_ofi_gin_resources.cpp:89-166, 574-599).

The fabric is a Python object behind the two callbacks, so a test decides which post is
refused and when completions appear.  The expected post / retry / completion orders are worked
out by hand from the reference code; oracle and product run the same scripts and must produce
the same fabric log.  A random differential run and the product's own in-process fabric follow."""
import ctypes

import numpy as np
import pytest

import _oracle
import aws_ofi_nccl_amd as m

W, M, A = 1, 2, 3          # post kinds: write, metadata send, ACK send
EAGAIN, EIO, ENOMEM, EINVAL = -11, -5, -12, -22


class Fabric:
    """Per rail: a send queue of `depth` entries (an entry leaves it when `complete` is told so)
    and a completion queue.  Everything the engine does to it is logged."""

    def __init__(self, mod, rails, depth, fail_at=None):
        self.mod, self.depth = mod, depth
        self.sq = [[] for _ in range(rails)]
        self.cq = [[] for _ in range(rails)]
        self.log = []
        self.fail_at = fail_at          # (attempt number, errno) -> that post attempt fails for good
        self.attempts = 0
        self._post = mod.FABRIC_POST_FN(self.post)
        self._cq_read = mod.FABRIC_CQ_READ_FN(self.cq_read)
        self.ops = mod.GinFabricOps(self._post, self._cq_read, None)

    def post(self, _fabric, p):
        p = p.contents
        self.attempts += 1
        rec = (p.kind, p.rail, p.more, p.context)
        if self.fail_at and self.fail_at[0] == self.attempts:
            self.log.append(("failed",) + rec)
            return self.fail_at[1]
        if len(self.sq[p.rail]) >= self.depth:
            self.log.append(("refused",) + rec)
            return EAGAIN
        self.sq[p.rail].append(p.context)
        self.log.append(("post",) + rec)
        return 0

    def cq_read(self, _fabric, rail, contexts, cap):
        n = min(cap, len(self.cq[rail]))
        for i in range(n):
            contexts[i] = self.cq[rail].pop(0)
        self.log.append(("cq_read", rail, n))
        return n

    def complete(self, rail, n=1):
        for _ in range(n):
            self.cq[rail].append(self.sq[rail].pop(0))

    def take_log(self):
        out, self.log = self.log, []
        return out


class Engine:
    def __init__(self, which, oracle, lib, fabric_args, cq_read_count=4, max_iter=4, max_requests=64, rails=4):
        self.product = which == "product"
        self.mod = m if self.product else _oracle
        self.fabric = Fabric(self.mod, rails, *fabric_args)
        if self.product:
            self.lib, self.pre = lib, "ofi_amd_gin_tx_"
            self.tx = ctypes.c_void_p()
            assert lib.ofi_amd_gin_tx_create(rails, cq_read_count, max_iter, max_requests,
                                             ctypes.byref(self.fabric.ops), ctypes.byref(self.tx)) == 0
        else:
            self.lib, self.pre = oracle, "oracle_gin_tx_"
            self.tx = ctypes.c_void_p(oracle.oracle_gin_tx_create(rails, cq_read_count, max_iter, max_requests,
                                                                  ctypes.byref(self.fabric.ops)))
            assert self.tx.value

    def fn(self, name):
        return getattr(self.lib, self.pre + name)

    def op(self, writes, meta=None, peer=0, imm=0x1234):
        """writes: [(rail, more)], meta: (rail, more) or None -> (rc, request handle)"""
        w = self.mod.GinWire()
        w.imm, w.num_writes = imm, len(writes)
        for k, (rail, more) in enumerate(writes):
            w.writes[k].rail, w.writes[k].more = rail, more
            w.writes[k].src, w.writes[k].len, w.writes[k].dest, w.writes[k].key = 0x1000 + k, 64, 0x2000 + k, 7
        if meta is not None:
            w.has_meta, w.meta_rail, w.meta_more = 1, meta[0], meta[1]
            w.meta[0], w.meta[2], w.meta[3] = 0x55, 8, 1
        req = ctypes.c_int32(-7)
        rc = self.fn("iput_signal")(self.tx, peer, ctypes.byref(w), ctypes.byref(req))
        return rc, req.value

    def ack(self, peer, msg):
        return self.fn("send_ack")(self.tx, peer, msg)

    def progress(self):
        return self.fn("progress")(self.tx)

    def test(self, req):
        done = ctypes.c_int(-1)
        rc = self.fn("test")(self.tx, req, ctypes.byref(done))
        return rc, done.value

    def stats(self):
        st = self.mod.GinTxStats()
        self.fn("stats")(self.tx, ctypes.byref(st))
        return {f[0]: getattr(st, f[0]) for f in st._fields_ if f[0] != "pad"}

    def close(self):
        self.fn("destroy")(self.tx)


@pytest.fixture(params=["oracle", "product"])
def which(request):
    return request.param


def test_refused_posts_queue_and_retry_without_fi_more(which, oracle, lib):
    """Send queues of one entry per rail.  Pool entries are handed out lowest first and the entry
    freed last is handed out next, so the contexts below are fixed.
      op A = entry 0: write0 (entry 1) rail 0 with FI_MORE (first stripe of a put-signal), write1
        (entry 2) rail 1, metadata (entry 3) rail 0: rail 0 is full -> queued.  iputSignal still
        succeeds (:768-771, :840-842).
      op B = entry 4: one deferred write (entry 5) on rail 0 with FI_MORE -> refused, queued behind 3.
      progress without completions: only the head of the queue (3) is tried again; it is refused, so
        5 is not tried (retry_pending_reqs stops at the first -FI_EAGAIN, :592-593).
      rail 0's entry completes; progress: the CQs of all four rails are read (rail 0 gives entry 1,
        then nothing), then 3 is posted, then 5 is tried -- without FI_MORE now, although it has
        never been accepted (post() drops the flag at the first attempt) -- and refused again.
      entries 2 and 3 complete; progress reads 3 (rail 0) then 2 (rail 1), posts 5.
      op A is done; its entry 0 is freed last, after 3 and 2: the next operation is entry 0 again
      and its write is entry 2."""
    e = Engine(which, oracle, lib, (1,))
    f = e.fabric
    assert e.op([(0, 1), (1, 0)], meta=(0, 0)) == (0, 0)
    assert f.take_log() == [("post", W, 0, 1, 1), ("post", W, 1, 0, 2), ("refused", M, 0, 0, 3)]
    assert e.op([(0, 1)]) == (0, 4)
    assert f.take_log() == [("refused", W, 0, 1, 5)]
    st = e.stats()
    assert (st["posts"], st["refused"], st["pending"], st["requests"]) == (2, 2, 2, 6)

    assert e.progress() == 0
    assert f.take_log() == [("cq_read", 0, 0), ("cq_read", 1, 0), ("cq_read", 2, 0), ("cq_read", 3, 0),
                            ("refused", M, 0, 0, 3)]
    assert e.test(0) == (0, 0) and e.test(4) == (0, 0)

    f.complete(0)
    assert e.progress() == 0
    assert f.take_log() == [("cq_read", 0, 1), ("cq_read", 0, 0), ("cq_read", 1, 0), ("cq_read", 2, 0),
                            ("cq_read", 3, 0), ("post", M, 0, 0, 3), ("refused", W, 0, 0, 5)]
    assert e.test(0) == (0, 0)                       # write1 and the metadata send are still out

    f.complete(0)
    f.complete(1)
    assert e.progress() == 0
    assert f.take_log() == [("cq_read", 0, 1), ("cq_read", 0, 0), ("cq_read", 1, 1), ("cq_read", 1, 0),
                            ("cq_read", 2, 0), ("cq_read", 3, 0), ("post", W, 0, 0, 5)]
    assert e.test(0) == (0, 1)                       # done: the request is freed by this call
    assert e.test(0)[0] == EINVAL
    assert e.test(4) == (0, 0)
    st = e.stats()
    assert (st["retries"], st["retried_ok"], st["completions"], st["pending"], st["pending_max"]) == (4, 2, 3, 0, 2)
    assert st["requests"] == 2                       # op B and its write

    assert e.op([(2, 0)]) == (0, 0)
    assert f.take_log() == [("post", W, 2, 0, 2)]
    e.close()


def test_retry_stops_at_the_head_and_a_new_post_overtakes(which, oracle, lib):
    """Queue = [X on rail 0, Y on rail 1].  Rail 1 drains, rail 0 does not: the retry tries X, is
    refused, and leaves Y queued although its rail has room; the next operation's write on rail 1
    is posted at once and so overtakes Y (the target reassembles by sequence number)."""
    e = Engine(which, oracle, lib, (1,))
    f = e.fabric
    assert e.op([(0, 0)]) == (0, 0) and e.op([(1, 0)]) == (0, 2)          # fill rails 0 and 1
    assert e.op([(0, 0)]) == (0, 4) and e.op([(1, 0)]) == (0, 6)          # X = 5, Y = 7, both queued
    f.take_log()
    f.complete(1)
    assert e.progress() == 0
    assert [x for x in f.take_log() if x[0] != "cq_read"] == [("refused", W, 0, 0, 5)]
    assert e.stats()["pending"] == 2
    assert e.op([(1, 0)])[0] == 0
    # entry 3 (the completed write of rail 1) was freed last: the new operation takes it, its write
    # the next untouched entry
    assert f.take_log() == [("post", W, 1, 0, 8)]
    f.complete(0)
    assert e.progress() == 0
    assert [x for x in f.take_log() if x[0] != "cq_read"] == [("post", W, 0, 0, 5), ("refused", W, 1, 0, 7)]
    e.close()


@pytest.mark.parametrize("count,iters", [(4, 4), (2, 3), (8, 1)])
def test_progress_reads_a_bounded_number_of_completions_per_rail(which, oracle, lib, count, iters):
    """gin_process_cq_rail (:89-150): at most cq_read_count entries per read and at most
    cq_process_max_iter reads per rail and progress call; a read that returns nothing ends the rail
    early, a short read does not."""
    e = Engine(which, oracle, lib, (1000,), cq_read_count=count, max_iter=iters, max_requests=400, rails=2)
    f = e.fabric
    for _ in range(40):
        assert e.op([(0, 0)])[0] == 0
    for _ in range(3):
        assert e.op([(1, 0)])[0] == 0
    f.complete(0, 40)
    f.complete(1, 3)
    f.take_log()
    left0, left1 = 40, 3
    while left0 or left1:
        assert e.progress() == 0
        want = []
        for rail, left in ((0, left0), (1, left1)):
            for _ in range(iters):
                got = min(count, left)
                want.append(("cq_read", rail, got))
                left -= got
                if got == 0:
                    break
            if rail == 0:
                left0 = left
            else:
                left1 = left
        assert f.take_log() == want
    assert e.stats()["completions"] == 43
    # by hand for the default 4 x 4: 16 + 16 + 8 from rail 0, the 3 of rail 1 in the first call
    if (count, iters) == (4, 4):
        assert e.stats()["requests"] == 43           # the operations wait for test()
    e.close()


def test_a_failed_post_gives_the_operation_up(which, oracle, lib):
    """A post that fails with anything but -FI_EAGAIN (:772-783): the error is returned, the failed
    request and the umbrella go back to the pool, the write already posted completes without a
    parent to report to."""
    e = Engine(which, oracle, lib, (4, (2, EIO)))
    f = e.fabric
    assert e.op([(0, 1), (1, 0)], meta=(0, 0)) == (EIO, -1)
    assert f.take_log() == [("post", W, 0, 1, 1), ("failed", W, 1, 0, 2)]
    assert e.stats()["requests"] == 1
    f.complete(0)
    assert e.progress() == 0
    assert e.stats()["requests"] == 0 and e.stats()["completions"] == 1
    # the pool is a stack: the umbrella (0) was freed after the failed write (2), entry 1 last
    assert e.op([(3, 0)]) == (0, 1)
    assert f.take_log()[-1] == ("post", W, 3, 0, 0)
    e.close()


def test_acks_go_out_on_rail_zero_and_are_counted_while_in_flight(which, oracle, lib):
    e = Engine(which, oracle, lib, (1,))
    f = e.fabric
    assert e.ack(3, 0x601D) == 0 and e.ack(4, 0x701D) == 0
    assert f.take_log() == [("post", A, 0, 0, 0), ("refused", A, 0, 0, 1)]
    assert e.stats()["outstanding_acks"] == 1        # counted when the post is accepted (:187-189)
    f.complete(0)
    assert e.progress() == 0
    assert e.stats()["outstanding_acks"] == 1        # the first completed, the second went out
    f.complete(0)
    assert e.progress() == 0
    st = e.stats()
    assert (st["outstanding_acks"], st["requests"], st["completions"]) == (0, 0, 2)
    e.close()


def test_pool_exhaustion_posts_nothing(which, oracle, lib):
    e = Engine(which, oracle, lib, (8,), max_requests=5)
    f = e.fabric
    assert e.op([(0, 0), (1, 0), (2, 0), (3, 0)], meta=(0, 0)) == (ENOMEM, -1)      # needs 6
    assert f.take_log() == [] and e.stats()["requests"] == 0
    assert e.op([(0, 0), (1, 0), (2, 0), (3, 0)]) == (0, 0)                          # needs 5
    assert e.ack(0, 1) == ENOMEM
    e.close()


def test_an_unknown_completion_context_is_an_error(which, oracle, lib):
    e = Engine(which, oracle, lib, (8,))
    assert e.op([(0, 0)]) == (0, 0)
    e.fabric.cq[2].append(40)                        # a context no request owns
    assert e.progress() == EINVAL
    e.fabric.cq[2].clear()
    e.fabric.cq[1].append(0)                         # the umbrella is not a post
    assert e.progress() == EINVAL
    e.close()


@pytest.mark.parametrize("seed", range(6))
def test_random_scripts_oracle_and_product_agree(oracle, lib, seed):
    """The same random program (operations with 0-4 writes and optional metadata, ACKs, partial
    completions, progress and test calls) against both engines, each on its own copy of the
    scripted fabric: identical fabric logs, return values and counters."""
    logs = []
    for which in ("oracle", "product"):
        rng = np.random.default_rng(seed)
        e = Engine(which, oracle, lib, (int(rng.integers(1, 4)),), cq_read_count=int(rng.integers(1, 5)),
                   max_iter=int(rng.integers(1, 4)), max_requests=48)
        f, trace, open_reqs = e.fabric, [], []
        for step in range(1500):
            r = rng.random()
            if r < 0.45:
                nw = int(rng.integers(0, 5))
                writes = [(int(rng.integers(0, 4)), int(rng.integers(0, 2))) for _ in range(nw)]
                meta = (int(rng.integers(0, 4)), int(rng.integers(0, 2))) if (nw == 0 or rng.random() < 0.3) else None
                rc, req = e.op(writes, meta, peer=int(rng.integers(0, 3)))
                trace.append(("op", rc, req))
                if rc == 0:
                    open_reqs.append(req)
            elif r < 0.55:
                trace.append(("ack", e.ack(int(rng.integers(0, 3)), int(rng.integers(0, 1 << 20)))))
            elif r < 0.8:
                rail = int(rng.integers(0, 4))
                f.complete(rail, min(len(f.sq[rail]), int(rng.integers(0, 4))))
            elif r < 0.93:
                trace.append(("progress", e.progress()))
            elif open_reqs:
                req = open_reqs[int(rng.integers(0, len(open_reqs)))]
                rc, done = e.test(req)
                trace.append(("test", req, rc, done))
                if done:
                    open_reqs.remove(req)
        for _ in range(200):                          # drain: everything completes in the end
            for rail in range(4):
                f.complete(rail, len(f.sq[rail]))
            trace.append(("progress", e.progress()))
        trace.append(tuple(e.test(r) for r in open_reqs))
        logs.append((f.take_log(), trace, e.stats()))
        e.close()
    assert logs[0][1] == logs[1][1]
    assert logs[0][0] == logs[1][0]
    assert logs[0][2] == logs[1][2]
    st = logs[1][2]
    assert st["refused"] > 50 and st["retried_ok"] == st["refused"] and st["pending"] == 0
    assert st["requests"] == 0 and st["outstanding_acks"] == 0
    assert all(done == (0, 1) for done in logs[1][1][-1])


# ---- the product's in-process fabric ----

def test_loop_fabric_send_queue_doorbells_and_completions(lib):
    """Depth 3 on two rails.  Posts with FI_MORE wait for a doorbell: a later post without it on
    the same rail, or the queue filling up.  Transmission order is the order the doorbells rang,
    per rail in post order; a taken post's completion is readable; reading it frees the entry."""
    fab = ctypes.c_void_p()
    assert lib.ofi_amd_loopfab_create(2, 3, ctypes.byref(fab)) == 0
    ops = m.GinFabricOps()
    assert lib.ofi_amd_loopfab_ops(fab, ctypes.byref(ops)) == 0
    out = (m.GinPost * 16)()
    ctxs = (ctypes.c_uint32 * 16)()

    def post(rail, more, ctx):
        return ops.post(ops.fabric, ctypes.byref(m.GinPost(W, rail, more, ctx, 0, 0, 0, 0, 0, 0)))

    def taken():
        n = lib.ofi_amd_loopfab_take_transmitted(fab, out, 16)
        return [(out[i].rail, out[i].context) for i in range(n)]

    def read(rail, cap=16):
        n = ops.cq_read(ops.fabric, rail, ctxs, cap)
        return [ctxs[i] for i in range(n)]

    assert post(0, 1, 10) == 0 and post(0, 1, 11) == 0 and taken() == []       # deferred: nothing on the wire
    assert post(1, 0, 20) == 0 and taken() == [(1, 20)]
    assert read(0) == [] and read(1) == [20]
    assert post(0, 0, 12) == 0                                                 # rings rail 0: 10, 11, 12 go
    assert post(0, 0, 13) == EAGAIN                                            # three entries: full
    assert taken() == [(0, 10), (0, 11), (0, 12)]
    assert read(0, 2) == [10, 11]                                              # two entries free again
    assert post(0, 1, 13) == 0 and post(0, 1, 14) == 0                         # 12, 13, 14: full -> rings itself
    assert post(0, 0, 15) == EAGAIN
    assert taken() == [(0, 13), (0, 14)]
    assert read(0) == [12, 13, 14] and read(0) == []
    assert post(3, 0, 1) == EINVAL
    # one at a time and in place: the same order, the same completions, NULL when nothing waits
    def next_one():
        p = lib.ofi_amd_loopfab_next_transmitted(fab)
        return (p.contents.rail, p.contents.context) if p else None

    assert post(1, 1, 30) == 0 and post(0, 0, 31) == 0 and post(1, 0, 32) == 0
    assert next_one() == (0, 31) and next_one() == (1, 30)
    assert read(1) == [30] and read(0) == [31]           # taken: readable; the third is still on its way
    assert next_one() == (1, 32) and next_one() is None and read(1) == [32]
    assert not lib.ofi_amd_loopfab_next_transmitted(None)
    assert lib.ofi_amd_loopfab_destroy(fab) == 0
    assert lib.ofi_amd_loopfab_create(0, 3, ctypes.byref(fab)) == EINVAL
    assert lib.ofi_amd_loopfab_create(2, 0, ctypes.byref(fab)) == EINVAL


def test_engine_rejects_bad_arguments(lib):
    tx = ctypes.c_void_p()
    fab = Fabric(m, 4, 1)
    assert lib.ofi_amd_gin_tx_create(0, 4, 4, 8, ctypes.byref(fab.ops), ctypes.byref(tx)) == EINVAL
    assert lib.ofi_amd_gin_tx_create(5, 4, 4, 8, ctypes.byref(fab.ops), ctypes.byref(tx)) == EINVAL
    assert lib.ofi_amd_gin_tx_create(4, 0, 4, 8, ctypes.byref(fab.ops), ctypes.byref(tx)) == EINVAL
    assert lib.ofi_amd_gin_tx_create(4, 4, 0, 8, ctypes.byref(fab.ops), ctypes.byref(tx)) == EINVAL
    assert lib.ofi_amd_gin_tx_create(4, 4, 4, 0, ctypes.byref(fab.ops), ctypes.byref(tx)) == EINVAL
    assert lib.ofi_amd_gin_tx_create(4, 4, 4, 8, None, ctypes.byref(tx)) == EINVAL
    assert lib.ofi_amd_gin_tx_create(4, 4, 4, 8, ctypes.byref(fab.ops), ctypes.byref(tx)) == 0
    w = m.GinWire()
    req = ctypes.c_int32()
    w.num_writes = 5
    assert lib.ofi_amd_gin_tx_iput_signal(tx, 0, ctypes.byref(w), ctypes.byref(req)) == EINVAL
    w.num_writes, w.writes[0].rail = 1, 4
    assert lib.ofi_amd_gin_tx_iput_signal(tx, 0, ctypes.byref(w), ctypes.byref(req)) == EINVAL
    assert fab.log == []
    assert lib.ofi_amd_gin_tx_test(tx, 3, ctypes.byref(ctypes.c_int())) == EINVAL
    assert lib.ofi_amd_gin_tx_destroy(tx) == 0 and lib.ofi_amd_gin_tx_destroy(None) == EINVAL
