"""A sender and a receiver of the send/receive protocol joined by a wire the test controls.

The same harness drives the oracle's state machines (oracle_*) and the product's (ofi_amd_*):
`Link(flavour)` creates one send comm and one receive comm, posts sends and receives, and moves
what the state machines hand out -- eager messages, RDMA writes, eager copies -- between the
two ends in whatever order the test asks for.  Payloads are labels: `memory[dst]` records
which send's label, and how many bytes of it, ended up in which receive buffer.
"""
import ctypes

import _oracle
import aws_ofi_nccl_amd as m

EAGER_SEND_SIZE = 8192
AGAIN, EAGER, WRITE = 0, 1, 2


class Flavour:
    def __init__(self, lib, prefix, mod):
        self.lib, self.prefix, self.mod = lib, prefix, mod
        self.is_oracle = prefix == "oracle_"

    def fn(self, name):
        return getattr(self.lib, self.prefix + name)


def flavours(oracle, lib):
    return {"oracle": Flavour(oracle, "oracle_", _oracle), "product": Flavour(lib, "ofi_amd_", m)}


class Link:
    def __init__(self, fl, num_rails=4, eager_send_size=EAGER_SEND_SIZE, comm_id=77,
                 min_stripe=131072, max_small=64):
        self.fl, self.num_rails = fl, num_rails
        if fl.is_oracle:
            self.s = ctypes.c_void_p(fl.fn("send_comm_create")(comm_id, num_rails, eager_send_size,
                                                               min_stripe, max_small))
            self.r = ctypes.c_void_p(fl.fn("recv_comm_create")(num_rails))
            assert self.s.value and self.r.value
        else:
            self.s, self.r = ctypes.c_void_p(), ctypes.c_void_p()
            assert fl.fn("send_comm_create")(comm_id, num_rails, eager_send_size, min_stripe, max_small,
                                             ctypes.byref(self.s)) == 0
            assert fl.fn("recv_comm_create")(num_rails, ctypes.byref(self.r)) == 0
        self.mailbox = fl.fn("send_comm_mailbox")(self.s)
        self.sends = []          # per send handle: dict(req, label, size, tag, kind, done, reported)
        self.recvs = []          # per recv handle: dict(req, seq, n, dsts, sizes, tags, done, reported)
        self.wire = []           # in flight: ("eager", send handle, action) / ("write", handle, action, k)
        self.rx = {}             # rx cookie -> (label, recv_len)
        self.next_cookie = 1
        self.memory = {}         # dst address -> (label, bytes)
        self.trace = []          # every decision, for oracle/product comparison
        self.next_dst = 0x10000000
        self.strict = True       # False: a write for a receive that is gone is recorded, not fatal

    def close(self):
        self.fl.fn("send_comm_destroy")(self.s)
        self.fl.fn("recv_comm_destroy")(self.r)

    # ------------------------------------------------------------------ sender
    def send(self, size, tag, label):
        """One isend call: a handle, or None when the plugin says "call again"."""
        act = self.fl.mod.SendAction()
        rc = self.fl.fn("send_comm_send")(self.s, size, tag, ctypes.byref(act))
        assert rc == 0, rc
        xf = tuple((act.xfers[k].rail_id, act.xfers[k].offset, act.xfers[k].msg_size)
                   for k in range(act.num_xfers))
        self.trace.append(("send", size, tag, act.kind, act.msg_seq_num, act.recv_idx, act.imm,
                           (act.hdr.eager_offset, act.hdr.prev_batch_count, act.hdr.eager_seq, act.hdr.tag)
                           if act.kind == EAGER else None, act.size, act.remote_buff_offset, xf,
                           act.no_target_completion))
        if act.kind == AGAIN:
            assert act.req == -1
            return None
        h = len(self.sends)
        self.sends.append(dict(req=act.req, label=label, size=size, tag=tag, kind=act.kind, done=False,
                               reported=None))
        if act.kind == EAGER:
            self.wire.append(("eager", h, act, 0))
        else:
            for k in range(act.num_xfers):
                self.wire.append(("write", h, act, k))
        return h

    def test_send(self, h):
        s = self.sends[h]
        if s["done"]:
            return True
        done, size = ctypes.c_int(), ctypes.c_uint64()
        assert self.fl.fn("send_comm_test")(self.s, s["req"], ctypes.byref(done), ctypes.byref(size)) == 0
        if done.value:
            s["done"], s["reported"] = True, size.value
            self.trace.append(("send_done", h, size.value))
        return bool(done.value)

    # ---------------------------------------------------------------- receiver
    def recv(self, tags, sizes, completion_optional=0):
        n = len(tags)
        dsts = [self.next_dst + 0x100000 * i for i in range(n)]
        self.next_dst += 0x100000 * 8
        keys = [0xA000 + 16 * len(self.recvs) + 4 * i + r for i in range(n) for r in range(self.num_rails)]
        req, seq = ctypes.c_int32(), ctypes.c_uint16()
        rc = self.fl.fn("recv_comm_recv")(self.r, n, (ctypes.c_uint64 * n)(*dsts), (ctypes.c_uint64 * n)(*sizes),
                                          (ctypes.c_int * n)(*tags), (ctypes.c_uint64 * len(keys))(*keys),
                                          completion_optional, self.mailbox, ctypes.byref(req),
                                          ctypes.byref(seq))
        self.trace.append(("recv", tuple(tags), tuple(sizes), rc, seq.value if rc == 0 else None))
        if rc != 0:
            return rc
        h = len(self.recvs)
        self.recvs.append(dict(req=req.value, seq=seq.value, n=n, dsts=dsts, sizes=list(sizes),
                               tags=list(tags), done=False, reported=None))
        # the control message is in the sender's mailbox already; its post completes at once
        assert self.fl.fn("recv_comm_ctrl_sent")(self.r, req.value) == 0
        self.copies()
        return h

    def copies(self):
        """Execute the eager copies the receiver has decided on."""
        items = (self.fl.mod.EagerCopyItem * 64)()
        while True:
            k = self.fl.fn("recv_comm_take_copies")(self.r, items, 64)
            if k == 0:
                return
            for i in range(k):
                it = items[i]
                label, recv_len = self.rx.pop(it.rx_cookie)
                assert recv_len == it.recv_len
                self.trace.append(("copy", label, it.dst, it.dst_len, it.recv_len, it.sub_idx, it.needs_copy))
                self.memory.setdefault(it.dst, []).append([label, min(it.recv_len, it.dst_len), None])
                if it.needs_copy:
                    assert self.fl.fn("recv_comm_copy_done")(self.r, it.req, it.sub_idx) == 0

    def test_recv(self, h):
        r = self.recvs[h]
        if r["done"]:
            return True
        done, sizes = ctypes.c_int(), (ctypes.c_int * 8)()
        assert self.fl.fn("recv_comm_test")(self.r, r["req"], ctypes.byref(done), sizes) == 0
        if done.value:
            r["done"], r["reported"] = True, [sizes[i] for i in range(r["n"])]
            self.trace.append(("recv_done", h, tuple(r["reported"])))
        return bool(done.value)

    # -------------------------------------------------------------------- wire
    def deliver(self, order=None):
        """Everything in flight reaches the other end, in `order` (indices into the in-flight
        list; default: as sent), and the sender gets its completions."""
        flight, self.wire = self.wire, []
        for idx in (order if order is not None else range(len(flight))):
            kind, h, act, k = flight[idx]
            s = self.sends[h]
            if kind == "eager":
                cookie = self.next_cookie
                self.next_cookie += 1
                self.rx[cookie] = (s["label"], act.size)
                hdr = self.fl.mod.EagerHdr(act.hdr.eager_offset, act.hdr.prev_batch_count,
                                           act.hdr.eager_seq, act.hdr.tag)
                rc = self.fl.fn("recv_comm_eager_arrival")(self.r, act.msg_seq_num, ctypes.byref(hdr),
                                                           act.size, cookie)
                assert rc == 0, rc
                self.copies()
            else:
                x = act.xfers[k]
                ent = self.memory.setdefault(act.remote_buff_offset, [])
                mine = [e for e in ent if e[2] == h]
                if mine:
                    mine[0][1] += x.msg_size
                else:
                    ent.append([s["label"], x.msg_size, h])
                if not act.no_target_completion:
                    rc = self.fl.fn("recv_comm_write_arrival")(self.r, act.imm, x.msg_size)
                    self.trace.append(("write_arrival", act.imm, x.msg_size, rc))
                    assert rc == 0 or not self.strict, rc
            assert self.fl.fn("send_comm_completion")(self.s, s["req"]) == 0

    # ------------------------------------------------------------------ states
    def send_state(self):
        st = self.fl.mod.SendState()
        self.fl.fn("send_comm_state")(self.s, ctypes.byref(st))
        return {f[0]: getattr(st, f[0]) for f in st._fields_ if not f[0].startswith("pad")}

    def recv_state(self):
        st = self.fl.mod.RecvState()
        self.fl.fn("recv_comm_state")(self.r, ctypes.byref(st))
        return {f[0]: getattr(st, f[0]) for f in st._fields_ if not f[0].startswith("pad")}

    # ----------------------------------------------------------------- helpers
    def post_sends_interleaved(self, msgs, pump=None, max_rounds=200):
        """The rotating send queue of the reference's functional test: sends that get "call
        again" are retried in later rounds, and within a round a tag that failed blocks later
        sends of the same tag.  `pump()` runs between rounds (deliveries, receiver progress).
        msgs: list of (size, tag, label).  Returns the handles in msgs order."""
        handles = [None] * len(msgs)
        queue = list(range(len(msgs)))
        for _ in range(max_rounds):
            if not queue:
                return handles
            blocked, again = set(), []
            for i in queue:
                size, tag, label = msgs[i]
                if tag in blocked:
                    again.append(i)
                    continue
                h = self.send(size, tag, label)
                if h is None:
                    blocked.add(tag)
                    again.append(i)
                else:
                    handles[i] = h
            queue = again
            if pump:
                pump()
        raise AssertionError("sends did not drain: %r" % (queue,))

    def run_to_completion(self, max_rounds=50):
        for _ in range(max_rounds):
            self.deliver()
            self.copies()
            s_done = all([self.test_send(h) for h in range(len(self.sends))])
            r_done = all([self.test_recv(h) for h in range(len(self.recvs))])
            if s_done and r_done and not self.wire:
                return
        raise AssertionError("link did not quiesce: sends %r recvs %r" % (
            [s["done"] for s in self.sends], [r["done"] for r in self.recvs]))

    def landed(self, recv_handle, sub=0):
        """[(label, bytes)] written into that receive buffer."""
        return [(e[0], e[1]) for e in self.memory.get(self.recvs[recv_handle]["dsts"][sub], [])]
