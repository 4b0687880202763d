"""Builds receiver-side completion streams from sender-side wire records (test helper).

A sender op becomes `num_writes` write-with-immediate completions plus, when it carries a
signal, one 32-byte metadata message.  The network may deliver those in any order; the
helper reorders them within a bounded look-ahead so that no more than `window` ops are
ever outstanding (the sender's TX window guarantees < 8192 on the wire)."""
import ctypes

import numpy as np

from _oracle import GinComm, GinDesc, GinMr, GinWire

INC, ADD = 1, 2
NO_MR = 0xFFFF


def make_mrs(sig_base=0x7F0000000000):
    mrs = (GinMr * 3)()
    for i, m in enumerate(mrs):
        m.local_base = 0x100000000 * (i + 1)
        m.remote_address = 0x200000000 * (i + 1)
        m.remote_address_offset = 0
        for r in range(4):
            m.key[r] = 0x1000 * (i + 1) + r
    mrs[2].remote_address = sig_base
    return mrs


def sender_ops(oracle, ops, comm_id=5, rails=4, ack_model=1, sig_base=0x7F0000000000, feedback=None):
    """ops: list of (size, signal_op, value, sig_off).  Returns the wire records
    [(imm, num_writes, meta or None, ack_req, seq)].  `feedback(comm, k)` may be called
    after op k to apply ACKs to the sender."""
    c = GinComm()
    oracle.oracle_gin_comm_init(ctypes.byref(c), comm_id, rails, 131072, 64, ack_model)
    mrs = make_mrs(sig_base)
    out = []
    for k, (size, sop, val, soff) in enumerate(ops):
        d = GinDesc(8 * k, 8 * k, size, soff, val, 1, sop, 0, 0, 0, 1, 2 if sop else NO_MR,
                    2 if sop else 1)
        w = GinWire()
        rc = oracle.oracle_gin_iput_signal(ctypes.byref(c), mrs, ctypes.byref(d), ctypes.byref(w))
        assert rc == 0, "sender refused op %d: %d" % (k, rc)
        meta = [int(x) for x in w.meta] if w.has_meta else None
        out.append((int(w.imm), int(w.num_writes), meta, int(w.ack_req), int(w.seq)))
        if feedback is not None:
            feedback(c, k)
    return out


def events_of(wire):
    """[(op index, 'w', imm) | (op index, 'm', meta)] in issue order"""
    ev = []
    for k, (imm, nw, meta, _ack, _seq) in enumerate(wire):
        ev += [(k, "w", imm)] * nw
        if meta is not None:
            ev.append((k, "m", meta))
    return ev


def reorder(events, rng, lookahead):
    """Random arrival order in which an event overtakes at most `lookahead` ops."""
    if lookahead <= 0:
        return list(events)
    keyed = [(k + float(rng.uniform(0, lookahead)), i) for i, (k, _t, _p) in enumerate(events)]
    keyed.sort()
    return [events[i] for _key, i in keyed]


def feed(api, rx, peer, events):
    """api: (write_fn, meta_fn) taking (rx, peer, payload)"""
    write_fn, meta_fn = api
    for _k, kind, payload in events:
        if kind == "w":
            rc = write_fn(rx, peer, payload)
        else:
            arr = (ctypes.c_uint64 * 4)(*payload)
            rc = meta_fn(rx, peer, arr)
        assert rc == 0


def take_all(take_fn, rx, struct, chunk=4096):
    out = []
    buf = (struct * chunk)()
    while True:
        n = take_fn(rx, buf, chunk)
        out += [tuple(getattr(buf[i], f[0]) for f in struct._fields_) for i in range(n)]
        if n < chunk:
            return out


def slot_sums(work, n_slots, base):
    """Independent end state: per-slot sum of delivered values (mod 2^64)."""
    acc = np.zeros(n_slots, dtype=np.uint64)
    for b, off, val, _peer, _gate, _run in work:
        assert b == base and off % 8 == 0
        acc[off // 8] = np.uint64((int(acc[off // 8]) + val) % (1 << 64))
    return acc
