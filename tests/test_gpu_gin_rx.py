"""GIN signal delivery on the GPU: work items produced by the receiver become atomic adds on
counters in HBM; the counters must end bit-exact where the oracle's batch-wise
read-modify-write path (and a plain scatter-add) leaves them."""
import ctypes

import numpy as np
import pytest
import torch

import _gin_rx as G
import _gpu
import _oracle
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

SIG_BASE = 0x7F0000000000
c_u32 = ctypes.c_uint32


def work_array(items):
    """[(base, offset, value, peer, gate_seq, run_len)] -> packed bytes of ofi_amd_gin_signal_work_t"""
    dt = np.dtype([("base", "<u8"), ("offset", "<u8"), ("value", "<u8"), ("peer", "<u4"),
                   ("gate_seq", "<u2"), ("run_len", "<u2")])
    assert dt.itemsize == ctypes.sizeof(m.GinSignalWork) == 32
    a = np.zeros(len(items), dtype=dt)
    for i, it in enumerate(items):
        a[i] = it
    return a


def oracle_apply(oracle, work, regions, batch=64):
    """The reference-shaped path: batches of 64 work items, folded per slot, one r-m-w each."""
    n_r = len(regions)
    bases = (ctypes.c_uint64 * n_r)(*[b for b, _c in regions])
    sizes = (ctypes.c_uint64 * n_r)(*[c.nbytes for _b, c in regions])
    ptrs = (ctypes.c_void_p * n_r)(*[c.ctypes.data for _b, c in regions])
    raw = work.tobytes()
    for lo in range(0, len(work), batch):
        n = min(batch, len(work) - lo)
        buf = (_oracle.GinSignalWork * n).from_buffer_copy(raw[32 * lo:32 * (lo + n)])
        assert oracle.oracle_gin_signal_apply(buf, n, bases, sizes, ptrs, n_r) > 0


def gpu_apply(lib, work, dev_regions, rejected=None):
    d_work = _gpu.to_dev(work.view(np.uint8))
    regs = (m.GinSignalRegion * len(dev_regions))()
    for i, (base, t) in enumerate(dev_regions):
        regs[i] = m.GinSignalRegion(base, t.numel() * 8, t.data_ptr())
    rc = lib.ofi_amd_gin_signal_apply(ctypes.c_void_p(d_work.data_ptr()), len(work), regs,
                                      len(dev_regions),
                                      ctypes.c_void_p(rejected.data_ptr()) if rejected is not None else None,
                                      _gpu.stream())
    _gpu.sync()
    return rc


def test_receiver_stream_to_counters(lib, oracle, gpu):
    """Sender wire records -> reordered completions -> product receiver -> GPU counters."""
    rng = np.random.default_rng(41)
    slots = 512
    ops = []
    for i in range(7000):
        size = int(2 ** rng.uniform(3, 20))
        if i % 3 == 0:
            ops.append((size, G.INC, 0, 8 * ((i // 64) % slots)))
        elif i % 3 == 1:
            ops.append((size, G.ADD, int(rng.integers(0, 1 << 64, dtype=np.uint64)),
                        8 * int(rng.integers(0, slots))))
        else:
            ops.append((size, 0, 0, 0))
    wire = G.sender_ops(oracle, ops, ack_model=0)
    ev = G.reorder(G.events_of(wire), rng, 30)
    prx = ctypes.c_void_p()
    assert lib.ofi_amd_gin_rx_create(1, None, ctypes.byref(prx)) == 0
    G.feed((lib.ofi_amd_gin_rx_write_completion, lib.ofi_amd_gin_rx_metadata), prx, 0, ev)
    items = G.take_all(lib.ofi_amd_gin_rx_take_work, prx, m.GinSignalWork)
    assert lib.ofi_amd_gin_rx_destroy(prx) == 0
    assert sum(it[5] for it in items) == sum(1 for o in ops if o[1])

    work = work_array(items)
    start = rng.integers(0, 1 << 64, slots, dtype=np.uint64)
    host = start.copy()
    oracle_apply(oracle, work, [(SIG_BASE, host)])
    # straight from the ops, without receiver or folding
    want = [int(x) for x in start]
    for _size, sop, val, off in ops:
        if sop:
            want[off // 8] = (want[off // 8] + (1 if sop == G.INC else val)) % (1 << 64)
    assert [int(x) for x in host] == want

    d_cnt = _gpu.to_dev(start)
    assert gpu_apply(lib, work, [(SIG_BASE, d_cnt)]) == 0
    assert np.array_equal(_gpu.to_host(d_cnt, np.uint64), host)


@pytest.mark.parametrize("n,slots", [(1, 1), (63, 2), (100000, 8), (1 << 20, 512), (300000, 1 << 16)])
def test_contended_slots_bit_exact(lib, oracle, gpu, n, slots):
    rng = np.random.default_rng(n + slots)
    vals = rng.integers(0, 1 << 64, n, dtype=np.uint64)
    idx = rng.integers(0, slots, n)
    dt_items = np.zeros(n, dtype=work_array([]).dtype)
    dt_items["base"] = SIG_BASE
    dt_items["offset"] = 8 * idx.astype(np.uint64)
    dt_items["value"] = vals
    dt_items["run_len"] = 1
    start = rng.integers(0, 1 << 64, slots, dtype=np.uint64)
    want = start.copy()
    with np.errstate(over="ignore"):
        np.add.at(want, idx, vals)
    if n <= 100000:
        host = start.copy()
        oracle_apply(oracle, dt_items, [(SIG_BASE, host)])
        assert np.array_equal(host, want)
    d_cnt = _gpu.to_dev(start)
    assert gpu_apply(lib, dt_items, [(SIG_BASE, d_cnt)]) == 0
    assert np.array_equal(_gpu.to_host(d_cnt, np.uint64), want)
    # a second batch accumulates on top
    assert gpu_apply(lib, dt_items, [(SIG_BASE, d_cnt)]) == 0
    with np.errstate(over="ignore"):
        np.add.at(want, idx, vals)
    assert np.array_equal(_gpu.to_host(d_cnt, np.uint64), want)


def test_several_regions_and_rejects(lib, oracle, gpu):
    rng = np.random.default_rng(43)
    bases = [SIG_BASE + (i << 32) for i in range(16)]
    sizes = [int(rng.integers(1, 200)) for _ in bases]
    host = [np.zeros(s, dtype=np.uint64) for s in sizes]
    items, n_bad = [], 0
    for i in range(20000):
        r = int(rng.integers(0, 16))
        kind = rng.random()
        if kind < 0.9:
            s = int(rng.integers(0, sizes[r]))
            v = int(rng.integers(0, 1 << 64, dtype=np.uint64))
            items.append((bases[r], 8 * s, v, 0, i & 0x1FFF, 1))
            host[r][s] = np.uint64((int(host[r][s]) + v) % (1 << 64))
        elif kind < 0.94:
            items.append((bases[r] + 8, 0, 1, 0, 0, 1)); n_bad += 1          # unknown base
        elif kind < 0.97:
            items.append((bases[r], 8 * sizes[r], 1, 0, 0, 1)); n_bad += 1   # one past the end
        else:
            items.append((bases[r], 4, 1, 0, 0, 1)); n_bad += 1              # misaligned
    work = work_array(items)
    dev = [(b, torch.zeros(s + 1, dtype=torch.int64, device="cuda")) for b, s in zip(bases, sizes)]
    # the extra trailing word per region is a canary: declared size excludes it
    regs = [(b, t[:-1]) for b, t in dev]
    rejected = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert gpu_apply(lib, work, regs, rejected) == 0
    assert int(rejected.item()) == n_bad and n_bad > 500
    for (b, t), h in zip(dev, host):
        got = _gpu.to_host(t, np.uint64)
        assert np.array_equal(got[:-1], h)
        assert got[-1] == 0


def test_windows_backed_by_several_segments(lib, oracle, gpu):
    """Four windows of one to four contiguous segments each (16 regions, every segment an allocation of its
    own with a canary word behind it): items addressed by a window's base and an offset anywhere in the
    window, or by a later segment's own base, against the oracle; items past a window, straddling
    nothing (a counter never straddles: sizes are multiples of 8) and misaligned ones are rejected."""
    rng = np.random.default_rng(47)
    windows, regions = [], []                      # windows: (base, [segment sizes in counters])
    for w in range(4):
        base = SIG_BASE + (w << 32)
        segs = [int(rng.integers(1, 60)) for _ in range(1 + w)] + ([int(rng.integers(1, 60)) for _ in range(3 - w)] if w == 0 else [])
        windows.append((base, len(regions), segs))
        at = base
        for sz in segs:
            regions.append((at, sz))
            at += 8 * sz
    while len(regions) < 16:                       # unrelated single regions far away
        regions.append((SIG_BASE + (len(regions) << 36), int(rng.integers(1, 60))))
    host = [np.zeros(sz, dtype=np.uint64) for _b, sz in regions]
    items, n_bad = [], 0
    for i in range(20000):
        base, first, segs = windows[int(rng.integers(0, len(windows)))]
        total = sum(segs)
        kind = rng.random()
        if kind < 0.85:
            slot = int(rng.integers(0, total))
            start = int(rng.integers(0, len(segs))) if rng.random() < 0.3 else 0    # address by a later segment's base
            skip = sum(segs[:start])
            if slot < skip:
                start, skip = 0, 0
            v = int(rng.integers(0, 1 << 64, dtype=np.uint64))
            items.append((base + 8 * skip, 8 * (slot - skip), v, 0, i & 0x1FFF, 1))
            k, rem = 0, slot
            while rem >= segs[k]:
                rem -= segs[k]
                k += 1
            host[first + k][rem] = np.uint64((int(host[first + k][rem]) + v) % (1 << 64))
        elif kind < 0.93:
            items.append((base, 8 * total, 1, 0, 0, 1)); n_bad += 1                  # one past the window
        else:
            items.append((base, 8 * int(rng.integers(0, total)) + 4, 1, 0, 0, 1)); n_bad += 1   # misaligned
    work = work_array(items)
    good = work_array([it for it in items if it[1] % 8 == 0 and not any(it[0] == b and it[1] == 8 * sum(sg) for b, _f, sg in windows)])
    oracle_host = [np.zeros(sz, dtype=np.uint64) for _b, sz in regions]
    oracle_apply(oracle, good, [(b, h) for (b, _sz), h in zip(regions, oracle_host)])
    for a, b in zip(host, oracle_host):
        assert np.array_equal(a, b)                # the oracle agrees with the image built by hand above
    dev = [(b, torch.zeros(sz + 1, dtype=torch.int64, device="cuda")) for b, sz in regions]
    rejected = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert gpu_apply(lib, work, [(b, t[:-1]) for b, t in dev], rejected) == 0
    assert int(rejected.item()) == n_bad and n_bad > 1000
    for (b, t), h in zip(dev, host):
        got = _gpu.to_host(t, np.uint64)
        assert np.array_equal(got[:-1], h) and got[-1] == 0


def test_work_items_in_pinned_host_memory(lib, oracle, gpu):
    """The proxy writes work items into pinned host memory and launches straight from there."""
    n = 5000
    rng = np.random.default_rng(44)
    work = work_array([(SIG_BASE, 8 * int(rng.integers(0, 32)), int(rng.integers(0, 1 << 62)), 0,
                        i & 0x1FFF, 1) for i in range(n)])
    pinned = torch.empty(work.nbytes, dtype=torch.uint8, pin_memory=True)
    pinned.numpy()[:] = work.view(np.uint8)
    d_cnt = torch.zeros(32, dtype=torch.int64, device="cuda")
    regs = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, 256, d_cnt.data_ptr()))
    assert lib.ofi_amd_gin_signal_apply(ctypes.c_void_p(pinned.data_ptr()), n, regs, 1, None,
                                        _gpu.stream()) == 0
    _gpu.sync()
    want = np.zeros(32, dtype=np.uint64)
    np.add.at(want, (work["offset"] // 8).astype(np.int64), work["value"])
    assert np.array_equal(_gpu.to_host(d_cnt, np.uint64), want)


def test_bad_arguments(lib, gpu):
    d_cnt = torch.zeros(8, dtype=torch.int64, device="cuda")
    regs = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, 64, d_cnt.data_ptr()))
    d_work = torch.zeros(32, dtype=torch.uint8, device="cuda")
    p = ctypes.c_void_p(d_work.data_ptr())
    assert lib.ofi_amd_gin_signal_apply(p, 0, regs, 1, None, _gpu.stream()) == 0
    assert lib.ofi_amd_gin_signal_apply(None, 1, regs, 1, None, _gpu.stream()) == -22
    assert lib.ofi_amd_gin_signal_apply(p, 1, None, 1, None, _gpu.stream()) == -22
    assert lib.ofi_amd_gin_signal_apply(p, 1, regs, 0, None, _gpu.stream()) == -22
    assert lib.ofi_amd_gin_signal_apply(p, 1, regs, 17, None, _gpu.stream()) == -22
    odd = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, 64, d_cnt.data_ptr() + 4))
    assert lib.ofi_amd_gin_signal_apply(p, 1, odd, 1, None, _gpu.stream()) == -22
    _gpu.sync()


@pytest.mark.parametrize("n,slots", [(0, 1), (1, 1), (257, 2), (4096, 8), (65536, 64)])
def test_adds_and_the_flush_read_behind_them_in_one_launch(lib, oracle, gpu, n, slots):
    """ofi_amd_gin_signal_apply_post: the counters end where ofi_amd_gin_signal_apply leaves them (the
    oracle's batch-wise path and a plain scatter-add), the slots hold the flush buffer's words afterwards, and
    a host that polls the slot's flag and then has the counters copied by a kernel on another stream, without
    waiting for the launch's stream, already finds every add: they were performed before the flush buffer was read back."""
    rng = np.random.default_rng(n + slots)
    vals = rng.integers(0, 1 << 64, n, dtype=np.uint64)
    idx = rng.integers(0, slots, n)
    items = np.zeros(n, dtype=work_array([]).dtype)
    items["base"], items["offset"], items["value"], items["run_len"] = SIG_BASE, 8 * idx.astype(np.uint64), vals, 1
    start = rng.integers(0, 1 << 64, slots, dtype=np.uint64)
    want = start.copy()
    with np.errstate(over="ignore"):
        np.add.at(want, idx, vals)
    if 0 < n <= 4096:
        host = start.copy()
        oracle_apply(oracle, items, [(SIG_BASE, host)])
        assert np.array_equal(host, want)
    sentinel = 0xdeadbeefdeadbeef
    d_flush = torch.zeros(8, dtype=torch.int64, device="cuda")
    assert lib.ofi_amd_flush_buffer_fill(ctypes.c_void_p(d_flush.data_ptr()), sentinel, _gpu.stream()) == 0
    slots_host = torch.zeros(4 * 8, dtype=torch.int64, pin_memory=True)
    d_cnt = _gpu.to_dev(start)
    d_work = _gpu.to_dev(items.view(np.uint8)) if n else torch.zeros(32, dtype=torch.uint8, device="cuda")
    regs = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, slots * 8, d_cnt.data_ptr()))
    other = torch.cuda.Stream()
    _gpu.sync()
    for rails, rounds in ((4, 1), (1, 2)):
        slots_host.zero_()
        rc = lib.ofi_amd_gin_signal_apply_post(ctypes.c_void_p(d_work.data_ptr()), n, regs, 1, None,
                                               ctypes.c_void_p(d_flush.data_ptr()),
                                               ctypes.c_void_p(slots_host.data_ptr()), rails, _gpu.stream())
        assert rc == 0
        for _ in range(10_000_000):
            if lib.ofi_amd_flush_test(ctypes.c_void_p(slots_host.data_ptr()), rails, sentinel) == 1:
                break
        else:
            raise AssertionError("the flag never showed")
        with torch.cuda.stream(other):                   # not the launch's stream, and no wait for it
            snapshot = d_cnt.clone()
        other.synchronize()
        seen = _gpu.to_host(snapshot, np.uint64)
        if rounds == 2:
            with np.errstate(over="ignore"):
                np.add.at(want, idx, vals)
        assert np.array_equal(seen, want)
        got = slots_host.numpy().view(np.uint64)
        assert all(int(w) == sentinel for w in got[:8 * rails]) and not got[8 * rails:].any()
    _gpu.sync()


def test_apply_post_arguments(lib, gpu):
    d = torch.zeros(64, dtype=torch.int64, device="cuda")
    slots_host = torch.zeros(32, dtype=torch.int64, pin_memory=True)
    regs = (m.GinSignalRegion * 1)(m.GinSignalRegion(SIG_BASE, 64, d.data_ptr()))
    p, s = ctypes.c_void_p(d.data_ptr()), ctypes.c_void_p(slots_host.data_ptr())
    f = lambda *a: lib.ofi_amd_gin_signal_apply_post(*a, _gpu.stream())
    assert f(p, 65537, regs, 1, None, p, s, 1) == -7          # -E2BIG: more than one workgroup takes
    assert f(p, 1, regs, 1, None, None, s, 1) == -22 and f(p, 1, regs, 1, None, p, None, 1) == -22
    assert f(p, 1, regs, 1, None, p, s, 0) == -22 and f(p, 1, regs, 1, None, p, s, 5) == -22
    assert f(None, 1, regs, 1, None, p, s, 1) == -22 and f(p, 1, None, 1, None, p, s, 1) == -22
    assert f(p, 1, regs, 17, None, p, s, 1) == -22
    assert f(None, 0, None, 0, None, p, s, 1) == 0            # the flush read alone needs no work and no regions
    _gpu.sync()
