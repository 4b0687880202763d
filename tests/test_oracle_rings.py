"""Pins the ring oracle: the behaviour cases of the reference's tests/unit/mpsc_ring.cpp
and spsc_ring.cpp, and a side-by-side run against the reference headers compiled as-is."""
import ctypes

import numpy as np
import pytest

import _oracle

u32 = ctypes.c_uint32
u64 = ctypes.c_uint64


class Ring:
    def __init__(self, oracle, cap, width=4):
        self.o, self.w = oracle, width
        self.r = oracle.oracle_mpsc_create(cap, width)
        assert self.r

    def push(self, v):
        b = (u32 if self.w == 4 else u64)(v)
        return self.o.oracle_mpsc_push(self.r, ctypes.byref(b))

    def pop(self):
        b = (u32 if self.w == 4 else u64)(0xDEAD)
        ok = self.o.oracle_mpsc_pop(self.r, ctypes.byref(b))
        return (ok, b.value)

    def close(self):
        self.o.oracle_mpsc_destroy(self.r)


def test_empty_pop(oracle):                       # mpsc_ring.cpp:16-21
    r = Ring(oracle, 4)
    assert r.pop()[0] == 0
    r.close()


def test_push_pop_fifo(oracle):                   # :23-36
    r = Ring(oracle, 8)
    for i in range(8):
        assert r.push(i) == 1
    for i in range(8):
        assert r.pop() == (1, i)
    assert r.pop()[0] == 0
    r.close()


def test_full_uses_all_slots(oracle):             # :41-57
    r = Ring(oracle, 4)
    for v in (10, 11, 12, 13):
        assert r.push(v) == 1
    assert r.push(14) == 0
    assert r.pop() == (1, 10)
    assert r.push(14) == 1
    assert r.push(15) == 0
    r.close()


def test_wraparound(oracle):                      # :61-71
    r = Ring(oracle, 4)
    for i in range(100):
        assert r.push(i) == 1
        assert r.pop() == (1, i)
        assert r.pop()[0] == 0
    r.close()


def test_interleaved(oracle):                     # :74-97
    r = Ring(oracle, 4)
    assert r.push(1) and r.push(2)
    assert r.pop() == (1, 1)
    assert r.push(3) and r.push(4) and r.push(5)
    assert r.push(6) == 0
    for v in (2, 3, 4, 5):
        assert r.pop() == (1, v)
    assert r.pop()[0] == 0
    r.close()


def test_position_wrap_at_2_32(oracle):
    # positions are 32-bit and wrap; the signed sequence difference keeps working
    r = Ring(oracle, 8)
    oracle.oracle_mpsc_set_positions(r.r, 0xFFFFFFFA)
    for lap in range(5):
        for i in range(8):
            assert r.push(lap * 8 + i) == 1
        assert r.push(999) == 0
        for i in range(8):
            assert r.pop() == (1, lap * 8 + i)
        assert r.pop()[0] == 0
    r.close()


def test_capacity_must_be_power_of_two(oracle):   # static_assert, mpsc_ring.h:57-58
    assert not oracle.oracle_mpsc_create(6, 4)
    assert not oracle.oracle_mpsc_create(0, 4)


def test_single_producer_threaded_fifo(oracle):   # :101-124
    assert oracle.oracle_mpsc_stress(1024, 1, 300000) == 0


def test_four_producers_threaded(oracle):         # :134-189
    assert oracle.oracle_mpsc_stress(1024, 4, 100000) == 0
    assert oracle.oracle_mpsc_stress(8, 4, 20000) == 0    # tiny ring: mostly-full regime


def test_spsc_holds_capacity_minus_one(oracle):   # tests/unit/spsc_ring.cpp
    r = oracle.oracle_spsc_create(8, 8)
    v = u64(0)
    assert oracle.oracle_spsc_pop(r, ctypes.byref(v)) == 0
    for i in range(7):
        assert oracle.oracle_spsc_push(r, ctypes.byref(u64(i))) == 1
    assert oracle.oracle_spsc_push(r, ctypes.byref(u64(7))) == 0
    for i in range(7):
        assert oracle.oracle_spsc_pop(r, ctypes.byref(v)) == 1 and v.value == i
    assert oracle.oracle_spsc_pop(r, ctypes.byref(v)) == 0
    for i in range(50):   # wrap
        assert oracle.oracle_spsc_push(r, ctypes.byref(u64(i))) == 1
        assert oracle.oracle_spsc_pop(r, ctypes.byref(v)) == 1 and v.value == i
    oracle.oracle_spsc_destroy(r)


@pytest.mark.parametrize("kind,cap,width", [(1, 8, 8), (2, 1024, 8), (0, 4096, 64)])
def test_side_by_side_with_reference_header(oracle, ref, kind, cap, width):
    """Same random push/pop script on nccl_ofi_mpsc_ring (compiled from the reference) and
    on the oracle: every return code and every popped payload must agree."""
    rng = np.random.default_rng(kind)
    rr = ref.ref_mpsc_create(kind)
    orr = oracle.oracle_mpsc_create(cap, width)
    bias = 0.5
    for step in range(40000):
        if step % 5000 == 0:
            bias = rng.choice([0.3, 0.5, 0.7])   # drift between mostly-empty and mostly-full
        if rng.random() < bias:
            payload = rng.integers(0, 256, width, dtype=np.uint8)
            a = ref.ref_mpsc_push(kind, rr, _oracle.ptr(payload))
            b = oracle.oracle_mpsc_push(orr, _oracle.ptr(payload))
            assert a == b
        else:
            pa = np.zeros(width, dtype=np.uint8)
            pb = np.zeros(width, dtype=np.uint8)
            a = ref.ref_mpsc_pop(kind, rr, _oracle.ptr(pa))
            b = oracle.oracle_mpsc_pop(orr, _oracle.ptr(pb))
            assert a == b
            if a:
                assert np.array_equal(pa, pb)
    ref.ref_mpsc_destroy(kind, rr)
    oracle.oracle_mpsc_destroy(orr)


def test_spsc_side_by_side(oracle, ref):
    rng = np.random.default_rng(9)
    rr = ref.ref_spsc_create()
    orr = oracle.oracle_spsc_create(8, 8)
    for _ in range(20000):
        if rng.random() < 0.55:
            v = int(rng.integers(0, 1 << 60))
            assert ref.ref_spsc_push(rr, v) == oracle.oracle_spsc_push(orr, ctypes.byref(u64(v)))
        else:
            a, b = u64(0), u64(0)
            ra = ref.ref_spsc_pop(rr, ctypes.byref(a))
            rb = oracle.oracle_spsc_pop(orr, ctypes.byref(b))
            assert ra == rb and (not ra or a.value == b.value)
    ref.ref_spsc_destroy(rr)
    oracle.oracle_spsc_destroy(orr)


@pytest.mark.parametrize("producers", [1, 3])
def test_cpu_producers_through_rings_deliver_the_seeded_stream(oracle, producers):
    """Producer threads -> one ring per context -> one consumer: what the consumer folds is the
    seeded stream itself, whatever the interleaving (small rings, so full and wrap both occur)."""
    ck, secs = ctypes.c_uint64(), ctypes.c_double()
    assert oracle.oracle_gin_cpu_rings_run(7, 12, 3000, 64, producers, 1, 64, 1, 1,
                                           ctypes.byref(ck), ctypes.byref(secs)) == 0
    want = oracle.oracle_gin_stream_checksum(7, 12, 3000, 1, 64, 1, 1, 0, 4, 131072, 64, 1,
                                             _oracle.default_mrs())
    assert ck.value == want and secs.value > 0
    assert oracle.oracle_gin_cpu_rings_run(7, 2, 10, 64, 3, 1, 64, 1, 1, ctypes.byref(ck),
                                           ctypes.byref(secs)) == -22    # more producers than contexts
