"""Pins the bounce-copy oracle: plain byte-copy semantics (the reference's eager copy is a NIC
loop-back read, src/nccl_ofi_rdma.cpp:2729-2776, so there is no arithmetic to match) and the
copy patterns of the reference's device-copy unit test, tests/unit/gdrcopy.cpp:15-133."""
import numpy as np

import _oracle
from aws_ofi_nccl_amd import synthetic


def run(oracle, src, arena, src_off, dst_off, length):
    n = len(length)
    flush = np.zeros(n, dtype=np.uint32)
    oracle.oracle_bounce_scatter(_oracle.ptr(src), _oracle.ptr(arena), _oracle.ptr(src_off),
                                 _oracle.ptr(dst_off), _oracle.ptr(length), n, _oracle.ptr(flush))
    return flush


def test_matches_numpy_slicing(oracle):
    w = synthetic.bounce_workload(11, n=2000, arena_bytes=32 << 20)
    src = synthetic.random_bytes(11, w["src_bytes"])
    arena = np.full(w["arena_bytes"], 0xCC, dtype=np.uint8)
    want = arena.copy()
    for s, d, l in zip(w["src_off"], w["dst_off"], w["len"]):
        want[int(d):int(d) + int(l)] = src[int(s):int(s) + int(l)]
    flush = run(oracle, src, arena, w["src_off"], w["dst_off"], w["len"])
    assert np.array_equal(arena, want)                  # nothing outside [dst, dst+len) changed
    first = np.stack([want[int(d):int(d) + 4] for d in w["dst_off"]]).view(np.uint32)[:, 0]
    assert np.array_equal(flush, first)


def test_workload_generator_properties():
    w = synthetic.bounce_workload(3, n=65536, arena_bytes=2 << 30)
    assert w["len"].min() == 0 and w["len"].max() == 8192
    assert np.all(w["dst_off"] % 64 == 0)
    order = np.argsort(w["dst_off"])
    end = w["dst_off"][order] + np.maximum(1, w["len"][order])
    assert np.all(end[:-1] <= w["dst_off"][order][1:])   # disjoint
    assert int(end[-1]) <= 2 << 30
    assert w["dst_off"].max() > (3 << 29)               # spread over the arena
    assert np.array_equal(w["src_off"][1:], np.cumsum(w["len"][:-1], dtype=np.uint64))


def test_gdrcopy_patterns(oracle):
    # 2 MiB of 'A' in one copy (tests/unit/gdrcopy.cpp:15-75)
    size = 2 << 20
    src = np.full(size, ord("A"), dtype=np.uint8)
    arena = np.zeros(size, dtype=np.uint8)
    flush = run(oracle, src, arena, np.zeros(1, np.uint64), np.zeros(1, np.uint64),
                np.array([size], np.uint32))
    assert np.all(arena == ord("A")) and flush[0] == 0x41414141
    # ten single-byte writes at offsets 0..9 (:78-133): each call is one 1-byte buffer
    arena = np.zeros(64, dtype=np.uint8)
    for i in range(10):
        byte = np.array([ord("a") + i], dtype=np.uint8)
        oracle.oracle_bounce_scatter(_oracle.ptr(byte), _oracle.ptr(arena[i:]),
                                     _oracle.ptr(np.zeros(1, np.uint64)),
                                     _oracle.ptr(np.zeros(1, np.uint64)),
                                     _oracle.ptr(np.ones(1, np.uint32)), 1, None)
    assert bytes(arena[:10]) == b"abcdefghij" and not arena[10:].any()


def test_zero_length_is_a_no_op(oracle):
    arena = np.full(256, 7, dtype=np.uint8)
    src = np.arange(16, dtype=np.uint8)
    flush = run(oracle, src, arena, np.array([3, 5], np.uint64), np.array([64, 128], np.uint64),
                np.array([0, 0], np.uint32))
    assert np.all(arena == 7) and list(flush) == [0x07070707] * 2
