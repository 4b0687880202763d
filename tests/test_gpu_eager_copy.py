"""Eager arrivals in rx-buffer format (8-byte header + payload) copied to receive buffers at
arbitrary alignment: destination bytes, byte counts and flush words bit-exact against the
oracle's per-buffer memcpy loop, and nothing written outside [dst, dst + count)."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import _oracle
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

RX_STRIDE = 8320          # 8200-byte rx buffer rounded up to the 128-byte alignment


def make_case(rng, n, max_len=8184, truncate_some=True):
    recv_len = rng.integers(0, max_len + 1, n).astype(np.uint32)
    rx_off = (rng.permutation(n).astype(np.uint64)) * np.uint64(RX_STRIDE)
    dst_len = recv_len.copy()
    if truncate_some:
        cut = rng.random(n) < 0.2
        dst_len[cut] = (recv_len[cut] * rng.random(int(cut.sum()))).astype(np.uint32)
        grow = rng.random(n) < 0.2
        dst_len[grow] += 100
    # destinations packed with random gaps and random alignment, guard bytes between them
    room = np.minimum(recv_len, dst_len).astype(np.uint64)
    gaps = rng.integers(1, 40, n).astype(np.uint64)
    starts = (np.cumsum(room + gaps) - room).astype(np.uint64)
    arena_bytes = int(starts[-1] + room[-1]) + 64
    rx = rng.integers(0, 256, n * RX_STRIDE, dtype=np.uint8)
    return rx, rx_off, recv_len, starts, dst_len, arena_bytes


def expected(oracle, rx, rx_off, recv_len, dst_off, dst_len, arena_bytes, fill):
    arena = np.full(arena_bytes, fill, dtype=np.uint8)
    copied = np.zeros(len(recv_len), dtype=np.uint32)
    oracle.oracle_eager_copy_batch(_oracle.ptr(rx), _oracle.ptr(rx_off), _oracle.ptr(recv_len),
                                   _oracle.ptr(arena), _oracle.ptr(dst_off), _oracle.ptr(dst_len),
                                   len(recv_len), _oracle.ptr(copied))
    flush = np.zeros(len(recv_len), dtype=np.uint32)
    for i in range(len(recv_len)):
        k = min(4, int(copied[i]))
        flush[i] = int.from_bytes(arena[int(dst_off[i]):int(dst_off[i]) + k].tobytes(), "little")
    return arena, copied, flush


def run_gpu(lib, rx_dev_ptr, rx_off, recv_len, dst_off, dst_len, arena_bytes, fill, base_offset=0,
            want_flush=True):
    n = len(recv_len)
    d_arena = torch.full((arena_bytes + base_offset,), fill, dtype=torch.uint8, device="cuda")
    d = [_gpu.to_dev(x) for x in (rx_off, recv_len, dst_off, dst_len)]
    d_copied = torch.zeros(n, dtype=torch.int32, device="cuda")
    d_flush = torch.zeros(n, dtype=torch.int32, device="cuda")
    rc = lib.ofi_amd_eager_copy_batch(ctypes.c_void_p(rx_dev_ptr), d[0].data_ptr(), d[1].data_ptr(),
                                      ctypes.c_void_p(d_arena.data_ptr() + base_offset),
                                      d[2].data_ptr(), d[3].data_ptr(), n, d_copied.data_ptr(),
                                      d_flush.data_ptr() if want_flush else None, _gpu.stream())
    assert rc == 0
    _gpu.sync()
    return (_gpu.to_host(d_arena, np.uint8)[base_offset:], _gpu.to_host(d_copied, np.uint32),
            _gpu.to_host(d_flush, np.uint32))


@pytest.mark.parametrize("n,seed", [(1, 1), (257, 2), (5000, 3), (20000, 4)])
def test_random_alignment_and_truncation(lib, oracle, gpu, n, seed):
    rng = np.random.default_rng(seed)
    rx, rx_off, recv_len, dst_off, dst_len, arena_bytes = make_case(rng, n)
    want_arena, want_copied, want_flush = expected(oracle, rx, rx_off, recv_len, dst_off, dst_len,
                                                   arena_bytes, 0xA5)
    d_rx = _gpu.to_dev(rx)
    for base_offset in (0, 1, 7):             # shifts every destination's alignment
        arena, copied, flush = run_gpu(lib, d_rx.data_ptr(), rx_off, recv_len, dst_off, dst_len,
                                       arena_bytes, 0xA5, base_offset)
        assert np.array_equal(copied, want_copied)
        assert np.array_equal(arena, want_arena)        # includes every guard byte
        assert np.array_equal(flush, want_flush)


def test_every_short_length_at_every_alignment(lib, oracle, gpu):
    """lengths 0..200 x destination alignment 0..63 x source alignment (rx_off + 8) fixed by
    the format: the head (up to the destination's first 64-byte boundary) / body (whole 64-byte
    units) / tail (up to 63 bytes) split is exercised at each boundary, three bytes apart so
    that a byte written outside a buffer lands in its neighbour or in the fill"""
    lens, offs = [], []
    pos = 0
    for length in range(0, 201):
        for align in range(64):
            start = (pos + 63) // 64 * 64 + align
            offs.append(start)
            lens.append(length)
            pos = start + length + 3
    n = len(lens)
    rng = np.random.default_rng(5)
    recv_len = np.array(lens, dtype=np.uint32)
    dst_off = np.array(offs, dtype=np.uint64)
    rx_off = np.arange(n, dtype=np.uint64) * np.uint64(RX_STRIDE)
    rx = rng.integers(0, 256, n * RX_STRIDE, dtype=np.uint8)
    arena_bytes = pos + 64
    want = expected(oracle, rx, rx_off, recv_len, dst_off, recv_len, arena_bytes, 0x11)
    d_rx = _gpu.to_dev(rx)
    got = run_gpu(lib, d_rx.data_ptr(), rx_off, recv_len, dst_off, recv_len, arena_bytes, 0x11)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_unaligned_rx_buffers_and_large_payloads(lib, oracle, gpu):
    """The format only fixes payload = buffer + 8; buffers themselves may sit at any byte
    (a test of the source-side funnel shift), and payloads may exceed one 8 KiB trip."""
    rng = np.random.default_rng(6)
    n = 300
    recv_len = rng.integers(0, 40000, n).astype(np.uint32)
    stride = 40100
    rx_off = np.arange(n, dtype=np.uint64) * np.uint64(stride) + rng.integers(0, 64, n).astype(np.uint64)
    rx = rng.integers(0, 256, n * stride + 128, dtype=np.uint8)
    room = recv_len.astype(np.uint64) + rng.integers(1, 30, n).astype(np.uint64)
    dst_off = (np.cumsum(room) - room).astype(np.uint64)
    arena_bytes = int(dst_off[-1] + room[-1]) + 64
    want = expected(oracle, rx, rx_off, recv_len, dst_off, recv_len, arena_bytes, 0)
    d_rx = _gpu.to_dev(rx)
    got = run_gpu(lib, d_rx.data_ptr(), rx_off, recv_len, dst_off, recv_len, arena_bytes, 0, base_offset=3)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_rx_buffers_in_pinned_host_memory(lib, oracle, gpu):
    """The reference's rx buffers are host memory the NIC writes; the kernel reads them in place."""
    rng = np.random.default_rng(7)
    n = 2000
    rx, rx_off, recv_len, dst_off, dst_len, arena_bytes = make_case(rng, n)
    pinned = torch.empty(len(rx), dtype=torch.uint8, pin_memory=True)
    pinned.numpy()[:] = rx
    want = expected(oracle, rx, rx_off, recv_len, dst_off, dst_len, arena_bytes, 0x3C)
    got = run_gpu(lib, pinned.data_ptr(), rx_off, recv_len, dst_off, dst_len, arena_bytes, 0x3C)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_headers_written_by_the_sender_side_codec_are_skipped(lib, oracle, gpu):
    """End to end with the wire codec: headers from ofi_amd_eager_tx_assign in front of each
    payload; the copy must deliver the payload only."""
    rng = np.random.default_rng(8)
    n = 64
    tx = m.EagerTx()
    lib.ofi_amd_eager_tx_init(ctypes.byref(tx))
    rx = np.zeros(n * RX_STRIDE, dtype=np.uint8)
    recv_len = rng.integers(1, 8185, n).astype(np.uint32)
    payloads = []
    for i in range(n):
        h = m.EagerHdr()
        lib.ofi_amd_eager_tx_assign(ctypes.byref(tx), 1000 + i, ctypes.byref(h))
        if i % 5 == 4:
            lib.ofi_amd_eager_tx_advance(ctypes.byref(tx))
        rx[i * RX_STRIDE:i * RX_STRIDE + 8] = np.frombuffer(bytes(h), dtype=np.uint8)
        p = rng.integers(0, 256, int(recv_len[i]), dtype=np.uint8)
        rx[i * RX_STRIDE + 8:i * RX_STRIDE + 8 + len(p)] = p
        payloads.append(p)
    rx_off = np.arange(n, dtype=np.uint64) * np.uint64(RX_STRIDE)
    dst_off = np.arange(n, dtype=np.uint64) * np.uint64(8192 + 64) + np.uint64(5)
    arena_bytes = n * (8192 + 64) + 64
    d_rx = _gpu.to_dev(rx)                    # stays referenced until the copy has run
    arena, copied, _f = run_gpu(lib, d_rx.data_ptr(), rx_off, recv_len, dst_off, recv_len,
                                arena_bytes, 0)
    assert np.array_equal(copied, recv_len)
    for i in range(n):
        assert np.array_equal(arena[int(dst_off[i]):int(dst_off[i]) + len(payloads[i])], payloads[i])


def test_bad_arguments(lib, gpu):
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")
    p = t.data_ptr()
    assert lib.ofi_amd_eager_copy_batch(p, p, p, p, p, p, 0, None, None, _gpu.stream()) == 0
    assert lib.ofi_amd_eager_copy_batch(None, p, p, p, p, p, 1, None, None, _gpu.stream()) == -22
    assert lib.ofi_amd_eager_copy_batch(p, None, p, p, p, p, 1, None, None, _gpu.stream()) == -22
    assert lib.ofi_amd_eager_copy_batch(p, p, p, p, p, None, 1, None, None, _gpu.stream()) == -22
    _gpu.sync()
