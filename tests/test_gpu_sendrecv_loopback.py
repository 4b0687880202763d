"""The send/receive path end to end in one process on one GPU (ofi_amd_sendrecv_loopback_run):
send comm and receive comm state machines, eager sends through rx buffers and the batched eager
copy, rendezvous as striped device copies.  Checked byte for byte against the source buffers.

Sizes: the ten (send, receive) pairs of the reference's tests/functional/
nccl_message_transfer.cpp:44-56 with NCCL_NET_MAX_REQUESTS = 32 requests each, and the
powers of two of the configured sweep, 8 B to 1 GiB: 64 in flight up to 1 MiB, then as many as
128 MiB hold, and 4 / 4 / 2 / 2 messages of 128 MiB / 256 MiB / 512 MiB / 1 GiB."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

RX_STRIDE = 8320
PAIRS = [(512, 512), (4096, 4096), (16384, 16384), (1 << 20, 1 << 20), (5120, 4096), (17408, 16384),
         (2 << 20, 1 << 20), (4096, 5120), (16384, 17408), (1 << 20, 2 << 20)]


def run(lib, send_sizes, recv_sizes, inflight, flags=0, dst_skew=0, seed=0, group=1, tags=None):
    """Distinct source and receive buffers per message; returns (stats, per-message check)."""
    n = len(send_sizes)
    rng = np.random.default_rng(seed)
    srcs = [torch.from_numpy(rng.integers(0, 256, max(s, 1), dtype=np.uint8)).cuda() for s in send_sizes]
    dsts = [torch.full((max(r, 1) + 64,), 0xCD, dtype=torch.uint8, device="cuda") for r in recv_sizes]
    pool = torch.zeros(inflight * RX_STRIDE, dtype=torch.uint8, device="cuda")
    a_src = np.array([t.data_ptr() for t in srcs], dtype=np.uint64)
    a_dst = np.array([t.data_ptr() + dst_skew for t in dsts], dtype=np.uint64)
    a_size = np.array(send_sizes, dtype=np.uint64)
    a_cap = np.array(recv_sizes, dtype=np.uint64)
    stats = m.SendrecvLoopbackStats()
    torch.cuda.synchronize()
    a_tags = None if tags is None else np.array(tags, dtype=np.int32)
    rc = lib.ofi_amd_sendrecv_loopback_run(a_src.ctypes.data, a_dst.ctypes.data, a_size.ctypes.data,
                                           a_cap.ctypes.data, None if tags is None else a_tags.ctypes.data, n,
                                           inflight, 4, group, pool.data_ptr(),
                                           pool.numel(), flags, _gpu.stream(), ctypes.byref(stats))
    assert rc == 0, rc
    torch.cuda.synchronize()
    for i in range(n):
        k = min(send_sizes[i], recv_sizes[i])
        got = dsts[i].cpu().numpy()
        want = srcs[i].cpu().numpy()
        assert np.array_equal(got[dst_skew:dst_skew + k], want[:k]), (i, send_sizes[i], recv_sizes[i])
        assert np.all(got[:dst_skew] == 0xCD) and np.all(got[dst_skew + k:] == 0xCD), (i, "wrote outside")
    assert stats.messages == n and stats.payload_bytes == sum(min(s, r) for s, r in zip(send_sizes, recv_sizes))
    assert stats.eager_messages + stats.write_messages == n
    assert stats.flushes <= stats.rounds and (stats.flushes == stats.rounds or 0 in send_sizes)
    return stats


def test_round_without_a_byte_needs_no_flush(lib, gpu):
    st = run(lib, [0] * 64 + [8] * 64, [16] * 128, 64)
    assert st.rounds == 2 and st.flushes == 1 and st.eager_messages == 128


@pytest.mark.parametrize("pair", PAIRS)
def test_reference_size_pairs_thirty_two_requests_each(lib, gpu, pair):
    send, recv = pair
    st = run(lib, [send] * 32, [recv] * 32, 32, seed=send + recv)
    if send + 8 <= 8192:
        assert st.eager_messages >= 1                # the sender was ahead of the receiver
    else:
        assert st.eager_messages == 0 and st.write_messages == 32


def test_power_of_two_sweep_sixty_four_in_flight(lib, gpu):
    sizes = [8 << k for k in range(24)]                       # 8 B .. 64 MiB
    for size in sizes:
        count = 64 if size <= (1 << 20) else max(2, (128 << 20) // size)
        st = run(lib, [size] * count, [size] * count, 64, seed=size)
        stripes = 1 if size <= 131072 else (2 if size <= 262144 else 4)
        if size + 8 > 8192:
            assert st.rdma_writes == count * stripes


@pytest.mark.parametrize("size,count", [(128 << 20, 4), (256 << 20, 4), (512 << 20, 2), (1 << 30, 2)])
def test_power_of_two_sweep_large_messages(lib, gpu, size, count):
    """The top of the configured sweep.  Payloads are random 16-bit words (bf16 bit patterns)
    generated on the device; every received byte, and the guard bytes behind each receive
    buffer, are compared on the device."""
    gen = torch.Generator(device="cuda").manual_seed(size + count)
    srcs = [torch.randint(-32768, 32768, (size // 2,), dtype=torch.int16, device="cuda", generator=gen)
            for _ in range(count)]
    dsts = [torch.full((size // 2 + 32,), 0x4DCD, dtype=torch.int16, device="cuda") for _ in range(count)]
    pool = torch.zeros(64 * RX_STRIDE, dtype=torch.uint8, device="cuda")
    a_src = np.array([t.data_ptr() for t in srcs], dtype=np.uint64)
    a_dst = np.array([t.data_ptr() for t in dsts], dtype=np.uint64)
    a_size = np.array([size] * count, dtype=np.uint64)
    stats = m.SendrecvLoopbackStats()
    torch.cuda.synchronize()
    rc = lib.ofi_amd_sendrecv_loopback_run(a_src.ctypes.data, a_dst.ctypes.data, a_size.ctypes.data,
                                           a_size.ctypes.data, None, count, 64, 4, 1, pool.data_ptr(),
                                           pool.numel(), 0, _gpu.stream(), ctypes.byref(stats))
    assert rc == 0, rc
    torch.cuda.synchronize()
    for i in range(count):
        assert torch.equal(dsts[i][:size // 2], srcs[i]), (i, size)
        assert bool((dsts[i][size // 2:] == 0x4DCD).all()), (i, "wrote past the receive buffer")
    assert stats.messages == count and stats.payload_bytes == size * count
    assert stats.write_messages == count and stats.rdma_writes == 4 * count and stats.eager_messages == 0
    # one table entry per RDMA write: a stripe is not cut (the copy launch gives each 8 KiB a wavefront)
    assert stats.copy_entries == count * 4


@pytest.mark.parametrize("size", [2 << 20, 64 << 20, 1 << 30])
def test_sixty_four_in_flight_above_one_mebibyte(lib, gpu, size):
    """The configured depth at the sizes where a message is striped writes: 64 messages open at
    once, each with a source and a receive buffer of its own (2 x 64 GiB at 1 GiB, which the
    288 GB of the part hold), random 16-bit words (bf16 bit patterns) generated on the device.
    Every received byte and the guard words behind each receive buffer are compared on the
    device (tests/functional/nccl_message_transfer.cpp:45-56 checks the same on the host)."""
    count, guard = 64, 32
    free_bytes, _ = torch.cuda.mem_get_info()
    if 2 * count * (size + 2 * guard) + (4 << 30) > free_bytes:
        pytest.skip("needs %d GiB of free device memory" % ((2 * count * size) >> 30))
    src = torch.empty(count * (size // 2), dtype=torch.int16, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(size)
    for k in range(count):
        src[k * (size // 2):(k + 1) * (size // 2)].random_(-32768, 32767, generator=gen)
    stride = size // 2 + guard
    dst = torch.full((count * stride,), 0x4DCD, dtype=torch.int16, device="cuda")
    pool = torch.zeros(64 * RX_STRIDE, dtype=torch.uint8, device="cuda")
    a_src = np.array([src.data_ptr() + k * size for k in range(count)], dtype=np.uint64)
    a_dst = np.array([dst.data_ptr() + 2 * k * stride for k in range(count)], dtype=np.uint64)
    a_size = np.full(count, size, dtype=np.uint64)
    stats = m.SendrecvLoopbackStats()
    torch.cuda.synchronize()
    rc = lib.ofi_amd_sendrecv_loopback_run(a_src.ctypes.data, a_dst.ctypes.data, a_size.ctypes.data,
                                           a_size.ctypes.data, None, count, 64, 4, 1, pool.data_ptr(),
                                           pool.numel(), 0, _gpu.stream(), ctypes.byref(stats))
    assert rc == 0, rc
    torch.cuda.synchronize()
    for k in range(count):
        got = dst[k * stride:(k + 1) * stride]
        assert torch.equal(got[:size // 2], src[k * (size // 2):(k + 1) * (size // 2)]), (k, size)
        assert bool((got[size // 2:] == 0x4DCD).all()), (k, "wrote past the receive buffer")
    assert stats.rounds == 1 and stats.messages == count and stats.payload_bytes == size * count
    assert stats.write_messages == count and stats.rdma_writes == 4 * count and stats.eager_messages == 0
    del src, dst
    torch.cuda.empty_cache()


def test_receiver_first_sends_everything_as_writes(lib, gpu):
    sizes = [8, 100, 1024, 8184, 8185, 70000, 300000, 1 << 20] * 8
    st = run(lib, sizes, sizes, 64, flags=1, seed=3)
    assert st.eager_messages == 0 and st.write_messages == len(sizes) and st.send_again == 0


def test_mixed_sizes_unaligned_receive_buffers_and_zero_length(lib, gpu):
    rng = np.random.default_rng(11)
    sizes = [int(s) for s in rng.choice([0, 1, 7, 8, 63, 64, 1000, 8184, 8185, 9000, 131072, 131073, 524289], 192)]
    caps = [s if rng.random() < 0.7 else max(s // 3, 1) for s in sizes]
    st = run(lib, sizes, caps, 64, dst_skew=5, seed=12)
    assert st.eager_messages > 0 and st.write_messages > 0 and st.rounds == 3


@pytest.mark.parametrize("group", [2, 3, 8])
def test_grouped_receives_mixed_eager_and_write_subreceives(lib, gpu, group):
    """`group` messages per grouped receive (the phase shape of the reference's
    tests/functional/grouped_recv.cpp): sub-receive k of a request gets the message with tag 1 + k,
    eager where it fits and as striped writes where it does not, sizes 1 KiB * (k + 1) and larger."""
    rng = np.random.default_rng(group)
    n = 64 * 3 + group - 1                                      # the last request is a short one
    sizes = [int(rng.choice([1024 * (1 + i % group), 262144, 8184, 8185, 0, 524288 + 3])) for i in range(n)]
    caps = [s if i % 5 else max(s // 2, 1) for i, s in enumerate(sizes)]
    st = run(lib, sizes, caps, 64, seed=100 + group, group=group, dst_skew=1)
    assert st.eager_messages > 0 and st.write_messages > 0
    # explicit tags, distinct within each request but not in order
    tags = [1000 + (7 * i) % group for i in range(n)]
    if len(set(tags[:group])) == group:
        run(lib, sizes, caps, 64, seed=200 + group, group=group, tags=tags)


def test_rejects_bad_arguments(lib, gpu):
    pool = torch.zeros(64 * RX_STRIDE, dtype=torch.uint8, device="cuda")
    one = np.array([pool.data_ptr()], dtype=np.uint64)
    size = np.array([8], dtype=np.uint64)
    big = np.array([1 << 32], dtype=np.uint64)
    stats = m.SendrecvLoopbackStats()
    call = lib.ofi_amd_sendrecv_loopback_run
    p = lambda a: a.ctypes.data
    assert call(p(one), p(one), p(size), p(size), None, 1, 0, 4, 1, pool.data_ptr(), pool.numel(), 0,
                _gpu.stream(), ctypes.byref(stats)) == -22          # nothing in flight
    assert call(p(one), p(one), p(size), p(size), None, 1, 129, 4, 1, pool.data_ptr(), pool.numel(), 0,
                _gpu.stream(), ctypes.byref(stats)) == -22          # more than the receiver allows
    assert call(p(one), p(one), p(size), p(size), None, 1, 64, 4, 1, pool.data_ptr(), 1000, 0,
                _gpu.stream(), ctypes.byref(stats)) == -22          # rx pool too small
    assert call(p(one), p(one), p(big), p(big), None, 1, 64, 4, 1, pool.data_ptr(), pool.numel(), 0,
                _gpu.stream(), ctypes.byref(stats)) == -90          # -EMSGSIZE: 32-bit control length
    assert call(p(one), p(one), p(size), p(size), None, 1, 64, 4, 9, pool.data_ptr(), pool.numel(), 0,
                _gpu.stream(), ctypes.byref(stats)) == -22          # more sub-receives than a request holds
