"""The data-path members of ncclNet_vN_t (net_v12.h:110-119: isend, irecv, iflush, test) as this
library exports them (include/ofi_amd_net_abi.h), driven the way the reference's two-rank
functional test drives the plugin (tests/functional/functional_test.cpp:242-294, 592-731:
post_send / post_recv retry while the request is NULL, every request is polled with test() until
done, the receiving rank flushes after each completed receive and polls the flush), with both
ranks in this process: the two ends of ofi_amd_net_link_create on one GPU.

What is checked: every received buffer byte for byte against its source (up to min(send, receive)
bytes, nothing beyond), the sizes test() reports on both ends, which protocol each message took
(eager below the threshold when the sender is ahead, rendezvous writes on 1, 2 or 4 rails
otherwise), the argument checks and result codes of src/nccl_ofi_api.cpp:440-567, and that the
in-flight limits of the reference hold (128 receives, "call again" without a control message)."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import aws_ofi_nccl_amd as m
from _netlink import TAG, Link, ncclSuccess, vp

pytestmark = pytest.mark.gpu

ncclSystemError, ncclInternalError, ncclInvalidArgument = 2, 3, 4
NUM_REQUESTS = 32        # NCCL_NET_MAX_REQUESTS, tests/functional/functional_test.h:28
PAIRS = [(512, 512), (4096, 4096), (16384, 16384), (1 << 20, 1 << 20), (5120, 4096), (17408, 16384),
         (2 << 20, 1 << 20), (4096, 5120), (16384, 17408), (1 << 20, 2 << 20)]

def buffers(send_sizes, recv_sizes, seed):
    rng = np.random.default_rng(seed)
    srcs = [torch.from_numpy(rng.integers(0, 256, max(s, 1), dtype=np.uint8)).cuda() for s in send_sizes]
    dsts = [torch.full((max(r, 1) + 64,), 0xCD, dtype=torch.uint8, device="cuda") for r in recv_sizes]
    torch.cuda.synchronize()
    return srcs, dsts


def check_bytes(srcs, dsts, send_sizes, recv_sizes, skew=0):
    torch.cuda.synchronize()
    for i, (s, r) in enumerate(zip(send_sizes, recv_sizes)):
        k = min(s, r)
        got, want = dsts[i].cpu().numpy(), srcs[i].cpu().numpy()
        assert np.array_equal(got[skew:skew + k], want[:k]), (i, s, r)
        assert np.all(got[:skew] == 0xCD) and np.all(got[skew + k:] == 0xCD), (i, "wrote outside")


def poll_all(link, send_reqs, recv_reqs, dsts, recv_sizes, expect_send, expect_recv):
    """poll_and_validate, both ranks in turn: test every open request; flush behind each receive."""
    open_s, open_r = dict(enumerate(send_reqs)), dict(enumerate(recv_reqs))
    for _ in range(2_000_000):
        if not open_s and not open_r:
            return
        for i in list(open_s):
            done, sizes = link.test(open_s[i])
            if done:
                assert sizes[0] == expect_send[i], (i, sizes)
                del open_s[i]
        for i in list(open_r):
            done, sizes = link.test(open_r[i])
            if done:
                assert sizes[0] == expect_recv[i], (i, sizes)
                flushed = link.flush([dsts[i]], [recv_sizes[i]])
                assert flushed == (recv_sizes[i] != 0)
                del open_r[i]
    raise AssertionError("requests never completed: %d sends, %d receives open" % (len(open_s), len(open_r)))


@pytest.mark.parametrize("pair", PAIRS)
@pytest.mark.parametrize("sender_first", [False, True])
def test_reference_size_pairs_thirty_two_requests_each(lib, gpu, pair, sender_first):
    """The ten (send, receive) size pairs of tests/functional/nccl_message_transfer.cpp:44-56, 32 requests
    each.  Receiver first: every message finds its control message and goes as writes.  Sender first:
    what fits an rx buffer goes eager ahead of its receive, the rest is answered "call again" until the
    receive is posted."""
    send, recv = pair
    link = Link(lib)
    srcs, dsts = buffers([send] * NUM_REQUESTS, [recv] * NUM_REQUESTS, seed=send * 3 + recv)
    send_reqs, recv_reqs = [None] * NUM_REQUESTS, [None] * NUM_REQUESTS
    again = 0
    if sender_first:
        for i in range(NUM_REQUESTS):
            send_reqs[i] = link.isend(srcs[i], send)
            again += send_reqs[i] is None
    for i in range(NUM_REQUESTS):
        recv_reqs[i] = link.irecv([dsts[i]], [recv])
    for i in range(NUM_REQUESTS):
        for _ in range(1000):
            if send_reqs[i] is not None:
                break
            send_reqs[i] = link.isend(srcs[i], send)       # post_send: retry until there is a request
        assert send_reqs[i] is not None
    moved = min(send, recv)
    poll_all(link, send_reqs, recv_reqs, dsts, [recv] * NUM_REQUESTS, [moved] * NUM_REQUESTS, [moved] * NUM_REQUESTS)
    check_bytes(srcs, dsts, [send] * NUM_REQUESTS, [recv] * NUM_REQUESTS)
    st = link.stats()
    eager_possible = send + 8 <= 8192          # payload and the 8-byte header fit an rx buffer
    if sender_first and eager_possible:
        assert st.eager_sends == NUM_REQUESTS and again == 0 and st.eager_copies == NUM_REQUESTS
    elif sender_first:
        assert st.eager_sends == 0 and again == NUM_REQUESTS          # no control message yet: call again
    else:
        stripes = 1 if moved <= 131072 else (2 if moved <= 262144 else 4)
        assert st.eager_sends == 0 and st.write_sends == NUM_REQUESTS and st.rdma_writes == NUM_REQUESTS * stripes
    # an eager message crosses the wire in full and is cut to the receive buffer on the way out of the rx buffer
    on_wire = send if (sender_first and eager_possible) else moved
    assert st.payload_bytes == NUM_REQUESTS * on_wire and st.flushes == NUM_REQUESTS
    ss, rs = m.SendState(), m.RecvState()
    assert lib.ofi_amd_net_link_state(link.h, ctypes.byref(ss), ctypes.byref(rs)) == 0
    assert ss.num_inflight_reqs == 0 and rs.num_inflight_reqs == 0 and ss.next_msg_seq_num == rs.next_msg_seq_num
    link.close()


def test_grouped_receives_matched_by_tag_with_ragged_sizes_and_odd_addresses(lib, gpu):
    """Eight receives per request (NCCL_OFI_MAX_RECVS), sends in a shuffled tag order, sizes from 0 to
    3 MiB around the eager and striping thresholds, destinations at odd addresses, several rounds so
    that rx buffers, launch groups and request entries are reused."""
    rng = np.random.default_rng(77)
    link = Link(lib, rx_buffers=16)
    choices = [0, 1, 7, 8, 63, 4096, 8191, 8192, 8193, 65536, 131072, 131073, 262144, 262145, 1 << 20, 3 << 20]
    for rnd in range(6):
        n = 8
        send_sizes = [int(rng.choice(choices)) for _ in range(n)]
        recv_sizes = [s if rng.random() < 0.6 else int(rng.choice(choices)) for s in send_sizes]
        srcs, dsts = buffers(send_sizes, recv_sizes, seed=1000 + rnd)
        tags = [int(t) for t in rng.permutation(n) + 10]
        skew = 3
        sender_first = rnd % 2 == 0
        order = [int(k) for k in rng.permutation(n)]
        send_reqs = {}
        if sender_first:
            for k in order:
                q = link.isend(srcs[k], send_sizes[k], tags[k])
                if q is not None:
                    send_reqs[k] = q
        recv_req = link.irecv(dsts, recv_sizes, tags, offset=skew)
        for k in order:
            for _ in range(1000):
                if k in send_reqs:
                    break
                q = link.isend(srcs[k], send_sizes[k], tags[k])
                if q is not None:
                    send_reqs[k] = q
            assert k in send_reqs, (rnd, k)
        moved = [min(s, r) for s, r in zip(send_sizes, recv_sizes)]
        recv_done = False
        for _ in range(2_000_000):
            for k in list(send_reqs):
                done, sizes = link.test(send_reqs[k])
                if done:
                    assert sizes[0] == moved[k], (rnd, k, sizes)
                    del send_reqs[k]
            if not recv_done:
                recv_done, sizes = link.test(recv_req, n)
                if recv_done:
                    assert sizes == moved, (rnd, sizes, moved)
                    assert link.flush(dsts, recv_sizes) == any(recv_sizes)
            if recv_done and not send_reqs:
                break
        assert recv_done and not send_reqs
        check_bytes(srcs, dsts, send_sizes, recv_sizes, skew=skew)
    st = link.stats()
    assert st.eager_sends > 0 and st.write_sends > 0 and st.eager_sends + st.write_sends == 48
    link.close()


def test_more_eager_sends_than_rx_buffers_and_more_receives_than_requests(lib, gpu):
    """With 4 rx buffers posted at the receiving end the fifth eager send ahead of any receive is refused by
    the fabric (-FI_EAGAIN in the reference): its request is returned and its post waits in the sending end's
    queue (post_with_pending_retry, src/nccl_ofi_rdma.cpp:1375-1387), and while it waits further isend calls
    answer "call again" (process_cq_if_pending, :3523-3545).  The 129th receive in flight is refused with
    -ENOSPC -> ncclSystemError (NCCL_OFI_MAX_REQUESTS, :3571-3577).  Everything drains afterwards."""
    link = Link(lib, rx_buffers=4)
    n = 128
    srcs, dsts = buffers([256] * n, [256] * n, seed=5)
    send_reqs = []
    for i in range(8):
        q = link.isend(srcs[i], 256)
        if q is None:
            break
        send_reqs.append(q)
    assert len(send_reqs) == 5 and link.stats().posts_refused == 1
    for _ in range(100):
        assert link.isend(srcs[5], 256) is None
    recv_reqs = [link.irecv([dsts[i]], [256]) for i in range(n)]
    data, sizes, tags, mhs = (vp * 1)(dsts[0].data_ptr()), (ctypes.c_size_t * 1)(256), (ctypes.c_int * 1)(TAG), (vp * 1)(0)
    req = vp()
    assert lib.ofi_amd_net_irecv(link.r, 1, data, sizes, tags, mhs, None, ctypes.byref(req)) == ncclSystemError
    assert not req.value

    def poll_receives():
        """The receiving rank polls: arrivals are matched, copied out, and their rx buffers posted again."""
        for k, r in enumerate(recv_reqs):
            if r is not None and link.test(r)[0]:
                recv_reqs[k] = None

    for i in range(5, n):
        q = None
        for _ in range(100_000):
            q = link.isend(srcs[i], 256)
            if q is not None:
                break
            poll_receives()
        assert q is not None, i
        send_reqs.append(q)
    poll_all(link, send_reqs, [r for r in recv_reqs if r is not None],
             [dsts[i] for i in range(n) if recv_reqs[i] is not None],
             [256] * n, [256] * n, [256] * n)
    check_bytes(srcs, dsts, [256] * n, [256] * n)
    link.close()


def test_argument_checks_and_result_codes(lib, gpu):
    """nccl_net_ofi_isend / _irecv / _iflush / _test, src/nccl_ofi_api.cpp:440-567."""
    link = Link(lib)
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    req = vp(1)
    data, sizes, tags, mhs = (vp * 9)(*[buf.data_ptr()] * 9), (ctypes.c_size_t * 9)(*[64] * 9), \
        (ctypes.c_int * 9)(*range(9)), (vp * 9)()
    isizes = (ctypes.c_int * 9)(*[64] * 9)
    # isend: NULL comm or request -> ncclInternalError
    assert lib.ofi_amd_net_isend(None, vp(buf.data_ptr()), 8, TAG, None, None, ctypes.byref(req)) == ncclInternalError
    assert req.value is None
    assert lib.ofi_amd_net_isend(link.s, vp(buf.data_ptr()), 8, TAG, None, None, None) == ncclInternalError
    # the receiving end is no send comm, and the other way round
    assert lib.ofi_amd_net_isend(link.r, vp(buf.data_ptr()), 8, TAG, None, None, ctypes.byref(req)) == ncclInternalError
    assert lib.ofi_amd_net_irecv(link.s, 1, data, sizes, tags, mhs, None, ctypes.byref(req)) == ncclInternalError
    # irecv: NULL pointers and n outside 1..8 -> ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(None, 1, data, sizes, tags, mhs, None, ctypes.byref(req)) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 1, None, sizes, tags, mhs, None, ctypes.byref(req)) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 1, data, None, tags, mhs, None, ctypes.byref(req)) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 1, data, sizes, None, mhs, None, ctypes.byref(req)) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 1, data, sizes, tags, None, None, ctypes.byref(req)) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 1, data, sizes, tags, mhs, None, None) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 0, data, sizes, tags, mhs, None, ctypes.byref(req)) == ncclInvalidArgument
    assert lib.ofi_amd_net_irecv(link.r, 9, data, sizes, tags, mhs, None, ctypes.byref(req)) == ncclInvalidArgument
    big = (ctypes.c_size_t * 1)(1 << 32)
    assert lib.ofi_amd_net_irecv(link.r, 1, data, big, tags, mhs, None, ctypes.byref(req)) == ncclInternalError
    # bytes from or into address 0 would be a fault on the device: an error code, and no sequence number is used up
    nulls = (vp * 1)(None)
    assert lib.ofi_amd_net_isend(link.s, None, 8, TAG, None, None, ctypes.byref(req)) == ncclInternalError
    assert lib.ofi_amd_net_irecv(link.r, 1, nulls, sizes, tags, mhs, None, ctypes.byref(req)) == ncclInternalError
    assert req.value is None
    # iflush: n above 8, NULL comm / mhandles / request -> ncclInternalError; all sizes 0 -> no request
    assert lib.ofi_amd_net_iflush(link.r, 9, data, isizes, mhs, ctypes.byref(req)) == ncclInternalError
    assert lib.ofi_amd_net_iflush(None, 1, data, isizes, mhs, ctypes.byref(req)) == ncclInternalError
    assert lib.ofi_amd_net_iflush(link.r, 1, data, isizes, None, ctypes.byref(req)) == ncclInternalError
    assert lib.ofi_amd_net_iflush(link.r, 1, data, isizes, mhs, None) == ncclInternalError
    zeros = (ctypes.c_int * 2)(0, 0)
    req = vp(1)
    assert lib.ofi_amd_net_iflush(link.r, 2, data, zeros, mhs, ctypes.byref(req)) == ncclSuccess and req.value is None
    # test: NULL request, a request that has already reported done
    done = ctypes.c_int()
    assert lib.ofi_amd_net_test(None, ctypes.byref(done), None) == ncclInternalError
    r = link.irecv([buf], [64])
    s = link.isend(buf, 64, offset=2048)
    assert s is not None
    for q in (s, r):
        for _ in range(1_000_000):
            if link.test(q)[0]:
                break
        assert lib.ofi_amd_net_test(q, ctypes.byref(done), None) == ncclInternalError
    # the older spellings reach the same path: int sizes (v6-v8), no profiler handles (v9)
    for isend, irecv, size_t in ((lib.ofi_amd_net_isend_v5, lib.ofi_amd_net_irecv_v5, ctypes.c_int),
                                 (lib.ofi_amd_net_isend_v9, lib.ofi_amd_net_irecv_v9, ctypes.c_size_t)):
        src = torch.arange(200, dtype=torch.uint8, device="cuda")
        dst = torch.zeros(256, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        rq, sq = vp(), vp()
        assert irecv(link.r, 1, (vp * 1)(dst.data_ptr()), (size_t * 1)(256), (ctypes.c_int * 1)(TAG), (vp * 1)(0),
                     ctypes.byref(rq)) == ncclSuccess and rq.value
        assert isend(link.s, vp(src.data_ptr()), 200, TAG, None, ctypes.byref(sq)) == ncclSuccess and sq.value
        got = {}
        for name, q in (("send", sq), ("recv", rq)):
            for _ in range(1_000_000):
                d, sz = link.test(q)
                if d:
                    got[name] = sz[0]
                    break
        assert got == {"send": 200, "recv": 200}
        torch.cuda.synchronize()
        assert torch.equal(dst[:200], src) and int(dst[200:].sum()) == 0
    link.close()


def test_same_bytes_and_protocol_split_as_the_one_call_loop_back(lib, gpu):
    """The power-of-two sweep of the configured workload, 8 B to 64 MiB, up to 64 messages in flight,
    through isend / irecv / test, against ofi_amd_sendrecv_loopback_run on the same sizes: the same
    bytes arrive and the same number of messages go eager, as writes, and on how many stripes."""
    link = Link(lib, rx_buffers=64)
    for k in range(0, 24, 3):
        size = 8 << k
        count = 64 if size <= (1 << 20) else max(2, (128 << 20) // size)
        srcs, dsts = buffers([size] * count, [size] * count, seed=size)
        before = link.stats()
        # the loop-back's order: the sender is ahead, one receive after each send that did not go
        send_reqs, recv_reqs = [], []
        for i in range(count):
            q = link.isend(srcs[i], size)
            recv_reqs.append(link.irecv([dsts[i]], [size]))
            for _ in range(100_000):
                if q is not None:
                    break
                q = link.isend(srcs[i], size)
            assert q is not None
            send_reqs.append(q)
        poll_all(link, send_reqs, recv_reqs, dsts, [size] * count, [size] * count, [size] * count)
        check_bytes(srcs, dsts, [size] * count, [size] * count)
        st = link.stats()
        ref = m.SendrecvLoopbackStats()
        pool = torch.zeros(count * 8320, dtype=torch.uint8, device="cuda")
        dsts2 = [torch.zeros_like(d) for d in dsts]
        a_src = np.array([t.data_ptr() for t in srcs], dtype=np.uint64)
        a_dst = np.array([t.data_ptr() for t in dsts2], dtype=np.uint64)
        a_size = np.array([size] * count, dtype=np.uint64)
        torch.cuda.synchronize()
        assert lib.ofi_amd_sendrecv_loopback_run(a_src.ctypes.data, a_dst.ctypes.data, a_size.ctypes.data,
                                                 a_size.ctypes.data, None, count, count, 4, 1, pool.data_ptr(),
                                                 pool.numel(), 0, _gpu.stream(), ctypes.byref(ref)) == 0
        torch.cuda.synchronize()
        assert st.eager_sends - before.eager_sends == ref.eager_messages
        assert st.write_sends - before.write_sends == ref.write_messages
        assert st.rdma_writes - before.rdma_writes == ref.rdma_writes
        assert st.payload_bytes - before.payload_bytes == ref.payload_bytes
        for a, b in zip(dsts, dsts2):
            assert torch.equal(a[:size], b[:size])
    assert _gpu.fetch_async_errors(lib) == 0
    link.close()


def test_link_closed_with_requests_in_flight(lib, gpu):
    """tests/functional/inflight_close.cpp: NUM_REQUESTS sends and receives of 1 MiB are posted and the comms
    are closed without waiting for them.  Here: the link is destroyed with requests open, some launched and
    some not, three times over; destruction waits for what was launched and a new link works afterwards."""
    for it in range(3):
        link = Link(lib)
        srcs, dsts = buffers([1 << 20] * NUM_REQUESTS, [1 << 20] * NUM_REQUESTS, seed=it)
        reqs = [link.irecv([dsts[i]], [1 << 20]) for i in range(NUM_REQUESTS)]
        reqs += [link.isend(srcs[i], 1 << 20) for i in range(NUM_REQUESTS)]
        assert all(q is not None for q in reqs)
        if it:
            link.test(reqs[0])                      # launches the first group; the rest may still be gathering
            for i in range(4):                      # a few more posts behind the launched group
                link.irecv([dsts[i]], [1 << 20])
                assert link.isend(srcs[i], 1 << 20) is not None
        link.close()
        torch.cuda.synchronize()
    link = Link(lib)
    srcs, dsts = buffers([4096, 1 << 20], [4096, 1 << 20], seed=9)
    s0 = link.isend(srcs[0], 4096)
    r = [link.irecv([dsts[i]], [srcs[i].numel()]) for i in range(2)]
    s1 = link.isend(srcs[1], 1 << 20)
    poll_all(link, [s0, s1], r, dsts, [4096, 1 << 20], [4096, 1 << 20], [4096, 1 << 20])
    check_bytes(srcs, dsts, [4096, 1 << 20], [4096, 1 << 20])
    link.close()
    assert _gpu.fetch_async_errors(lib) == 0
