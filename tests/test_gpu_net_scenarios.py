"""The scenarios of the reference's tests/functional/eager_multirecv.cpp (T5 .. T25) through the net
entry points (include/ofi_amd_net_abi.h) on the GPU, both ranks in this process.  The reference runs
them between two ranks over a fabric; their assertion is always the same: the k-th send of a tag
lands, whole, in the k-th posted (sub-)receive of that tag, and test() reports its size on both sides.

The sender posts with the reference's post_sends_interleaved (eager_multirecv.cpp:74-103: a rotating
queue, a send told to call again goes to the back and blocks later sends of its tag for the round);
"late" scenarios post the receives after the sender's first round, so that whatever can go eager has
gone eager (the reference sleeps 10 ms on the receiving rank), "early" ones post them first.  Every
message has its own byte pattern, every (sub-)receive its own buffer, checked byte for byte together
with the bytes around it."""
import ctypes

import numpy as np
import pytest
import torch

import aws_ofi_nccl_amd as m
from _netlink import Link

pytestmark = pytest.mark.gpu

E, L = 1024, 16384          # EAGER_SIZE, LARGE_SIZE: eager_multirecv.cpp:16-18
INTERLEAVED = [0, 1, 2, 3, 4, 5, 6, 1, 7, 0, 2, 3, 4, 5, 6, 7]   # T17 / T18


def scenarios():
    """name -> (messages as (size, tag), receives as (tags, sizes), receiver late?, (eager, write) or None
    [, sender sizes checked?])"""
    s = {}
    s["t5_single_eager_late"] = ([(E, 1)], [([1], [E])], True, (1, 0))
    s["t6_single_early"] = ([(E, 1)], [([1], [E])], False, (0, 1))
    s["t7_four_sequential_eager"] = ([(E, 1)] * 4, [([1], [E])] * 4, True, (4, 0))
    s["t8_grouped_all_eager"] = ([(E, 10), (E, 11), (E, 12)], [([10, 11, 12], [E, E, E])], True, (3, 0))
    s["t9_grouped_mixed"] = ([(E, 20), (L, 21)], [([20, 21], [E, L])], True, (1, 1))
    s["t10_grouped_no_eager"] = ([(L, 30), (L, 31), (L, 32)], [([30, 31, 32], [L, L, L])], True, (0, 3))
    s["t11_eager_across_single_and_grouped"] = ([(E, 1), (E, 40), (E, 41)], [([1], [E]), ([40, 41], [E, E])], True,
                                                (3, 0))
    s["t12_tag_pushback"] = ([(E, 51), (E, 53), (E, 50), (E, 52)], [([51, 53], [E, E]), ([50, 52], [E, E])], True, None)
    s["t13_thirty_two_eager"] = ([(E, 1)] * 32, [([1], [E])] * 32, True, (32, 0))
    s["t14_boundary_8184"] = ([(8184, 1)], [([1], [8184])], True, (1, 0))
    s["t14_boundary_8185"] = ([(8185, 1)], [([1], [8185])], True, (0, 1))
    is_eager = [[True, True, False, False], [True, False, True, False]]
    s["t15_eager_write_permutations"] = (
        [(E if is_eager[g][i] else L, 60 + i) for g in range(2) for i in range(4)],
        [([60, 61, 62, 63], [E if is_eager[g][i] else L for i in range(4)]) for g in range(2)], True, None)
    s["t16_ordering_per_tag"] = ([(E, 70 + (i & 1)) for i in range(8)], [([70, 71], [E, E])] * 4, True, None)
    s["t17_interleaved_all_write"] = ([(L, t) for t in INTERLEAVED], [(list(range(8)), [L] * 8)] * 2, False, (0, 16))
    s["t18_interleaved_all_eager"] = ([(E, t) for t in INTERLEAVED], [(list(range(8)), [E] * 8)] * 2, True, None)
    order = [(0, E), (1, E), (2, L), (1, E), (3, L), (0, E), (2, L), (3, L)]
    s["t19_interleaved_mixed"] = ([(sz, t) for t, sz in order], [([0, 1, 2, 3], [E, E, L, L])] * 2, True, None)
    gsz = [E, L, E]
    s["t21_three_groups"] = ([(gsz[g], t) for g, t in [(0, 0), (0, 1), (1, 0), (2, 0), (1, 1), (2, 1)]],
                             [([0, 1], [gsz[g]] * 2) for g in range(3)], True, None)
    s["t22_max_interleave_write"] = ([(L, t) for t in range(8) for _ in range(2)], [(list(range(8)), [L] * 8)] * 2,
                                     False, (0, 16))
    stags = [1, 2, 3, 4, 10, 11, 12, 13, 20, 21, 22, 23]
    s["t23_eager_spanning_three_groups"] = ([(E, t) for t in stags], [(stags[4 * g:4 * g + 4], [E] * 4) for g in range(3)],
                                            True, (12, 0))
    s["t24_eager_alternating_single_grouped"] = ([(E, t) for t in [1, 50, 51, 1, 60, 61]],
                                                 [([1], [E]), ([50, 51], [E, E]), ([1], [E]), ([60, 61], [E, E])], True, None)
    s["t25_rotated_queue"] = ([(E, 30), (E, 40), (L, 31), (L, 20)], [([30, 31], [E, L]), ([20], [L]), ([40], [E])], True,
                              (2, 2))
    # tests/functional/grouped_recv.cpp:158-240: n sends of 1024 * (i + 1) bytes, one tag, one grouped receive.
    # An eager send looks its receive-buffer length up by tag (get_ctrl_msg_buff_len,
    # src/nccl_ofi_rdma.cpp:2183-2196), which finds the group's first entry of that tag: with one tag for all
    # sub-receives the sender reports min(size, first buffer); the data and the receiver's sizes are right
    # and the reference's test does not read the sender's size ("sender sizes unchecked" below).
    for n in (1, 2, 4, 8):
        for late in (True, False):
            s["grouped_one_tag_growing_sizes_n%d_%s" % (n, "late" if late else "early")] = (
                [(1024 * (i + 1), 1) for i in range(n)], [([1] * n, [1024 * (i + 1) for i in range(n)])], late, None,
                not late)
    # grouped_recv.cpp:666-671: receive [tag 8] then receive [tags 0..7]; sends 0, 8, 1, 2, .. 7
    s["grouped_multi_tag_send_before_its_group"] = ([(L, t) for t in (0, 8, 1, 2, 3, 4, 5, 6, 7)],
                                                    [([8], [L]), (list(range(8)), [L] * 8)], False, (0, 9))
    s["zero_length_messages"] = ([(0, 5), (E, 5), (0, 6)], [([5], [E]), ([5, 6], [E, E])], True, (3, 0))
    s["receive_buffer_smaller_than_the_message"] = ([(E, 1), (L, 2)], [([1], [100]), ([2], [5000])], True, (1, 1))
    return s


SCENARIOS = scenarios()


@pytest.mark.parametrize("name", sorted(SCENARIOS))
def test_kth_send_of_a_tag_lands_in_the_kth_receive_of_that_tag(lib, gpu, name):
    msgs, recvs, late, split = SCENARIOS[name][:4]
    sender_sizes_checked = SCENARIOS[name][4] if len(SCENARIOS[name]) > 4 else True
    link = Link(lib)
    rng = np.random.default_rng(len(name) * 131 + len(msgs))
    srcs = [torch.from_numpy(rng.integers(0, 256, max(size, 1), dtype=np.uint8)).cuda() for size, _ in msgs]
    dsts = [[torch.full((cap + 64,), 0xCD, dtype=torch.uint8, device="cuda") for cap in sizes] for _, sizes in recvs]
    torch.cuda.synchronize()
    recv_reqs = []

    def post_receives():
        for (tags, sizes), bufs in zip(recvs, dsts):
            recv_reqs.append(link.irecv(bufs, sizes, tags))

    if not late:
        post_receives()
    # post_sends_interleaved, eager_multirecv.cpp:74-103
    send_reqs = [None] * len(msgs)
    queue = list(range(len(msgs)))
    for rnd in range(10_000):
        if not queue:
            break
        blocked, again = set(), []
        for idx in queue:
            size, tag = msgs[idx]
            if tag in blocked:
                again.append(idx)
                continue
            req = link.isend(srcs[idx], size, tag)
            if req is None:
                blocked.add(tag)
                again.append(idx)
            else:
                send_reqs[idx] = req
        queue = again
        if late and rnd == 0:
            post_receives()
    assert not queue, "sends never accepted: %r" % queue

    # both ranks poll to completion (poll_sends / poll_recv), keeping what test() reports
    send_sizes, recv_sizes = [None] * len(msgs), [None] * len(recvs)
    for _ in range(2_000_000):
        for i, q in enumerate(send_reqs):
            if send_sizes[i] is None:
                done, sz = link.test(q)
                if done:
                    send_sizes[i] = sz[0]
        for i, q in enumerate(recv_reqs):
            if recv_sizes[i] is None:
                done, sz = link.test(q, len(recvs[i][0]))
                if done:
                    recv_sizes[i] = sz
                    link.flush(dsts[i], recvs[i][1])
        if None not in send_sizes and None not in recv_sizes:
            break
    assert None not in send_sizes and None not in recv_sizes

    # the k-th send of a tag -> the k-th posted (sub-)receive of that tag
    slots = {}
    for r, (tags, sizes) in enumerate(recvs):
        for sub, (tag, cap) in enumerate(zip(tags, sizes)):
            slots.setdefault(tag, []).append((r, sub, cap))
    seen = {}
    torch.cuda.synchronize()
    used = set()
    for idx, (size, tag) in enumerate(msgs):
        k = seen.get(tag, 0)
        seen[tag] = k + 1
        r, sub, cap = slots[tag][k]
        used.add((r, sub))
        moved = min(size, cap)
        got = dsts[r][sub].cpu().numpy()
        assert np.array_equal(got[:moved], srcs[idx].cpu().numpy()[:moved]), (name, idx, tag, r, sub)
        assert np.all(got[moved:] == 0xCD), (name, idx, "wrote beyond the message")
        assert recv_sizes[r][sub] == moved, (name, idx, recv_sizes[r])
        if sender_sizes_checked:
            assert send_sizes[idx] == moved, (name, idx, send_sizes[idx])
    assert used == {(r, sub) for r, (tags, _) in enumerate(recvs) for sub in range(len(tags))}

    st = link.stats()
    assert st.eager_sends + st.write_sends == len(msgs)
    if split is not None:
        assert (st.eager_sends, st.write_sends) == split, (name, st.eager_sends, st.write_sends)
    ss, rs = m.SendState(), m.RecvState()
    assert lib.ofi_amd_net_link_state(link.h, ctypes.byref(ss), ctypes.byref(rs)) == 0
    assert ss.num_inflight_reqs == 0 and ss.num_inflight_writes == 0 and ss.eager_queue_count == 0
    assert rs.num_inflight_reqs == 0 and rs.eager_pending == 0
    assert ss.next_msg_seq_num == rs.next_msg_seq_num
    assert ss.n_ctrl_received == rs.n_ctrl_sent == len(recvs)
    link.close()


GROUPED_PATTERN = [(8, 20), (3, 1), (8, 10), (4, 1), (1, 1), (8, 10), (7, 1), (5, 1), (8, 4), (2, 1),
                   (1, 1), (8, 4), (7, 1)]          # (sends per receive, receives), grouped_recv.cpp:255-258


def test_grouped_receives_in_the_alltoall_pattern(lib, gpu):
    """tests/functional/grouped_recv.cpp:242-420, the production alltoall trace shape: phases of grouped
    receives of 1..8 sub-receives, 256 KiB sends into 512 KiB buffers, the receiver keeping a window of 16
    receives posted ahead, the sender going round its queue; 414 messages, every one checked."""
    link = Link(lib)
    msgs, recvs = [], []
    for per, count in GROUPED_PATTERN:
        for _ in range(count):
            recvs.append((list(range(per)), [524288] * per))
            msgs += [(262144, t) for t in range(per)]
    rng = np.random.default_rng(3)
    pool = torch.from_numpy(rng.integers(0, 256, 262144 + len(msgs), dtype=np.uint8)).cuda()
    dsts = [[torch.full((524288 + 64,), 0xCD, dtype=torch.uint8, device="cuda") for _ in tags] for tags, _ in recvs]
    torch.cuda.synchronize()
    # message i is the 256 KiB of `pool` that start at byte i: all different, one allocation
    recv_reqs, recv_sizes, posted = {}, {}, 0
    send_reqs, send_sizes = {}, {}
    queue = list(range(len(msgs)))
    for _ in range(200_000):
        while posted < len(recvs) and len(recv_reqs) < 16:
            tags, sizes = recvs[posted]
            recv_reqs[posted] = link.irecv(dsts[posted], sizes, tags)
            posted += 1
        blocked, again = set(), []
        for idx in queue:
            size, tag = msgs[idx]
            if tag in blocked:
                again.append(idx)
                continue
            req = link.isend(pool, size, tag, offset=idx)
            if req is None:
                blocked.add(tag)
                again.append(idx)
            else:
                send_reqs[idx] = req
        queue = again
        for idx in list(send_reqs):
            done, sz = link.test(send_reqs[idx])
            if done:
                send_sizes[idx] = sz[0]
                del send_reqs[idx]
        for r in list(recv_reqs):
            done, sz = link.test(recv_reqs[r], len(recvs[r][0]))
            if done:
                recv_sizes[r] = sz
                link.flush(dsts[r], recvs[r][1])
                del recv_reqs[r]
        if not queue and not send_reqs and not recv_reqs and posted == len(recvs):
            break
    assert len(send_sizes) == len(msgs) and len(recv_sizes) == len(recvs)
    assert all(v == 262144 for v in send_sizes.values())
    torch.cuda.synchronize()
    host = pool.cpu().numpy()
    idx = 0
    for r, (tags, _) in enumerate(recvs):          # messages were generated receive by receive, tag by tag
        assert recv_sizes[r] == [262144] * len(tags)
        for sub in range(len(tags)):
            got = dsts[r][sub].cpu().numpy()
            assert np.array_equal(got[:262144], host[idx:idx + 262144]), (r, sub)
            assert np.all(got[262144:] == 0xCD)
            idx += 1
    st = link.stats()
    assert st.write_sends == len(msgs) and st.eager_sends == 0 and st.rdma_writes == 2 * len(msgs)
    link.close()


def test_ring_of_four_ranks(lib, gpu):
    """tests/functional/ring.cpp:205-318 with four ranks in this process: every rank posts NUM_REQUESTS
    (NCCL_NET_MAX_REQUESTS = 32) receives of RECV_SIZE 5200 from its predecessor, then as many sends of
    SEND_SIZE 5000 to its successor, retrying an isend that says "call again"; then polls both lists until
    all are done.  Both sides report min(SEND_SIZE, RECV_SIZE); each completed receive is flushed and
    compared with what was sent."""
    ranks, nreq, send_size, recv_size = 4, 32, 5000, 5200
    links = [Link(lib) for _ in range(ranks)]          # links[k]: rank k -> rank k + 1
    rng = np.random.default_rng(11)
    src = [torch.from_numpy(rng.integers(0, 256, (nreq, send_size), dtype=np.uint8)).cuda() for _ in range(ranks)]
    dst = [[torch.full((recv_size + 64,), 0xCD, dtype=torch.uint8, device="cuda") for _ in range(nreq)]
           for _ in range(ranks)]
    torch.cuda.synchronize()
    recv_reqs = {(k, i): links[(k - 1) % ranks].irecv([dst[k][i]], [recv_size]) for k in range(ranks) for i in range(nreq)}
    send_reqs = {}
    for k in range(ranks):
        for i in range(nreq):
            for _ in range(100_000):
                req = links[k].isend(src[k][i], send_size)
                if req is not None:
                    break
            assert req is not None
            send_reqs[(k, i)] = req
    for _ in range(200_000):
        for key in list(send_reqs):
            done, sz = links[key[0]].test(send_reqs[key])
            if done:
                assert sz == [send_size]
                del send_reqs[key]
        for key in list(recv_reqs):
            k, i = key
            link = links[(k - 1) % ranks]
            done, sz = link.test(recv_reqs[key])
            if done:
                assert sz == [send_size]
                link.flush([dst[k][i]], [recv_size])
                got = dst[k][i].cpu().numpy()
                assert np.array_equal(got[:send_size], src[(k - 1) % ranks][i].cpu().numpy()), key
                assert np.all(got[send_size:] == 0xCD)
                del recv_reqs[key]
        if not send_reqs and not recv_reqs:
            break
    assert not send_reqs and not recv_reqs
    for link in links:
        st = link.stats()
        assert st.eager_sends + st.write_sends == nreq and st.payload_bytes == nreq * send_size
        link.close()
