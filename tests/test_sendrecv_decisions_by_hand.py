"""The sender's decision stream, call by call, against values worked out on paper from
nccl_net_ofi_rdma_send_comm::send (src/nccl_ofi_rdma.cpp:5646-5877), drain_sender_eager_queue
(:5561-5644), has_ctrl_msg (:2134-2178), update_send_data_from_remote (:574-640) and
alloc_rdma_send_req (:5395-5428): which call is answered "call again", which goes eager and
with which header, which goes as RDMA writes with which immediate data, schedule and size.

Fixed by the harness: remote comm id 77, 4 rails, eager_send_size 8192, min stripe 131,072,
max small message 64; a fresh comm starts at msg_seq_num 1 (include/nccl_ofi_rdma.h:66).
Immediate data = seq | comm << 10 | recv_idx << 25 | nseg << 28 (:68-103), so with comm 77
(77 << 10 = 0x13400) one segment of message 1 is 0x10013401.
"""
import pytest

import _sendrecv
from _sendrecv import AGAIN, EAGER, WRITE


@pytest.fixture(params=["oracle", "product"])
def fl(request, oracle, lib):
    return _sendrecv.flavours(oracle, lib)[request.param]


def last_send(link):
    t = link.trace[-1]
    assert t[0] == "send"
    return dict(kind=t[3], seq=t[4], recv_idx=t[5], imm=t[6], hdr=t[7], size=t[8], offset=t[9], xfers=t[10])


def state(link, *names):
    st = link.send_state()
    return tuple(st[n] for n in names)


def test_single_receives_decision_stream(fl):
    link = _sendrecv.Link(fl)
    S = ("next_msg_seq_num", "eager_queue_count", "eager_offset_next", "prev_eager_batch_count",
         "eager_seq_next", "num_inflight_reqs", "num_inflight_writes", "n_ctrl_received")

    # 1. 100 B, tag 5, nothing posted: no control message, queue empty -> eager.  First of a batch:
    #    eager_seq 0, offset 0, prev 0.  100 >= 64 -> the large counter: rail 0.
    assert link.send(100, 5, "a") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["imm"], d["hdr"], d["size"], d["xfers"]) == \
        (EAGER, 1, 0x10013401, (0, 0, 0, 5), 100, ((0, 0, 100),))
    assert state(link, *S) == (1, 1, 1, 0, 1, 1, 0, 0)

    # 2. 8,184 B, tag 6: 8,184 + 8 = 8,192 still fits; the queue is not empty but a batch is open
    #    (eager_offset_next 1 > 0) -> eager, offset 1 of the same batch, same msg_seq_num 1; rail 1
    assert link.send(8184, 6, "b") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["imm"], d["hdr"], d["xfers"]) == \
        (EAGER, 1, 0x10013401, (1, 0, 0, 6), ((1, 0, 8184),))
    assert state(link, *S) == (1, 2, 2, 0, 1, 2, 0, 0)

    # 3. 8,185 B, tag 7: one byte too many for eager and no control message -> call again, nothing moves
    assert link.send(8185, 7, "c") is None
    assert last_send(link)["kind"] == AGAIN and state(link, *S) == (1, 2, 2, 0, 1, 2, 0, 0)

    # 4. the receiver posts tag 5 (message 1).  5. The retry drains the queue first: the head
    #    (tag 5) takes message 1 -> n_ctrl 1, next 2, the open batch closes (prev 2, offset_next 0);
    #    message 2 has no control message -> stop.  Still too big for eager -> again.
    link.recv([5], [1000])
    assert link.send(8185, 7, "c") is None
    assert state(link, *S) == (2, 1, 0, 2, 1, 2, 0, 1)

    # 6. 50 B, tag 8: would fit, but one eager send is still unmatched and no batch is open
    #    (queue 1, eager_offset_next 0) -> again: a new batch may not start behind an unmatched one
    assert link.send(50, 8, "d") is None
    assert state(link, *S) == (2, 1, 0, 2, 1, 2, 0, 1)

    # 7. the receiver posts tag 6 (message 2).  8. Retry: the head (tag 6) takes message 2 -> n_ctrl 2,
    #    next 3; no batch open, so prev stays 2.  Queue empty, no control message for 3 -> eager, and
    #    a new batch: eager_seq 1, offset 0, prev 2.  50 < 64 -> the small counter: rail 0.
    link.recv([6], [4000])
    assert link.send(50, 8, "d") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["imm"], d["hdr"], d["xfers"]) == \
        (EAGER, 3, 0x10013403, (0, 2, 1, 8), ((0, 0, 50),))
    assert state(link, *S) == (3, 1, 1, 2, 2, 3, 0, 2)

    # 9. the receiver posts tag 8 (message 3) and tag 7 with room for 400,000 B (message 4).
    # 10. 300,000 B, tag 7: the drain matches tag 8 to message 3 (n_ctrl 3, next 4, batch closes:
    #     prev 1); message 4's control message names tag 7 -> rendezvous, n_ctrl 4.  Schedule of
    #     300,000: ceil(300,000 / 131,072) = 3 -> 2 stripes (4 rails), from the large counter (2):
    #     ceil(150,000 / 128) * 128 = 150,016 on rail 2, the rest 149,984 on rail 3.
    #     imm = 4 | 0x13400 | 2 << 28.  The target offset is the receive buffer's address.
    link.recv([8], [50])
    h4 = link.recv([7], [400000])
    assert link.send(300000, 7, "c") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["recv_idx"], d["imm"], d["size"], d["xfers"]) == \
        (WRITE, 4, 0, 0x20013404, 300000, ((2, 0, 150016), (3, 150016, 149984)))
    assert d["offset"] == link.recvs[h4]["dsts"][0]
    assert state(link, *S) == (5, 0, 0, 1, 2, 4, 1, 4)

    # 11. 10 B, tag 9: small enough, queue empty, but a rendezvous write is in flight -> again
    assert link.send(10, 9, "e") is None
    assert state(link, *S) == (5, 0, 0, 1, 2, 4, 1, 4)

    # 12. once everything has completed the same send goes eager: eager_seq 2, prev 1; small counter -> rail 1
    link.run_to_completion()
    assert link.send(10, 9, "e") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["imm"], d["hdr"], d["xfers"]) == \
        (EAGER, 5, 0x10013405, (0, 1, 2, 9), ((1, 0, 10),))
    # what the receiver reports: the eager 8,184 B message into a 4,000 B buffer is truncated
    assert [r["reported"] for r in link.recvs] == [[100], [4000], [50], [300000]]
    link.close()


def test_rendezvous_truncates_to_the_receive_buffer(fl):
    """update_send_data_from_remote :617-625: the schedule is made for min(send, receive) bytes.
    Receive of 20,000 B posted first; send of 300,000 B: one stripe of 20,000 B on rail 0, nseg 1."""
    link = _sendrecv.Link(fl)
    link.recv([3], [20000])
    assert link.send(300000, 3, "x") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["imm"], d["size"], d["xfers"]) == (WRITE, 1, 0x10013401, 20000, ((0, 0, 20000),))
    link.run_to_completion()
    assert link.sends[0]["reported"] == 20000 and link.recvs[0]["reported"] == [20000]
    link.close()


def test_grouped_receive_decision_stream(fl):
    """A grouped receive of three (tags 1, 2, 3; message 1) posted first, sends in the order 3, 1, 2.
    send() :5740-5749 starts the group on the first send (group_num_recvs = remaining = 3) and counts
    the control message once (:5776-5778: only while remaining == num_recvs); each send finds its
    entry by tag, takes that entry's recv_idx into the immediate data (recv_idx << 25), and only
    the third advances msg_seq_num (:5851-5857)."""
    link = _sendrecv.Link(fl)
    S = ("next_msg_seq_num", "group_sends_remaining", "group_num_recvs", "n_ctrl_received", "num_inflight_writes")
    h = link.recv([1, 2, 3], [70000, 70000, 70000])
    dsts = link.recvs[h]["dsts"]
    # tag 3 -> entry 2: imm = 1 | 0x13400 | 2 << 25 | 1 << 28 = 0x14013401; one stripe on rail 0
    assert link.send(65536, 3, "p") is not None
    d = last_send(link)
    assert (d["kind"], d["seq"], d["recv_idx"], d["imm"], d["offset"], d["xfers"]) == \
        (WRITE, 1, 2, 0x14013401, dsts[2], ((0, 0, 65536),))
    assert state(link, *S) == (1, 2, 3, 1, 1)
    # a fourth tag finds no free entry in the group -> again (and nothing is eager inside a group)
    assert link.send(8, 9, "q") is None
    assert state(link, *S) == (1, 2, 3, 1, 1)
    # tag 1 -> entry 0: imm 0x10013401, rail 1
    assert link.send(65536, 1, "r") is not None
    d = last_send(link)
    assert (d["recv_idx"], d["imm"], d["offset"], d["xfers"]) == (0, 0x10013401, dsts[0], ((1, 0, 65536),))
    assert state(link, *S) == (1, 1, 3, 1, 2)
    # tag 3 again: its entry is used up -> again
    assert link.send(65536, 3, "s") is None
    # tag 2 -> entry 1: imm = 0x10013401 | 1 << 25 = 0x12013401, rail 2; the group is complete: next 2
    assert link.send(65536, 2, "t") is not None
    d = last_send(link)
    assert (d["recv_idx"], d["imm"], d["offset"], d["xfers"]) == (1, 0x12013401, dsts[1], ((2, 0, 65536),))
    assert state(link, *S) == (2, 0, 0, 1, 3)
    link.run_to_completion()
    assert link.recvs[h]["reported"] == [65536, 65536, 65536]
    link.close()
