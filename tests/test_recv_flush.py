"""The receive comm's flush decision (nccl_net_ofi_rdma_recv_comm::flush,
src/nccl_ofi_rdma.cpp:4405-4510) and its completion test (has_flush_completed, :2110-2126),
oracle and product side by side: no flush for all-empty receives, one flush for any number of
buffers, the shared in-flight limit, done when every rail's slot shows the sentinel."""
import ctypes

import numpy as np
import pytest

import _sendrecv
from _sendrecv import Link

SENTINEL = 0x00000000FFFFFFFF


@pytest.fixture(params=["oracle", "product"])
def fl(request, oracle, lib):
    return _sendrecv.flavours(oracle, lib)[request.param]


def flush(link, sizes):
    req = ctypes.c_int32(7)
    rc = link.fl.fn("recv_comm_flush")(link.r, len(sizes), (ctypes.c_int * len(sizes))(*sizes), ctypes.byref(req))
    return rc, req.value


def flush_test(link, req, slots, rails=4):
    done = ctypes.c_int(-1)
    rc = link.fl.fn("recv_comm_flush_test")(link.r, req, slots.ctypes.data_as(ctypes.c_void_p), rails,
                                            SENTINEL, ctypes.byref(done))
    return rc, done.value


def test_empty_receives_need_no_flush(fl):
    link = Link(fl)
    assert flush(link, [0]) == (0, -1)
    assert flush(link, [0, 0, 0, 0, 0, 0, 0, 0]) == (0, -1)
    assert link.recv_state()["num_inflight_reqs"] == 0
    link.close()


def test_one_flush_covers_all_buffers_and_completes_on_the_sentinels(fl):
    link = Link(fl)
    rc, req = flush(link, [0, 0, 4096, 0, 100])
    assert rc == 0 and req >= 0 and link.recv_state()["num_inflight_reqs"] == 1
    slots = np.zeros(4 * 8, dtype=np.uint64)                 # one 64-byte slot per rail
    assert flush_test(link, req, slots) == (0, 0)
    for rail in range(4):
        assert flush_test(link, req, slots) == (0, 0)        # not before the last rail's slot
        slots[rail * 8] = SENTINEL
    assert flush_test(link, req, slots) == (0, 1)
    assert link.recv_state()["num_inflight_reqs"] == 0
    assert flush_test(link, req, slots)[0] == -22            # the request is gone
    link.close()


def test_flush_requests_share_the_in_flight_limit_with_receives(fl):
    link = Link(fl)
    for _ in range(100):
        assert isinstance(link.recv([1], [1024]), int)
    reqs = []
    for _ in range(28):
        rc, req = flush(link, [1024])
        assert rc == 0 and req >= 0
        reqs.append(req)
    assert len(set(reqs)) == 28
    assert link.recv_state()["num_inflight_reqs"] == 128
    assert flush(link, [1024]) == (-28, -1)                  # -ENOSPC, as for a receive
    assert link.recv([1], [1024]) == -28
    assert flush(link, [0]) == (-28, -1)                     # the limit is checked before the sizes
    slots = np.full(4 * 8, SENTINEL, dtype=np.uint64)
    assert flush_test(link, reqs[5], slots) == (0, 1)
    rc, req = flush(link, [8])
    assert rc == 0 and req == reqs[5]                        # the freed handle is handed out again
    link.close()
