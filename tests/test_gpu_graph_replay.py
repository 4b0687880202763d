"""The launch-bound entry points recorded into one HIP graph and replayed: striping (two
launches), bounce copy, eager-format copy and signal delivery.  None of them allocates or
synchronises once its stream has been used, so they can be captured; every replay is
checked against the oracle, with eager work and synchronisations between replays."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import _oracle
import aws_ofi_nccl_amd as m
from aws_ofi_nccl_amd import synthetic

pytestmark = pytest.mark.gpu


def test_graph_of_hot_path_launches_replays_exactly(lib, oracle, gpu):
    rng = np.random.default_rng(77)
    s = torch.cuda.Stream()
    sp = ctypes.c_void_p(s.cuda_stream)

    # striping inputs; the scheduler state lives on the device and advances with every replay
    n_msg = 50_000
    sizes = synthetic.stripe_sizes(5, n_msg)
    st = m.SchedState(2, 1, 64, 131072, 4, 0)
    d_state = _gpu.to_dev(np.frombuffer(bytes(st), dtype=np.uint8).copy())
    d_sizes = _gpu.to_dev(sizes)
    d_num = torch.zeros(n_msg, dtype=torch.int32, device="cuda")
    d_xf = torch.zeros(n_msg * 12, dtype=torch.int64, device="cuda")

    # bounce copy inputs
    w = synthetic.bounce_workload(9, n=2048, arena_bytes=32 << 20)
    src = synthetic.random_bytes(9, w["src_bytes"] + 16)
    d_src, d_so, d_do, d_len = (_gpu.to_dev(x) for x in (src, w["src_off"], w["dst_off"], w["len"]))
    d_arena = torch.zeros(w["arena_bytes"], dtype=torch.uint8, device="cuda")
    d_flush = torch.zeros(2048, dtype=torch.int32, device="cuda")
    want_arena = np.zeros(w["arena_bytes"], dtype=np.uint8)
    want_flush = np.zeros(2048, dtype=np.uint32)
    oracle.oracle_bounce_scatter(_oracle.ptr(src), _oracle.ptr(want_arena), _oracle.ptr(w["src_off"]),
                                 _oracle.ptr(w["dst_off"]), _oracle.ptr(w["len"]), 2048,
                                 _oracle.ptr(want_flush))

    # signal delivery inputs: counters accumulate across replays
    n_sig, base = 10_000, 0x7F0000000000
    work = np.zeros(n_sig, dtype=np.dtype([("base", "<u8"), ("offset", "<u8"), ("value", "<u8"),
                                            ("peer", "<u4"), ("gate_seq", "<u2"), ("run_len", "<u2")]))
    work["base"], work["run_len"] = base, 1
    work["offset"] = 8 * rng.integers(0, 128, n_sig).astype(np.uint64)
    work["value"] = rng.integers(0, 1 << 64, n_sig, dtype=np.uint64)
    d_work = _gpu.to_dev(work.view(np.uint8))
    d_cnt = torch.zeros(128, dtype=torch.int64, device="cuda")
    regions = (m.GinSignalRegion * 1)(m.GinSignalRegion(base, 1024, d_cnt.data_ptr()))
    per_replay = np.zeros(128, dtype=np.uint64)
    with np.errstate(over="ignore"):
        np.add.at(per_replay, (work["offset"] // 8).astype(np.int64), work["value"])

    # eager-format copy and table copy out of the same source bytes
    n_e, stride = 512, 8320
    e_len = rng.integers(0, 8185, n_e).astype(np.uint32)
    e_rx = (rng.permutation(n_e).astype(np.uint64) * np.uint64(stride))
    e_dst = (np.arange(n_e, dtype=np.uint64) * np.uint64(8192 + 64) + rng.integers(0, 16, n_e).astype(np.uint64))
    d_earena = torch.zeros(n_e * (8192 + 64), dtype=torch.uint8, device="cuda")
    d_erx, d_elen, d_edst = _gpu.to_dev(e_rx), _gpu.to_dev(e_len), _gpu.to_dev(e_dst)
    d_copied = torch.zeros(n_e, dtype=torch.int32, device="cuda")
    want_earena = np.zeros(n_e * (8192 + 64), dtype=np.uint8)
    oracle.oracle_eager_copy_batch(_oracle.ptr(src), _oracle.ptr(e_rx), _oracle.ptr(e_len), _oracle.ptr(want_earena),
                                   _oracle.ptr(e_dst), _oracle.ptr(e_len), n_e, None)
    n_t = 300
    t_len = rng.integers(1, 70000, n_t).astype(np.uint32)
    t_src_off = rng.integers(0, w["src_bytes"] - 70000, n_t).astype(np.uint64)
    t_dst_off = np.concatenate(([0], np.cumsum(t_len.astype(np.uint64) + np.uint64(3))[:-1])).astype(np.uint64)
    d_tarena = torch.zeros(int(t_dst_off[-1]) + 70000, dtype=torch.uint8, device="cuda")
    d_tsrc = _gpu.to_dev(t_src_off + np.uint64(d_src.data_ptr()))
    d_tdst = _gpu.to_dev(t_dst_off + np.uint64(d_tarena.data_ptr()))
    d_tlen = _gpu.to_dev(t_len)
    d_parena = torch.zeros_like(d_tarena)    # the same table through the launch with a wavefront per 8 KiB
    d_pdst = _gpu.to_dev(t_dst_off + np.uint64(d_parena.data_ptr()))
    want_tarena = np.zeros(d_tarena.numel(), dtype=np.uint8)
    for a, b, l in zip(t_src_off, t_dst_off, t_len):
        want_tarena[int(b):int(b) + int(l)] = src[int(a):int(a) + int(l)]

    def launches():
        assert lib.ofi_amd_eager_copy_batch(d_src.data_ptr(), d_erx.data_ptr(), d_elen.data_ptr(),
                                            d_earena.data_ptr(), d_edst.data_ptr(), d_elen.data_ptr(), n_e,
                                            d_copied.data_ptr(), None, sp) == 0
        assert lib.ofi_amd_copy_table(d_tsrc.data_ptr(), d_tdst.data_ptr(), d_tlen.data_ptr(), n_t, sp) == 0
        assert lib.ofi_amd_copy_table_pieces(d_tsrc.data_ptr(), d_pdst.data_ptr(), d_tlen.data_ptr(), n_t, 70000,
                                             sp) == 0
        assert lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n_msg, 128, d_num.data_ptr(),
                                       d_xf.data_ptr(), sp) == 0
        assert lib.ofi_amd_bounce_scatter(d_src.data_ptr(), d_src.numel(), d_arena.data_ptr(), w["arena_bytes"],
                                          d_so.data_ptr(), d_do.data_ptr(), d_len.data_ptr(), 2048,
                                          d_flush.data_ptr(), sp) == 0
        assert lib.ofi_amd_gin_signal_apply(d_work.data_ptr(), n_sig, regions, 1, None, sp) == 0

    # first use of the stream sets up the per-stream striping scratch (an allocation): outside capture
    with torch.cuda.stream(s):
        launches()
    s.synchronize()
    ost = _oracle.Sched(2, 1, 64, 131072, 4, 0)
    num = np.zeros(n_msg, dtype=np.uint32)
    xf = np.zeros((n_msg, 4, 3), dtype=np.uint64)
    oracle.oracle_sched_batch(ctypes.byref(ost), _oracle.ptr(sizes), n_msg, 128, _oracle.ptr(num),
                              _oracle.ptr(xf))
    assert np.array_equal(_gpu.to_host(d_xf, np.uint64).reshape(n_msg, 4, 3), xf)
    counters = per_replay.copy()

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        launches()

    for replay in range(4):
        # eager work and a synchronisation between replays; outputs wiped so a replay must rewrite them
        d_arena.zero_()
        d_earena.zero_()
        d_tarena.zero_()
        d_parena.zero_()
        d_copied.zero_()
        d_flush.zero_()
        d_num.fill_(-1)
        d_xf.fill_(-1)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        # the oracle advances its own state by one batch: replay k continues where k-1 stopped
        oracle.oracle_sched_batch(ctypes.byref(ost), _oracle.ptr(sizes), n_msg, 128, _oracle.ptr(num),
                                  _oracle.ptr(xf))
        assert np.array_equal(_gpu.to_host(d_num, np.uint32), num), replay
        assert np.array_equal(_gpu.to_host(d_xf, np.uint64).reshape(n_msg, 4, 3), xf), replay
        got_state = m.SchedState.from_buffer_copy(d_state.cpu().numpy().tobytes())
        assert (got_state.rr_small_counter, got_state.rr_counter) == (ost.rr_small_counter, ost.rr_counter)
        assert np.array_equal(d_arena.cpu().numpy(), want_arena), replay
        assert np.array_equal(d_earena.cpu().numpy(), want_earena), replay
        assert np.array_equal(_gpu.to_host(d_copied, np.uint32), e_len), replay
        assert np.array_equal(d_tarena.cpu().numpy(), want_tarena), replay
        assert np.array_equal(d_parena.cpu().numpy(), want_tarena), replay
        assert np.array_equal(_gpu.to_host(d_flush, np.uint32), want_flush), replay
        with np.errstate(over="ignore"):
            counters += per_replay
        assert np.array_equal(_gpu.to_host(d_cnt, np.uint64), counters), replay
    assert _gpu.fetch_async_errors(lib) == 0
