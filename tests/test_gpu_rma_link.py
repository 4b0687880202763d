"""The RMA entry points (include/ofi_amd_rma_abi.h) moving real bytes on the GPU: an initiator context
over the device fabric (ofi_amd_devfab_*), whose targets are this process.  The sequence is the
reference's tests/functional/rma.cpp:212-375 -- 64 puts and 64 put-signals of SEND_SIZE to a peer,
"test the oldest request, progress if it is not done", the target's signal reaching 64 -- followed by
what that test does not reach: multi-rail sizes, gets fenced by a flush, several target ranks, and more
operations than one sequence window holds, so that the target's ACKs have to come back.

Checked: destination bytes equal the source bytes (and nothing beyond them is touched), signal counters
equal the sum of what was sent, every request completes exactly once, and the initiator's window state
after the run is what the ACKs imply."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

ncclSuccess = 0
SIGNAL_INC, SIGNAL_ADD = 1, 2
SENTINEL = 0xdeadbeefdeadbeef
SIGNAL_BASE = 0x7F5500000000
vp = ctypes.c_void_p


class RmaLink:
    """createContext / regMrSym of a two-sided set-up, collapsed into one process."""

    def __init__(self, lib, nranks=2, rails=4, window=8 << 20, sq_depth=256, pool=4096, segments=1, seg_size=4096):
        self.lib, self.nranks = lib, nranks
        self.src = torch.randint(0, 256, (window,), dtype=torch.uint8, device="cuda")
        self.dst = [torch.full((window,), 0xCD, dtype=torch.uint8, device="cuda") for _ in range(nranks)]
        # a rank's signal window is `segments` regions side by side in its address range, each backed by
        # an allocation of its own (counters[r] is the first one's, segment_counters[r][k] the k-th's)
        self.segment_counters = [[torch.zeros(seg_size // 8, dtype=torch.int64, device="cuda") for _ in range(segments)]
                                 for _ in range(nranks)]
        self.counters = [segs[0] for segs in self.segment_counters]
        torch.cuda.synchronize()
        flat = [m.GinSignalRegion(SIGNAL_BASE + (r << 24) + k * seg_size, seg_size, self.segment_counters[r][k].data_ptr())
                for r in range(nranks) for k in range(segments)]
        regions = (m.GinSignalRegion * len(flat))(*flat)
        ids = (ctypes.c_uint32 * nranks)(*range(nranks))
        self.fab = vp()
        rc = lib.ofi_amd_devfab_create(rails, sq_depth, nranks, ids, regions, len(flat), _gpu.stream(), ctypes.byref(self.fab))
        assert rc == 0, rc
        self.ops = m.GinFabricOps()
        assert lib.ofi_amd_devfab_ops(self.fab, ctypes.byref(self.ops)) == 0
        self.ctx = vp()
        assert lib.ofi_amd_rma_ctx_create(nranks, rails, 131072, 64, ctypes.byref(self.ops), pool, 5000,
                                          ctypes.byref(self.ctx)) == 0
        # the target's ACKs reach the initiator the way handle_ack_completion does: straight into the context
        self.ack_fn = m.DEVFAB_ACK_FN(ctypes.cast(lib.ofi_amd_rma_ack_received, vp).value)
        assert lib.ofi_amd_devfab_on_ack(self.fab, self.ack_fn, self.ctx) == 0
        u64 = lambda vals: np.array(vals, dtype=np.uint64)
        keys = np.arange(nranks * 4, dtype=np.uint64) + 0x100

        def reg(local, remote):
            h = vp()
            addr = u64(remote)
            assert lib.ofi_amd_rma_mr_create(self.ctx, local, addr.ctypes.data, addr.ctypes.data, keys.ctypes.data,
                                             ctypes.byref(h)) == 0
            return h

        self.mr_src = reg(self.src.data_ptr(), [self.src.data_ptr()] * nranks)
        self.mr_dst = reg(self.dst[0].data_ptr(), [t.data_ptr() for t in self.dst])
        self.mr_sig = reg(SIGNAL_BASE, [SIGNAL_BASE + (r << 24) for r in range(nranks)])
        self.open = []

    def put(self, rank, src_off, dst_off, size, signal=None, flags=0):
        req = vp()
        if signal is None:
            rc = self.lib.ofi_amd_rma_iput(self.ctx, 0, src_off, self.mr_src, size, dst_off, self.mr_dst, rank, flags,
                                           ctypes.byref(req))
        else:
            slot, value, op = signal            # slot: index of the 8-byte counter within the rank's window
            rc = self.lib.ofi_amd_rma_iputSignal(self.ctx, 0, src_off, self.mr_src, size, dst_off, self.mr_dst, rank,
                                                 8 * slot, self.mr_sig, value, op, True, flags, ctypes.byref(req))
        assert rc == ncclSuccess and req.value, rc
        self.open.append(req)

    def get(self, rank, remote_off, local_off, size):
        """Reads `size` bytes of rank's destination buffer into this side's source buffer."""
        req = vp()
        rc = self.lib.ofi_amd_rma_iget(self.ctx, 0, remote_off, self.mr_dst, size, local_off, self.mr_src, rank, 0,
                                       ctypes.byref(req))
        assert rc == ncclSuccess and req.value, rc
        self.open.append(req)

    def poll_all(self, limit=5_000_000):
        """rma.cpp:316-330: test the oldest request; if it is not done, progress."""
        done = ctypes.c_int()
        for _ in range(limit):
            if not self.open:
                return
            assert self.lib.ofi_amd_rma_test(self.ctx, self.open[0], ctypes.byref(done)) == ncclSuccess
            if done.value:
                self.open.pop(0)
            else:
                assert self.lib.ofi_amd_rma_rmaProgress(self.ctx) == ncclSuccess
        raise AssertionError("%d requests never completed" % len(self.open))

    def wait_signal(self, rank, slot, value, limit=2_000_000):
        """The target polls its signal (rma.cpp:345-360) while the proxy keeps calling progress."""
        for _ in range(limit):
            assert self.lib.ofi_amd_rma_rmaProgress(self.ctx) == ncclSuccess
            if int(self.counters[rank][slot].item()) == value:
                return
        raise AssertionError("signal %d of rank %d stayed at %d" % (slot, rank, int(self.counters[rank][slot].item())))

    def stats(self):
        st = m.DevfabStats()
        assert self.lib.ofi_amd_devfab_stats(self.fab, ctypes.byref(st)) == 0
        return st

    def close(self):
        assert self.lib.ofi_amd_devfab_quiesce(self.fab, 0) == 0
        for h in (self.mr_src, self.mr_dst, self.mr_sig):
            assert self.lib.ofi_amd_rma_mr_destroy(h) == 0
        assert self.lib.ofi_amd_rma_ctx_destroy(self.ctx) == 0
        assert self.lib.ofi_amd_devfab_destroy(self.fab) == 0


@pytest.mark.parametrize("size", [5000, 4 << 20])
def test_sixty_four_puts_and_sixty_four_put_signals_then_the_signal_reads_sixty_four(lib, gpu, size):
    """size 5000 is the reference test's SEND_SIZE (tests/functional/functional_test.h:30): one write per
    operation; 4 MiB is striped over the four rails.  Every operation writes the same bytes to the same
    region, as there."""
    link = RmaLink(lib)
    for _ in range(64):
        link.put(1, 0, 0, size)
    for _ in range(64):
        link.put(1, 0, 0, size, signal=(1, 1, SIGNAL_INC))
    link.poll_all()
    link.wait_signal(1, 1, 64)
    torch.cuda.synchronize()
    assert torch.equal(link.dst[1][:size], link.src[:size])
    assert int((link.dst[1][size:size + 4096] != 0xCD).sum()) == 0 and int((link.dst[0] != 0xCD).sum()) == 0
    assert int(link.counters[1].sum().item()) == 64 and int(link.counters[0].sum().item()) == 0
    st = link.stats()
    stripes = 1 if size <= 131072 else 4
    assert st.writes == 128 * stripes and st.bytes == 128 * size and st.metas == 64
    link.close()


def test_distinct_regions_ragged_sizes_three_ranks_adds_and_aggregation(lib, gpu):
    """Random sizes from 0 bytes to 3 MiB at odd offsets to three target ranks, plain puts, increments and
    adds to several slots, some with the aggregation hint; the image of every destination buffer and
    every counter is rebuilt on the host from the argument stream."""
    rng = np.random.default_rng(11)
    nranks = 3
    link = RmaLink(lib, nranks=nranks, window=16 << 20)
    src = link.src.cpu().numpy()
    want_dst = [np.full(16 << 20, 0xCD, dtype=np.uint8) for _ in range(nranks)]
    want_cnt = [np.zeros(512, dtype=np.int64) for _ in range(nranks)]
    cursor = [0] * nranks
    choices = [0, 1, 7, 64, 65, 4096, 5000, 131072, 131073, 262145, 1 << 20, 3 << 20]
    for i in range(300):
        rank = int(rng.integers(0, nranks))
        size = int(rng.choice(choices))
        if cursor[rank] + size + 7 > (16 << 20):
            continue
        src_off = int(rng.integers(0, (16 << 20) - size + 1))
        dst_off = cursor[rank] + int(rng.integers(0, 4))       # destinations never overlap: order is free
        cursor[rank] = dst_off + size
        kind = int(rng.integers(0, 3))
        flags = int(rng.integers(0, 2))
        if kind == 0 and size:
            link.put(rank, src_off, dst_off, size, flags=flags)
        else:
            slot = int(rng.integers(0, 8))
            if kind == 1:
                link.put(rank, src_off, dst_off, size, signal=(slot, 1, SIGNAL_INC), flags=flags)
                want_cnt[rank][slot] += 1
            else:
                value = int(rng.integers(1, 1 << 40))
                link.put(rank, src_off, dst_off, size, signal=(slot, value, SIGNAL_ADD), flags=flags)
                want_cnt[rank][slot] += value
        want_dst[rank][dst_off:dst_off + size] = src[src_off:src_off + size]
        if i % 40 == 39:
            # an operation sent with the aggregation hint waits for its successor's doorbell: ring it
            assert lib.ofi_amd_devfab_ring_all(link.fab) == 0
            link.poll_all()
    # the last operations may sit behind a deferred doorbell (the aggregation hint promises a successor)
    assert lib.ofi_amd_devfab_ring_all(link.fab) == 0
    link.poll_all()
    assert lib.ofi_amd_devfab_quiesce(link.fab, 0) == 0
    for r in range(nranks):
        assert np.array_equal(link.dst[r].cpu().numpy(), want_dst[r]), r
        assert np.array_equal(link.counters[r].cpu().numpy(), want_cnt[r]), r
    assert _gpu.fetch_async_errors(lib) == 0
    link.close()


def test_gets_fenced_by_a_flush(lib, gpu):
    """iget reads a peer's buffer into the local one; iflush (nccl_ofi_rdma_gin_put_comm::iflush,
    src/rdma/gin/nccl_ofi_gin.cpp:941-1003) reads the sentinel buffer into one host slot per rail behind
    them, and its request is done when every slot shows the sentinel."""
    link = RmaLink(lib)
    pattern = torch.arange(1 << 20, dtype=torch.int32, device="cuda").view(torch.uint8)
    link.dst[1][:pattern.numel()] = pattern
    flush_buf, slots = vp(), vp()
    assert lib.ofi_amd_gpu_mem_alloc(ctypes.byref(flush_buf), 64) == 0
    assert lib.ofi_amd_flush_buffer_fill(flush_buf, SENTINEL, _gpu.stream()) == 0
    assert lib.ofi_amd_gpu_host_alloc(ctypes.byref(slots), 4 * 64) == 0
    torch.cuda.synchronize()
    assert lib.ofi_amd_rma_set_flush_buffers(link.ctx, slots, flush_buf.value, SENTINEL) == 0
    before = link.src.clone()
    for off, size in ((0, 5000), (8192 + 3, 262144), (1 << 20, 3 << 20)):
        link.get(1, off, off + 1, size)                      # remote offset off -> local offset off + 1
    req = vp()
    assert lib.ofi_amd_rma_iflush(link.ctx, 0, link.mr_src, 1, ctypes.byref(req)) == ncclSuccess and req.value
    link.open.append(req)
    link.poll_all()
    host_slots = np.ctypeslib.as_array(ctypes.cast(slots, ctypes.POINTER(ctypes.c_uint64)), shape=(32,))
    assert all(int(host_slots[8 * r]) == SENTINEL for r in range(4))
    torch.cuda.synchronize()
    want = before.clone()
    for off, size in ((0, 5000), (8192 + 3, 262144), (1 << 20, 3 << 20)):
        want[off + 1:off + 1 + size] = link.dst[1][off:off + size]
    assert torch.equal(link.src, want)
    st = link.stats()
    assert st.reads == 1 + 2 + 4 and st.flush_reads == 4 and st.writes == 0
    link.close()
    assert lib.ofi_amd_gpu_host_free(slots) == 0 and lib.ofi_amd_gpu_mem_free(flush_buf) == 0


def test_more_operations_than_a_window_holds_live_on_the_targets_acks(lib, gpu):
    """20,000 put-signals to one rank: the sequence window holds 8,192, so the initiator keeps going only
    because the target's ACKs come back through the fabric (the target answers every operation that asks
    for one, maybe_send_ack, src/rdma/gin/nccl_ofi_gin.cpp:1608-1620).  No call ever waits out the window."""
    link = RmaLink(lib, sq_depth=64, pool=8192)
    n = 20000
    for i in range(n):
        link.put(1, (i * 64) % (1 << 20), (i * 64) % (1 << 20), 64, signal=(i % 4, 1, SIGNAL_INC))
        if len(link.open) >= 512:
            link.poll_all()
    link.poll_all()
    assert lib.ofi_amd_devfab_quiesce(link.fab, 0) == 0
    assert link.counters[1][:4].tolist() == [n // 4] * 4
    assert torch.equal(link.dst[1][:1 << 20], link.src[:1 << 20])
    peer = lib.ofi_amd_rma_peer_state(link.ctx, 1).contents
    assert peer.tx_head == n & 0x3FFF or peer.tx_head == n      # a 14-bit cursor
    st = link.stats()
    assert st.acks > 0 and st.work_items <= n and st.metas == n
    window = (peer.tx_head - peer.tx_tail) & 0x3FFF
    assert window < 8192
    link.close()


def test_signal_window_of_two_segments_with_a_payload_across_the_middle(lib, gpu):
    """tests/functional/rma_multiseg_signal.cpp:285-405: the signal window is one address range backed by two
    allocations (the proxy there maps each segment on demand; here each is a region with counters of its
    own), 16 put-signals increment the first counter of segment 0 and 16 the first counter of segment 1, on
    every peer, each carrying 64 KiB that start 32 KiB before the 2 MiB mark of the payload windows."""
    seg = 2 << 20
    nranks = 3
    link = RmaLink(lib, nranks=nranks, segments=2, seg_size=seg)
    pay, pay_off = 64 << 10, seg - (32 << 10)
    for dst in range(1, nranks):
        for _ in range(16):
            link.put(dst, pay_off, pay_off, pay, signal=(0, 1, SIGNAL_INC))
            link.put(dst, pay_off, pay_off, pay, signal=(seg // 8, 1, SIGNAL_INC))
    link.poll_all()
    for dst in range(1, nranks):
        link.wait_signal(dst, 0, 16)
        for _ in range(1_000_000):
            assert lib.ofi_amd_rma_rmaProgress(link.ctx) == ncclSuccess
            if int(link.segment_counters[dst][1][0].item()) == 16:
                break
        assert int(link.segment_counters[dst][1][0].item()) == 16
        assert int(link.segment_counters[dst][0].sum().item()) == 16 and int(link.segment_counters[dst][1].sum().item()) == 16
        # "signals are delivered after the payload writes": the data is there once the counters are
        assert torch.equal(link.dst[dst][pay_off:pay_off + pay], link.src[pay_off:pay_off + pay])
        assert int((link.dst[dst][:pay_off] != 0xCD).sum()) == 0 and int((link.dst[dst][pay_off + pay:] != 0xCD).sum()) == 0
    assert int(link.segment_counters[0][0].sum().item()) == 0 and int((link.dst[0] != 0xCD).sum()) == 0
    assert _gpu.fetch_async_errors(lib) == 0
    link.close()


def test_context_and_fabric_torn_down_with_operations_in_flight(lib, gpu):
    """The RMA side of tests/functional/inflight_close.cpp: operations posted, some launched, none waited
    for; the context is destroyed, then the fabric (which waits for what it launched), and a fresh pair
    works afterwards."""
    for it in range(3):
        link = RmaLink(lib)
        for i in range(64):
            link.put(1, 0, i << 16, 1 << 16, signal=(i % 4, 1, SIGNAL_INC))
        if it:
            assert lib.ofi_amd_rma_rmaProgress(link.ctx) == ncclSuccess      # launches a group
            for i in range(8):
                link.put(1, 0, i << 16, 1 << 16)
        for h in (link.mr_src, link.mr_dst, link.mr_sig):
            assert lib.ofi_amd_rma_mr_destroy(h) == 0
        assert lib.ofi_amd_rma_ctx_destroy(link.ctx) == 0
        assert lib.ofi_amd_devfab_destroy(link.fab) == 0
        torch.cuda.synchronize()
    link = RmaLink(lib)
    link.put(1, 0, 0, 5000, signal=(0, 1, SIGNAL_INC))
    link.poll_all()
    link.wait_signal(1, 0, 1)
    assert torch.equal(link.dst[1][:5000], link.src[:5000])
    link.close()
    assert _gpu.fetch_async_errors(lib) == 0
