"""GPU parity: batched bounce copy + flush through the C ABI against the CPU oracle
(destination bytes, untouched bytes and flush words bit-exact)."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import _oracle
from aws_ofi_nccl_amd import synthetic

pytestmark = pytest.mark.gpu


def scatter(lib, src, arena_t, src_off, dst_off, length, flush=True):
    n = len(length)
    d_src = _gpu.to_dev(src)
    d_so, d_do, d_len = _gpu.to_dev(src_off), _gpu.to_dev(dst_off), _gpu.to_dev(length)
    d_flush = torch.full((max(n, 1),), -1, dtype=torch.int32, device="cuda")
    rc = lib.ofi_amd_bounce_scatter(d_src.data_ptr(), d_src.numel(), arena_t.data_ptr(), arena_t.numel(),
                                    d_so.data_ptr(), d_do.data_ptr(), d_len.data_ptr(), n,
                                    d_flush.data_ptr() if flush else None, _gpu.stream())
    assert rc == 0
    _gpu.sync()
    return _gpu.to_host(d_flush, np.uint32)[:n]


def oracle_scatter(oracle, src, arena, src_off, dst_off, length):
    flush = np.zeros(len(length), dtype=np.uint32)
    oracle.oracle_bounce_scatter(_oracle.ptr(src), _oracle.ptr(arena), _oracle.ptr(src_off),
                                 _oracle.ptr(dst_off), _oracle.ptr(length), len(length),
                                 _oracle.ptr(flush))
    return flush


@pytest.mark.parametrize("n,arena_mib,seed", [(1, 1, 0), (7, 1, 1), (1000, 16, 2), (4099, 64, 3)])
def test_parity_small(lib, oracle, gpu, n, arena_mib, seed):
    w = synthetic.bounce_workload(seed, n=n, arena_bytes=arena_mib << 20)
    src = synthetic.random_bytes(seed, w["src_bytes"] + 16)
    want = np.full(w["arena_bytes"], 0xCC, dtype=np.uint8)       # pre-filled: catches stray writes
    want_flush = oracle_scatter(oracle, src, want, w["src_off"], w["dst_off"], w["len"])
    arena = torch.full((w["arena_bytes"],), 0xCC, dtype=torch.uint8, device="cuda")
    flush = scatter(lib, src, arena, w["src_off"], w["dst_off"], w["len"])
    assert np.array_equal(arena.cpu().numpy(), want)
    assert np.array_equal(flush, want_flush)
    assert _gpu.fetch_async_errors(lib) == 0


def test_every_length_and_source_alignment(lib, oracle, gpu):
    """Lengths 0..300 plus the sizes around the 1 KiB / 4 KiB trip boundaries and the 8 KiB
    maximum, each at all 16 source byte alignments."""
    lens = list(range(0, 301)) + [1008, 1023, 1024, 1025, 1039, 4080, 4095, 4096, 4097, 4111,
                                  8176, 8191, 8192]
    length = np.array([l for l in lens for _ in range(16)], dtype=np.uint32)
    n = len(length)
    align = np.tile(np.arange(16, dtype=np.uint64), len(lens))
    slot = 8192 + 64
    src_off = np.arange(n, dtype=np.uint64) * np.uint64(slot) + align
    dst_off = np.random.default_rng(5).permutation(n).astype(np.uint64) * np.uint64(slot)
    src = synthetic.random_bytes(5, n * slot + 64)
    want = np.full(n * slot, 0x5A, dtype=np.uint8)
    want_flush = oracle_scatter(oracle, src, want, src_off, dst_off, length)
    arena = torch.full((n * slot,), 0x5A, dtype=torch.uint8, device="cuda")
    flush = scatter(lib, src, arena, src_off, dst_off, length)
    assert np.array_equal(arena.cpu().numpy(), want)
    assert np.array_equal(flush, want_flush)


def test_lengths_beyond_one_trip_and_every_row_count(lib, oracle, gpu):
    """Buffers larger than the 8 KiB eager limit loop over whole trips first; every number of
    1 KiB rows (1..8) in the last trip is hit at word-aligned and byte-misaligned sources."""
    lens = [r * 1024 + d for r in range(0, 9) for d in (-17, -1, 0, 1, 16)]
    lens += [8192 * k + d for k in (2, 3, 5) for d in (-1, 0, 1, 1000, 4097)] + [100_000, 1 << 20]
    lens = [l for l in lens if l >= 0]
    length = np.array([l for l in lens for _ in range(3)], dtype=np.uint32)
    n = len(length)
    align = np.tile(np.array([0, 1, 6], dtype=np.uint64), len(lens))
    room = ((length.astype(np.uint64) + np.uint64(64 + 63)) // np.uint64(64)) * np.uint64(64)
    starts = np.concatenate([[np.uint64(0)], np.cumsum(room)[:-1]]).astype(np.uint64)
    src_off = starts + align
    slot = np.uint64(((int(length.max()) + 127) // 64) * 64)
    dst_off = np.random.default_rng(6).permutation(n).astype(np.uint64) * slot
    total_src = int(starts[-1] + room[-1]) + 64
    src = synthetic.random_bytes(6, total_src)
    want = np.full(n * int(slot), 0x33, dtype=np.uint8)
    want_flush = oracle_scatter(oracle, src, want, src_off, dst_off, length)
    arena = torch.full((n * int(slot),), 0x33, dtype=torch.uint8, device="cuda")
    flush = scatter(lib, src, arena, src_off, dst_off, length)
    assert np.array_equal(arena.cpu().numpy(), want)
    assert np.array_equal(flush, want_flush)
    assert _gpu.fetch_async_errors(lib) == 0


def test_empty_batch_and_all_zero_lengths(lib, oracle, gpu):
    arena = torch.full((4096,), 9, dtype=torch.uint8, device="cuda")
    assert lib.ofi_amd_bounce_scatter(arena.data_ptr(), 4096, arena.data_ptr(), 4096, None, None, None, 0,
                                      None, _gpu.stream()) == 0
    src = np.arange(64, dtype=np.uint8)
    flush = scatter(lib, src, arena, np.zeros(8, np.uint64), np.arange(8, dtype=np.uint64) * 64,
                    np.zeros(8, np.uint32))
    assert torch.all(arena == 9) and list(flush) == [0x09090909] * 8


def test_without_flush_output(lib, oracle, gpu):
    w = synthetic.bounce_workload(8, n=500, arena_bytes=8 << 20)
    src = synthetic.random_bytes(8, w["src_bytes"] + 16)
    want = np.zeros(w["arena_bytes"], dtype=np.uint8)
    oracle_scatter(oracle, src, want, w["src_off"], w["dst_off"], w["len"])
    arena = torch.zeros(w["arena_bytes"], dtype=torch.uint8, device="cuda")
    scatter(lib, src, arena, w["src_off"], w["dst_off"], w["len"], flush=False)
    assert np.array_equal(arena.cpu().numpy(), want)


def test_flush_into_pinned_host_memory(lib, oracle, gpu):
    w = synthetic.bounce_workload(9, n=300, arena_bytes=4 << 20)
    src = synthetic.random_bytes(9, w["src_bytes"] + 16)
    want = np.zeros(w["arena_bytes"], dtype=np.uint8)
    want_flush = oracle_scatter(oracle, src, want, w["src_off"], w["dst_off"], w["len"])
    host = ctypes.c_void_p()
    assert lib.ofi_amd_gpu_host_alloc(ctypes.byref(host), 4 * 300) == 0
    dev = ctypes.c_void_p()
    assert lib.ofi_amd_gpu_host_get_device_pointer(ctypes.byref(dev), host) == 0
    arena = torch.zeros(w["arena_bytes"], dtype=torch.uint8, device="cuda")
    d_src = _gpu.to_dev(src)
    d = [_gpu.to_dev(w[k]) for k in ("src_off", "dst_off", "len")]
    assert lib.ofi_amd_bounce_scatter(d_src.data_ptr(), d_src.numel(), arena.data_ptr(), arena.numel(), d[0].data_ptr(),
                                      d[1].data_ptr(), d[2].data_ptr(), 300, dev, _gpu.stream()) == 0
    _gpu.sync()
    got = np.ctypeslib.as_array(ctypes.cast(host, ctypes.POINTER(ctypes.c_uint32)), shape=(300,)).copy()
    assert np.array_equal(got, want_flush)
    # flush-only entry point re-reads the same words
    d_flush = torch.zeros(300, dtype=torch.int32, device="cuda")
    assert lib.ofi_amd_flush_read(arena.data_ptr(), d[1].data_ptr(), 300, d_flush.data_ptr(),
                                  _gpu.stream()) == 0
    _gpu.sync()
    assert np.array_equal(_gpu.to_host(d_flush, np.uint32), want_flush)
    assert lib.ofi_amd_gpu_host_free(host) == 0


def test_out_of_range_destination_is_skipped_and_reported(lib, gpu):
    arena = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    src = np.full(256, 0xEE, dtype=np.uint8)
    # buffer 0 fine, 1 misaligned, 2 runs past the end, 3 starts past the end
    flush = scatter(lib, src, arena, np.zeros(4, np.uint64),
                    np.array([0, 100, 4096 - 64, 8192], dtype=np.uint64),
                    np.array([64, 64, 128, 8], dtype=np.uint32))
    got = arena.cpu().numpy()
    assert np.all(got[:64] == 0xEE) and not got[64:].any()
    assert _gpu.fetch_async_errors(lib) & 1
    assert _gpu.fetch_async_errors(lib) == 0          # fetch clears


def test_out_of_range_source_and_read_back_are_skipped_and_reported(lib, gpu):
    """A source range outside the bounce region, and a read-back whose four bytes would lie past
    the arena (a short buffer in its last bytes, or an empty one at its very end), are skipped."""
    src = np.full(256, 0xEE, dtype=np.uint8)
    for dst, soff, length, with_flush, bad in [
            (0, 0, 256, True, False), (0, 1, 256, True, True), (0, 257, 0, True, True), (0, 256, 0, True, False),
            (4096, 0, 0, True, True),            # empty buffer at the very end: nothing to read back from
            (4096, 0, 0, False, False),          # ... which is fine without a read-back
            (4096 - 64, 0, 64, True, False)]:
        arena = torch.zeros(4096, dtype=torch.uint8, device="cuda")
        scatter(lib, src, arena, np.array([soff], np.uint64), np.array([dst], np.uint64),
                np.array([length], np.uint32), flush=with_flush)
        got = arena.cpu().numpy()
        assert bool(_gpu.fetch_async_errors(lib) & 1) == bad, (dst, soff, length, with_flush)
        assert int(np.count_nonzero(got)) == (0 if bad else length)
    big = torch.zeros(8, dtype=torch.uint8, device="cuda")
    assert lib.ofi_amd_bounce_scatter(big.data_ptr(), 8, big.data_ptr(), 8, big.data_ptr(), big.data_ptr(),
                                      big.data_ptr(), (1 << 30) + 1, None, _gpu.stream()) == -22


def test_full_size_configuration(lib, oracle, gpu):
    """65,536 eager buffers of 0..8 KiB scattered over a 2 GiB arena."""
    w = synthetic.bounce_workload(1234)
    assert len(w["len"]) == 65536 and w["arena_bytes"] == 2 << 30
    src = synthetic.random_bytes(1234, w["src_bytes"] + 16)
    want = np.zeros(w["arena_bytes"], dtype=np.uint8)
    want_flush = oracle_scatter(oracle, src, want, w["src_off"], w["dst_off"], w["len"])
    arena = torch.zeros(w["arena_bytes"], dtype=torch.uint8, device="cuda")
    flush = scatter(lib, src, arena, w["src_off"], w["dst_off"], w["len"])
    assert np.array_equal(flush, want_flush)
    want_t = torch.from_numpy(want).cuda()
    assert torch.equal(arena, want_t)
    # size-independent property: the arena's byte sum equals the sum of all payload bytes
    assert int(arena.sum(dtype=torch.int64)) == int(src[:w["src_bytes"]].sum(dtype=np.int64))
    # idempotence: running the batch again changes nothing
    scatter(lib, src, arena, w["src_off"], w["dst_off"], w["len"])
    assert torch.equal(arena, want_t)


def test_device_copy_interface(lib, gpu):
    """The patterns of tests/unit/gdrcopy.cpp:15-133 through the nccl_ofi_device_copy mirror."""
    size = 2 << 20
    buf = torch.zeros(size, dtype=torch.uint8, device="cuda")
    h = ctypes.c_void_p()
    assert lib.ofi_amd_devcopy_register(buf.data_ptr(), size, ctypes.byref(h)) == 0
    # MI355X boxes have a large BAR and the runtime maps its allocations into the process: the small
    # copies below are CPU stores and loads, not copy-engine calls
    assert lib.ofi_amd_devcopy_cpu_mapped(h) == 1
    a = np.full(size, ord("A"), dtype=np.uint8)
    assert lib.ofi_amd_devcopy_to_device(a.ctypes.data, h, 0, size) == 0
    back = np.zeros(size, dtype=np.uint8)
    assert lib.ofi_amd_devcopy_from_device(h, 0, back.ctypes.data, size) == 0
    assert np.all(back == ord("A"))
    for i in range(10):
        b = np.array([ord("a") + i], dtype=np.uint8)
        assert lib.ofi_amd_devcopy_to_device(b.ctypes.data, h, i, 1) == 0
    for i in range(10):
        b = np.zeros(1, dtype=np.uint8)
        assert lib.ofi_amd_devcopy_from_device(h, i, b.ctypes.data, 1) == 0
        assert b[0] == ord("a") + i
    assert bytes(buf[:12].cpu().numpy()) == b"abcdefghijAA"
    assert lib.ofi_amd_devcopy_to_device(a.ctypes.data, h, size - 4, 8) < 0     # past the region
    assert lib.ofi_amd_devcopy_forced_pcie_copy() == 0
    assert lib.ofi_amd_devcopy_deregister(h) == 0
    host = np.zeros(16, dtype=np.uint8)
    assert lib.ofi_amd_devcopy_register(host.ctypes.data, 16, ctypes.byref(h)) < 0   # not device memory


def test_device_copy_is_ordered_with_gpu_work(lib, gpu):
    """The copies are CPU stores and loads through the mapping of device memory (no copy engine, no
    stream): a store is seen by a kernel launched after the call returns, a load sees what a
    kernel that has completed wrote -- for every size class (CPU path and copy-engine path) and at
    odd offsets."""
    size = 8 << 20
    buf = torch.zeros(size, dtype=torch.uint8, device="cuda")
    h = ctypes.c_void_p()
    assert lib.ofi_amd_devcopy_register(buf.data_ptr(), size, ctypes.byref(h)) == 0
    rng = np.random.default_rng(7)
    for n, off in [(1, 3), (8, 8), (63, 1), (64, 64), (255, 5), (256, 0), (257, 11), (4096, 4097),
                   (65537, 99), (2 << 20, 7), ((2 << 20) + 1, 13), (3 << 20, 1 << 20)]:
        data = rng.integers(0, 256, n, dtype=np.uint8)
        assert lib.ofi_amd_devcopy_to_device(data.ctypes.data, h, off, n) == 0
        # a kernel launched now reads the bytes and writes their complement next to them
        out = (buf[off:off + n] ^ 0xFF).clone()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), data ^ 0xFF), (n, off)
        buf[off:off + n] = out                       # a kernel writes the region ...
        torch.cuda.synchronize()
        back = np.zeros(n, dtype=np.uint8)
        assert lib.ofi_amd_devcopy_from_device(h, off, back.ctypes.data, n) == 0   # ... and the load sees it
        assert np.array_equal(back, data ^ 0xFF), (n, off)
        # nothing around the range was touched
        assert int(buf[:off].sum()) + int(buf[off + n:].sum()) == 0
        buf.zero_()
        torch.cuda.synchronize()
    # a signal counter updated from the host the way the reference's GDRCopy worker does
    # (read-modify-write of 8 bytes, src/rdma/gin/nccl_ofi_gin.cpp:1193-1256)
    cnt = torch.zeros(8, dtype=torch.int64, device="cuda")
    assert lib.ofi_amd_devcopy_deregister(h) == 0
    assert lib.ofi_amd_devcopy_register(cnt.data_ptr(), 64, ctypes.byref(h)) == 0
    word = np.zeros(1, dtype=np.uint64)
    for k in range(100):
        assert lib.ofi_amd_devcopy_from_device(h, 24, word.ctypes.data, 8) == 0
        word[0] += 3
        assert lib.ofi_amd_devcopy_to_device(word.ctypes.data, h, 24, 8) == 0
    torch.cuda.synchronize()
    assert cnt.cpu().tolist() == [0, 0, 0, 300, 0, 0, 0, 0]
    assert lib.ofi_amd_devcopy_deregister(h) == 0


def test_gpu_glue(lib, gpu):
    p = ctypes.c_void_p()
    assert lib.ofi_amd_gpu_mem_alloc(ctypes.byref(p), 1 << 20) == 0
    dev = ctypes.c_int(-5)
    assert lib.ofi_amd_gpu_get_device_for_addr(p, ctypes.byref(dev)) == 0 and dev.value == 0
    base, size = ctypes.c_void_p(), ctypes.c_size_t()
    assert lib.ofi_amd_gpu_get_address_range(ctypes.c_void_p(p.value + 4096), ctypes.byref(base),
                                             ctypes.byref(size)) == 0
    assert base.value == p.value and size.value >= 1 << 20
    is_host = ctypes.c_int(-1)
    assert lib.ofi_amd_gpu_seg_is_host(p, ctypes.byref(is_host)) == 0 and is_host.value == 0
    data = np.arange(256, dtype=np.uint8)
    assert lib.ofi_amd_gpu_mem_copy_host_to_device(p, data.ctypes.data, 256) == 0
    back = np.zeros(256, dtype=np.uint8)
    assert lib.ofi_amd_gpu_mem_copy_device_to_host(back.ctypes.data, p, 256) == 0
    assert np.array_equal(back, data)
    assert lib.ofi_amd_gpu_mem_free(p) == 0
    cur = ctypes.c_int(-1)
    assert lib.ofi_amd_gpu_get_current_device(ctypes.byref(cur)) == 0 and cur.value == 0
    assert lib.ofi_amd_gpu_set_current_device(0) == 0
    assert lib.ofi_amd_gpu_have_dma_buf_attr() in (0, 1)
    host = np.zeros(8, dtype=np.uint8)
    assert lib.ofi_amd_gpu_seg_is_host(host.ctypes.data, ctypes.byref(is_host)) == 0 and is_host.value == 1
    assert lib.ofi_amd_gpu_get_device_for_addr(host.ctypes.data, ctypes.byref(dev)) < 0 and dev.value == -1


def test_dma_buf_export_of_device_memory(lib, gpu, capsys):
    """nccl_net_ofi_gpu_get_dma_buf_fd (src/nccl_ofi_rocm.cpp:129-139), called as the reference
    calls it for its flush buffer (src/nccl_ofi_rdma.cpp:3842-3845: a page-aligned address, one
    system page) and for a whole registration: a dma-buf file descriptor and offset 0.  Where the
    device cannot export (have_dma_buf_attr 0) the call fails with a negative errno instead."""
    import os
    page = os.sysconf("SC_PAGE_SIZE")
    p = ctypes.c_void_p()
    assert lib.ofi_amd_gpu_mem_alloc(ctypes.byref(p), 4 << 20) == 0 and p.value % page == 0
    have = lib.ofi_amd_gpu_have_dma_buf_attr()
    assert have in (0, 1)
    links = []
    for addr, size in ((p.value, page), (p.value + 16 * page, 1 << 20), (p.value, 4 << 20)):
        fd, off = ctypes.c_int(-1), ctypes.c_size_t(99)
        rc = lib.ofi_amd_gpu_get_dma_buf_fd(ctypes.c_void_p(addr), size, ctypes.byref(fd), ctypes.byref(off))
        if not have:
            assert rc < 0
            continue
        assert rc == 0 and fd.value >= 0 and off.value == 0
        st = os.fstat(fd.value)                                  # a live descriptor of this process
        assert st.st_ino > 0
        link = os.readlink("/proc/self/fd/%d" % fd.value)
        assert "dmabuf" in link, link                            # an anonymous dma-buf inode
        links.append(link)
        try:
            end = os.lseek(fd.value, 0, os.SEEK_END)             # dma-buf files report their size
            assert end >= size, (end, size)
        except OSError:
            pass
        os.close(fd.value)
        with pytest.raises(OSError):
            os.fstat(fd.value)                                   # the caller owns the descriptor: closed means gone
    # which branch ran is part of the result: say so whatever pytest captures
    with capsys.disabled():
        print("\n[dma-buf] ofi_amd_gpu_have_dma_buf_attr() = %d; exported descriptors: %s" % (have, links or "none"))
    # the exported memory is untouched and still usable
    data = np.arange(256, dtype=np.uint8)
    back = np.zeros(256, dtype=np.uint8)
    assert lib.ofi_amd_gpu_mem_copy_host_to_device(p, data.ctypes.data, 256) == 0
    assert lib.ofi_amd_gpu_mem_copy_device_to_host(back.ctypes.data, p, 256) == 0 and np.array_equal(back, data)
    # a pointer the runtime does not know as device memory, and missing outputs
    host = np.zeros(2 * page, dtype=np.uint8)
    aligned = (host.ctypes.data + page - 1) // page * page
    fd, off = ctypes.c_int(-1), ctypes.c_size_t(0)
    assert lib.ofi_amd_gpu_get_dma_buf_fd(ctypes.c_void_p(aligned), page, ctypes.byref(fd), ctypes.byref(off)) < 0
    assert lib.ofi_amd_gpu_get_dma_buf_fd(p, page, None, ctypes.byref(off)) == -22
    assert lib.ofi_amd_gpu_get_dma_buf_fd(p, page, ctypes.byref(fd), None) == -22
    assert lib.ofi_amd_gpu_mem_free(p) == 0
    assert _gpu.fetch_async_errors(lib) == 0


@pytest.mark.parametrize("sentinel", [0x00000000FFFFFFFF, 0xDEADBEEFDEADBEEF])
def test_sentinel_flush_reaches_every_rail_slot(lib, oracle, gpu, sentinel):
    """GPU flush buffer -> one 64-byte pinned host slot per rail; complete when each slot's
    first word shows the sentinel (RDMA and GIN sentinels of the reference)."""
    d_buf = torch.zeros(8, dtype=torch.int64, device="cuda")
    assert lib.ofi_amd_flush_buffer_fill(d_buf.data_ptr(), sentinel, _gpu.stream()) == 0
    _gpu.sync()
    assert np.all(_gpu.to_host(d_buf, np.uint64) == np.uint64(sentinel))
    for rails in (1, 2, 3, 4):
        slots = torch.zeros(8 * 4 + 8, dtype=torch.int64, pin_memory=True)
        host = slots.numpy().view(np.uint64)
        ptr = ctypes.c_void_p(slots.data_ptr())
        assert lib.ofi_amd_flush_test(ptr, rails, sentinel) == 0
        assert lib.ofi_amd_flush_post(d_buf.data_ptr(), ptr, rails, _gpu.stream()) == 0
        _gpu.sync()
        assert lib.ofi_amd_flush_test(ptr, rails, sentinel) == 1
        want = np.zeros(40, dtype=np.uint64)
        buf_host = _gpu.to_host(d_buf, np.uint64).copy()
        oracle.oracle_flush_post(ctypes.c_void_p(buf_host.ctypes.data), ctypes.c_void_p(want.ctypes.data),
                                 rails)
        assert np.array_equal(host, want)               # slots of unused rails and the guard stay zero
    assert lib.ofi_amd_flush_post(d_buf.data_ptr(), ptr, 0, _gpu.stream()) == -22
    assert lib.ofi_amd_flush_post(d_buf.data_ptr(), ptr, 5, _gpu.stream()) == -22
    assert lib.ofi_amd_flush_post(None, ptr, 1, _gpu.stream()) == -22
    assert lib.ofi_amd_flush_buffer_fill(None, sentinel, _gpu.stream()) == -22
