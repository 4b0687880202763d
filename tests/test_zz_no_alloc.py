"""GPU parity of the striping entry point that allocates nothing (ofi_amd_sched_batch_noalloc)
against ofi_amd_sched_batch and the CPU oracle: two calls in a row on the same scratch, the
second with a smaller input, then a batch large enough for the separate scan launch."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import _oracle
import aws_ofi_nccl_amd as m
from aws_ofi_nccl_amd import synthetic

pytestmark = pytest.mark.gpu


def dev_state(rails, min_stripe, max_small, seeds):
    st = m.SchedState(seeds[0], seeds[1], max_small, min_stripe, rails, 0)
    return _gpu.to_dev(np.frombuffer(bytes(st), dtype=np.uint8).copy())


def run(fn, d_state, d_sizes, n):
    d_num = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    d_xf = torch.full((n * 12,), -1, dtype=torch.int64, device="cuda")
    rc = fn(d_state.data_ptr(), d_sizes.data_ptr(), n, 128, d_num.data_ptr(), d_xf.data_ptr(), _gpu.stream())
    _gpu.sync()
    assert rc == 0
    return _gpu.to_host(d_num, np.uint32), _gpu.to_host(d_xf, np.uint64).reshape(n, 4, 3), \
        d_state.cpu().numpy().tobytes()


def test_noalloc_matches_allocating_entry_point(lib, oracle, gpu):
    assert lib.ofi_amd_gpu_init() == 0
    # second call smaller than the first (stale totals of the first stay in the scratch),
    # third call beyond 4096 tiles of 1024 messages: the scan launch and the prefix half
    for seed, n in ((11, 300007), (12, 1234), (13, (1 << 23) + 4099)):
        sizes = synthetic.stripe_sizes(seed, n)
        sizes[::7] = sizes[::7] % np.uint64(150)
        d_sizes = _gpu.to_dev(sizes)
        got = run(lib.ofi_amd_sched_batch_noalloc, dev_state(4, 131072, 64, (3, 1)), d_sizes, n)
        ref = run(lib.ofi_amd_sched_batch, dev_state(4, 131072, 64, (3, 1)), d_sizes, n)
        assert np.array_equal(got[0], ref[0]) and np.array_equal(got[1], ref[1]) and got[2] == ref[2], n
        if n <= 400000:
            want_num, want_xf, ost = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (3, 1))
            assert np.array_equal(got[0], want_num) and np.array_equal(got[1], want_xf)
            st = m.SchedState.from_buffer_copy(got[2])
            assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)
        assert _gpu.fetch_async_errors(lib) == 0


def test_noalloc_at_its_largest_batch(lib, gpu):
    """2^26 messages use every tile word of the fixed scratch (65,536 tiles of 1,024).  Compared on
    the device with the allocating entry point's output for the same batch (6.4 GB of rows each),
    and through what does not depend on the size: every message's stripes add up to its size."""
    assert lib.ofi_amd_gpu_init() == 0
    n = 1 << 26
    gen = torch.Generator(device="cuda").manual_seed(5)
    octave = torch.randint(0, 28, (n,), generator=gen, device="cuda", dtype=torch.int64)
    d_sizes = (torch.randint(0, 1 << 28, (n,), generator=gen, device="cuda", dtype=torch.int64) >> (28 - octave))
    outs = []
    for fn in (lib.ofi_amd_sched_batch_noalloc, lib.ofi_amd_sched_batch):
        d_state = dev_state(4, 131072, 64, (2, 3))
        d_num = torch.full((n,), -1, dtype=torch.int32, device="cuda")
        d_xf = torch.full((n * 12,), -1, dtype=torch.int64, device="cuda")
        assert fn(d_state.data_ptr(), d_sizes.data_ptr(), n, 128, d_num.data_ptr(), d_xf.data_ptr(),
                  _gpu.stream()) == 0
        _gpu.sync()
        outs.append((d_num, d_xf, d_state))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert torch.equal(outs[0][2], outs[1][2])
    rows = outs[0][1].view(n, 4, 3)
    assert torch.equal(rows[:, :, 2].sum(dim=1), d_sizes)
    assert int(outs[0][0].min()) == 1 and int(outs[0][0].max()) == 4
    assert _gpu.fetch_async_errors(lib) == 0


def test_noalloc_calls_leave_free_device_memory_where_it_was(lib, gpu):
    """What the entry point is for: after ofi_amd_gpu_init() (which records the scratch array's
    address on every GPU) a call takes no device memory -- the runtime's count of free bytes
    (hipMemGetInfo) is the same before and after calls of several sizes, the larger ones through
    the separate scan launch, on a stream that has never been used with the allocating entry
    point (that one would allocate its per-stream scratch on such a stream)."""
    assert lib.ofi_amd_gpu_init() == 0
    side = torch.cuda.Stream()
    stream = ctypes.c_void_p(side.cuda_stream)
    big = (1 << 22) + 777
    d_sizes = _gpu.to_dev(synthetic.stripe_sizes(21, big))
    d_state = dev_state(4, 131072, 64, (0, 0))
    d_num = torch.zeros(big, dtype=torch.int32, device="cuda")
    d_xf = torch.zeros(big * 12, dtype=torch.int64, device="cuda")
    call = lambda n: lib.ofi_amd_sched_batch_noalloc(d_state.data_ptr(), d_sizes.data_ptr(), n, 128, d_num.data_ptr(),
                                                     d_xf.data_ptr(), stream)
    assert call(1000) == 0 and call(big) == 0              # code objects of every kernel are on the device now
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for n in (1, 513, 300007, big, 1234, 3_000_000):
        assert call(n) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert _gpu.fetch_async_errors(lib) == 0
    # the count does move when device memory is taken: the comparison above can tell
    p = ctypes.c_void_p()
    assert lib.ofi_amd_gpu_mem_alloc(ctypes.byref(p), 64 << 20) == 0
    assert torch.cuda.mem_get_info()[0] <= free_before - (64 << 20)
    assert lib.ofi_amd_gpu_mem_free(p) == 0


def test_noalloc_rejects_oversized_batch(lib, gpu):
    assert lib.ofi_amd_gpu_init() == 0
    d = torch.zeros(16, dtype=torch.int64, device="cuda")
    rc = lib.ofi_amd_sched_batch_noalloc(d.data_ptr(), d.data_ptr(), (1 << 26) + 1, 128, d.data_ptr(),
                                         d.data_ptr(), _gpu.stream())
    assert rc == -7                                            # -E2BIG, nothing launched
    _gpu.sync()
