"""GPU parity: batched rail striping through the C ABI against the CPU oracle
(stripe counts, (rail, offset, length) triples, padding and final counters bit-exact)."""
import ctypes
import json
import os

import numpy as np
import pytest
import torch

import _gpu
import _oracle
import aws_ofi_nccl_amd as m
from aws_ofi_nccl_amd import synthetic

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "scheduler_kat.json")


def dev_state(rails, min_stripe, max_small, seeds):
    st = m.SchedState(seeds[0], seeds[1], max_small, min_stripe, rails, 0)
    return _gpu.to_dev(np.frombuffer(bytes(st), dtype=np.uint8).copy())


def read_state(d_state):
    return m.SchedState.from_buffer_copy(d_state.cpu().numpy().tobytes())


def gpu_batch(lib, d_state, sizes, align=128):
    n = len(sizes)
    d_sizes = _gpu.to_dev(sizes) if n else torch.zeros(1, dtype=torch.int64, device="cuda")
    d_num = torch.full((max(n, 1),), -1, dtype=torch.int32, device="cuda")
    d_xf = torch.full((max(n, 1) * 12,), -1, dtype=torch.int64, device="cuda")
    rc = lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n, align, d_num.data_ptr(),
                                 d_xf.data_ptr(), _gpu.stream())
    _gpu.sync()
    return rc, _gpu.to_host(d_num, np.uint32)[:n], _gpu.to_host(d_xf, np.uint64)[:n * 12].reshape(n, 4, 3)


def test_reference_known_answers_on_gpu(lib, gpu):
    doc = json.load(open(GOLDEN))
    sizes = np.array([c["size"] for c in doc["calls"]], dtype=np.uint64)
    d_state = dev_state(doc["num_rails"], doc["min_stripe_size"], doc["max_small_msg_size"], (0, 0))
    rc, num, xf = gpu_batch(lib, d_state, sizes, doc["align"])
    assert rc == 0
    for i, call in enumerate(doc["calls"]):
        got = [(int(xf[i, k, 0]), int(xf[i, k, 1]), int(xf[i, k, 2])) for k in range(num[i])]
        assert got == [tuple(t) for t in call["stripes"]], call["size"]


@pytest.mark.parametrize("n", [1, 63, 64, 255, 256, 257, 1023, 1024, 1025, 4096, 100003])
@pytest.mark.parametrize("rails,min_stripe,max_small,seeds", [(4, 131072, 64, (0, 0)),
                                                              (3, 100000, 64, (2, 1)),
                                                              (2, 4096, 0, (1, 1)),
                                                              (1, 131072, 64, (0, 0)),
                                                              (4, 4097, 1000, (3, 2))])
def test_parity_random(lib, oracle, gpu, n, rails, min_stripe, max_small, seeds):
    sizes = synthetic.stripe_sizes(n * 31 + rails, n)
    sizes[::5] = sizes[::5] % np.uint64(200)                   # enough small messages
    want_num, want_xf, ost = _oracle.sched_batch(oracle, sizes, rails, min_stripe, max_small, seeds)
    d_state = dev_state(rails, min_stripe, max_small, seeds)
    rc, num, xf = gpu_batch(lib, d_state, sizes)
    assert rc == 0
    assert np.array_equal(num, want_num)
    assert np.array_equal(xf, want_xf)                          # includes zero padding and unused rows
    st = read_state(d_state)
    assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)
    assert (st.max_small_msg_size, st.min_stripe_size, st.num_rails) == (max_small, min_stripe, rails)


@pytest.mark.parametrize("n", [1, 2, 511, 513, 70001, 3_000_001])
def test_sizes_array_at_an_odd_eight_byte_offset(lib, oracle, gpu, n):
    """The sizes array only has to be 8-byte aligned."""
    sizes = synthetic.stripe_sizes(n + 5, n)
    sizes[::7] = sizes[::7] % np.uint64(100)
    want_num, want_xf, ost = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (3, 1))
    for shift in (0, 1):
        d_state = dev_state(4, 131072, 64, (3, 1))
        d_all = _gpu.to_dev(np.concatenate([np.zeros(shift, dtype=np.uint64), sizes]))
        d_sizes = d_all[shift:]
        assert d_sizes.data_ptr() % 16 == 8 * shift
        d_num = torch.full((n,), -1, dtype=torch.int32, device="cuda")
        d_xf = torch.full((n * 12,), -1, dtype=torch.int64, device="cuda")
        assert lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n, 128, d_num.data_ptr(),
                                       d_xf.data_ptr(), _gpu.stream()) == 0
        _gpu.sync()
        assert np.array_equal(_gpu.to_host(d_num, np.uint32), want_num)
        assert np.array_equal(_gpu.to_host(d_xf, np.uint64).reshape(n, 4, 3), want_xf)
        st = read_state(d_state)
        assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)


def test_chained_batches_carry_state(lib, oracle, gpu):
    sizes = synthetic.stripe_sizes(77, 30000)
    want_num, want_xf, ost = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (1, 2))
    d_state = dev_state(4, 131072, 64, (1, 2))
    cuts = [0, 1, 1000, 1001, 9999, 20480, 30000]
    for a, b in zip(cuts[:-1], cuts[1:]):
        rc, num, xf = gpu_batch(lib, d_state, sizes[a:b])
        assert rc == 0
        assert np.array_equal(num, want_num[a:b]) and np.array_equal(xf, want_xf[a:b])
    st = read_state(d_state)
    assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)


def test_extreme_sizes(lib, oracle, gpu):
    sizes = np.array([0, 1, 63, 64, (1 << 63) - 1, 1 << 63, (1 << 64) - 129, (1 << 64) - 1,
                      131072, 131073, 393216, 393217], dtype=np.uint64)
    want_num, want_xf, _ = _oracle.sched_batch(oracle, sizes)
    rc, num, xf = gpu_batch(lib, dev_state(4, 131072, 64, (0, 0)), sizes)
    assert rc == 0 and np.array_equal(num, want_num) and np.array_equal(xf, want_xf)


def test_non_power_of_two_alignment(lib, oracle, gpu):
    sizes = synthetic.stripe_sizes(5, 5000)
    want_num, want_xf, _ = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (0, 0), align=96)
    rc, num, xf = gpu_batch(lib, dev_state(4, 131072, 64, (0, 0)), sizes, align=96)
    assert rc == 0 and np.array_equal(num, want_num) and np.array_equal(xf, want_xf)


def test_bad_arguments(lib, gpu):
    d_state = dev_state(4, 131072, 64, (0, 0))
    rc, _, _ = gpu_batch(lib, d_state, np.zeros(0, np.uint64))
    assert rc == 0                                              # empty batch
    assert lib.ofi_amd_sched_batch(d_state.data_ptr(), None, 5, 128, None, None, None) < 0
    assert lib.ofi_amd_sched_batch(d_state.data_ptr(), 1, 5, 0, 1, 1, None) < 0      # align 0
    assert lib.ofi_amd_sched_batch(d_state.data_ptr(), 1, (1 << 28) + 1, 128, 1, 1, None) < 0
    # unusable state on the device: the batch is left unwritten and the error word says why
    for rails, min_stripe in [(5, 131072), (0, 131072), (4, 0)]:
        bad = dev_state(rails, min_stripe, 64, (0, 0))
        rc, num, xf = gpu_batch(lib, bad, np.arange(10, dtype=np.uint64))
        assert rc == 0
        assert np.all(num == 0xFFFFFFFF) and np.all(xf == np.uint64(0xFFFFFFFFFFFFFFFF))
        assert _gpu.fetch_async_errors(lib) & 4


@pytest.mark.parametrize("rails,seeds", [(4, (3, 2)), (3, (1, 2))])
def test_batches_beyond_the_inline_prefix_limit(lib, oracle, gpu, rails, seeds):
    """Batches up to 2^21 messages use 512-message tiles, larger ones 1024-message tiles; beyond 4096
    tiles the tile seeds come from the separate scan launch.  One message below and one above each
    boundary must chain exactly like the small form."""
    # ... and 9 << 19, from where the XCDs take runs of 16 tiles instead of single tiles in turn
    for n in ((1 << 21), (1 << 21) + 1, 4096 * 1024, 4096 * 1024 + 1, (9 << 19) - 1, 9 << 19, (9 << 19) + 16 * 1024 * 8 + 5,
              4096 * 2048 + 1, 9_000_011):
        sizes = synthetic.stripe_sizes(n + rails, n)
        want_num, want_xf, ost = _oracle.sched_batch(oracle, sizes, rails, 131072, 64, seeds)
        d_state = dev_state(rails, 131072, 64, seeds)
        rc, num, xf = gpu_batch(lib, d_state, sizes)
        assert rc == 0
        assert np.array_equal(num, want_num)
        assert np.array_equal(xf, want_xf)
        st = read_state(d_state)
        assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)


def test_full_size_configuration(lib, oracle, gpu):
    """1,000,000 messages log-uniform in [1 B, 256 MiB), 4 rails, default thresholds, seeded start rails."""
    sizes = synthetic.stripe_sizes(2024, 1_000_000)
    assert sizes.min() >= 1 and sizes.max() < (1 << 28)
    want_num, want_xf, ost = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (1, 3))
    d_state = dev_state(4, 131072, 64, (1, 3))
    rc, num, xf = gpu_batch(lib, d_state, sizes)
    assert rc == 0
    assert np.array_equal(num, want_num)
    assert np.array_equal(xf, want_xf)
    st = read_state(d_state)
    assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)
    # invariants that hold at any size
    assert np.array_equal(xf[:, :, 2].sum(axis=1), sizes)
    assert set(np.unique(num)) <= {1, 2, 4}


def test_largest_batch_against_a_prefix_sum_in_torch(lib, gpu):
    """2^28 messages, the most one call takes (131,072 tiles, 29 GB of output): too large for the
    scalar oracle's output to be held and compared, so the batch formulation is restated with
    torch on the device -- stripe counts from the thresholds, start rails from exclusive prefix
    sums of the two counters mod the rail count -- and every row is compared with it; lengths,
    offsets and padding through what holds at any size."""
    n, rails, seeds = 1 << 28, 4, (3, 2)
    gen = torch.Generator(device="cuda").manual_seed(17)
    octave = torch.randint(0, 28, (n,), generator=gen, device="cuda", dtype=torch.int64)
    d_sizes = torch.randint(0, 1 << 28, (n,), generator=gen, device="cuda", dtype=torch.int64) >> (28 - octave)
    del octave
    d_state = dev_state(rails, 131072, 64, seeds)
    d_num = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    d_xf = torch.full((n * 12,), -1, dtype=torch.int64, device="cuda")
    assert lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n, 128, d_num.data_ptr(),
                                   d_xf.data_ptr(), _gpu.stream()) == 0
    _gpu.sync()
    assert _gpu.fetch_async_errors(lib) == 0
    small = d_sizes < 64
    want = torch.clamp((d_sizes + 131071) >> 17, 1, 4)            # ceil(size / 128 KiB), 1..4
    want = torch.where(want == 3, torch.full_like(want, 2), want)  # 3 does not divide 4 rails
    want = torch.where(small, torch.ones_like(want), want)
    assert torch.equal(d_num.to(torch.int64), want)
    big_steps = torch.where(small, torch.zeros_like(want), want)
    first_rail = torch.where(small,
                             (seeds[0] + torch.cumsum(small.to(torch.int64), 0) - small.to(torch.int64)) % rails,
                             (seeds[1] + torch.cumsum(big_steps, 0) - big_steps) % rails)
    rows = d_xf.view(n, 4, 3)
    for k in range(4):
        used = want > k
        assert torch.equal(rows[:, k, 0], torch.where(used, (first_rail + k) % rails, torch.zeros_like(want)))
        if k == 0:
            assert int(rows[:, 0, 1].abs().max()) == 0          # the first stripe starts at 0
        else:
            # a used stripe starts where the one before it ends; unused entries are all zero
            assert torch.equal(rows[:, k, 1], torch.where(used, rows[:, k - 1, 1] + rows[:, k - 1, 2],
                                                           torch.zeros_like(want)))
            assert int(rows[:, k, 2][~used].abs().max()) == 0
        del used
    assert torch.equal(rows[:, :, 2].sum(dim=1), d_sizes)
    # every stripe but a message's last is a multiple of the alignment
    for k in range(3):
        not_last = want > k + 1
        assert int((rows[:, k, 2][not_last] % 128).max()) == 0
    st = read_state(d_state)
    assert st.rr_small_counter == (seeds[0] + int(small.sum())) % rails
    assert st.rr_counter == (seeds[1] + int(big_steps.sum())) % rails
    # one more than the most: refused, nothing launched
    assert lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n + 1, 128, d_num.data_ptr(),
                                   d_xf.data_ptr(), _gpu.stream()) == -22


def test_batches_on_two_streams_do_not_share_scratch(lib, oracle, gpu):
    """Two scheduler instances driven from two streams at once (two endpoints in one process):
    each stream has its own tile scratch, so overlapping launches cannot mix their seeds."""
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    cases = []
    for k, (rails, seeds, n) in enumerate([(4, (1, 2), 700_001), (3, (2, 0), 650_003)]):
        sizes = synthetic.stripe_sizes(900 + k, n)
        want = _oracle.sched_batch(oracle, sizes, rails, 131072, 64, seeds)
        cases.append((sizes, want, dev_state(rails, 131072, 64, seeds), _gpu.to_dev(sizes),
                      torch.full((n,), -1, dtype=torch.int32, device="cuda"),
                      torch.full((n * 12,), -1, dtype=torch.int64, device="cuda")))
    torch.cuda.synchronize()
    for s, (sizes, _w, d_state, d_sizes, d_num, d_xf) in zip(streams, cases):
        assert lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), len(sizes), 128,
                                       d_num.data_ptr(), d_xf.data_ptr(),
                                       ctypes.c_void_p(s.cuda_stream)) == 0
    torch.cuda.synchronize()
    for sizes, (want_num, want_xf, ost), d_state, _d, d_num, d_xf in cases:
        n = len(sizes)
        assert np.array_equal(_gpu.to_host(d_num, np.uint32), want_num)
        assert np.array_equal(_gpu.to_host(d_xf, np.uint64).reshape(n, 4, 3), want_xf)
        st = read_state(d_state)
        assert (st.rr_small_counter, st.rr_counter) == (ost.rr_small_counter, ost.rr_counter)


def test_stream_scratch_is_handed_back_and_made_again(lib, oracle, gpu):
    """ofi_amd_sched_stream_release: the per-stream scratch goes back to the device (the runtime's
    count of free memory does not fall over many streams used once each), a stream nothing was
    allocated for is fine, and a released stream can be used again with the same results."""
    n = 300_001
    sizes = synthetic.stripe_sizes(77, n)
    want_num, want_xf, _ = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (0, 0))
    d_sizes = _gpu.to_dev(sizes)
    d_num = torch.zeros(n, dtype=torch.int32, device="cuda")
    d_xf = torch.zeros(n * 12, dtype=torch.int64, device="cuda")

    def once(stream):
        d_state = dev_state(4, 131072, 64, (0, 0))
        assert lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n, 128, d_num.data_ptr(),
                                       d_xf.data_ptr(), ctypes.c_void_p(stream.cuda_stream)) == 0

    s = torch.cuda.Stream()
    once(s)
    assert lib.ofi_amd_sched_stream_release(ctypes.c_void_p(s.cuda_stream)) == 0     # waits for the launches
    assert np.array_equal(_gpu.to_host(d_num, np.uint32), want_num)
    assert lib.ofi_amd_sched_stream_release(ctypes.c_void_p(s.cuda_stream)) == 0     # nothing left: fine
    d_num.zero_()
    once(s)                                                                          # allocated afresh
    torch.cuda.synchronize()
    assert np.array_equal(_gpu.to_host(d_num, np.uint32), want_num)
    assert np.array_equal(_gpu.to_host(d_xf, np.uint64).reshape(n, 4, 3), want_xf)
    assert lib.ofi_amd_sched_stream_release(ctypes.c_void_p(s.cuda_stream)) == 0
    # torch hands out streams from a pool of 32: a first round makes them all (a stream's queue takes
    # device memory of its own), the second round must then leave the count of free memory alone
    free_before = None
    for rnd in range(2):
        for _ in range(64):
            t = torch.cuda.Stream()
            once(t)
            assert lib.ofi_amd_sched_stream_release(ctypes.c_void_p(t.cuda_stream)) == 0
        torch.cuda.synchronize()
        if rnd == 0:
            free_before, _ = torch.cuda.mem_get_info()
    assert torch.cuda.mem_get_info()[0] == free_before
