"""Pins the scheduler oracle: the reference's own known answers
(tests/unit/scheduler.cpp:126-309), an independent arbitrary-precision model of the batch
formulation, and the invariants the algorithm guarantees."""
import ctypes
import json
import os

import numpy as np
import pytest

import _oracle
from aws_ofi_nccl_amd import synthetic

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "scheduler_kat.json")


def rows(num, xf):
    """(num_xfers, xfers words) -> list of [(rail, offset, len), ...] per message."""
    out = []
    for i in range(len(num)):
        out.append([(int(xf[i, k, 0]) & 0xFFFF, int(xf[i, k, 1]), int(xf[i, k, 2]))
                    for k in range(int(num[i]))])
    return out


def model_schedule(sizes, rails, min_stripe, max_small, seeds, align=128):
    """Independent restatement as two prefix sums with Python integers (no wrap-around),
    written from the closed form, not from the oracle's loop."""
    out = []
    small_before, stripes_before = 0, 0
    for s in (int(x) for x in sizes):
        if s < max_small:
            out.append([((seeds[0] + small_before) % rails, 0, s)])
            small_before += 1
            continue
        want = -(-s // min_stripe)
        n = max(1, min(want, rails))
        # largest divisor of `rails` in [2, n]; when there is none the count stays as it is
        # (src/nccl_ofi_scheduler.cpp:57-62 -- e.g. 3 rails, 2 wanted stripes -> 2, not 1)
        n = next((i for i in range(n, 1, -1) if rails % i == 0), n)
        per = -(-s // n)
        stripe = -(-per // align) * align
        start = (seeds[1] + stripes_before) % rails
        stripes_before += n
        trip = []
        for k in range(n):
            off = min(k * stripe, s)
            trip.append(((start + k) % rails, off, min(stripe, s - off)))
        out.append(trip)
    return out, (seeds[0] + small_before) % rails, (seeds[1] + stripes_before) % rails


def test_reference_known_answers(oracle):
    doc = json.load(open(GOLDEN))
    sizes = np.array([c["size"] for c in doc["calls"]], dtype=np.uint64)
    num, xf, _ = _oracle.sched_batch(oracle, sizes, doc["num_rails"], doc["min_stripe_size"],
                                     doc["max_small_msg_size"], (0, 0), doc["align"])
    got = rows(num, xf)
    for call, g in zip(doc["calls"], got):
        assert g == [tuple(t) for t in call["stripes"]], call["size"]


def test_single_call_api_matches_batch(oracle):
    sizes = synthetic.stripe_sizes(7, 5000)
    num, xf, _ = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (2, 1))
    st = _oracle.Sched(2, 1, 64, 131072, 4, 0)
    x = (_oracle.Xfer * 4)()
    for i, s in enumerate(sizes):
        n = oracle.oracle_sched_get_schedule(ctypes.byref(st), int(s), 128, x)
        assert n == num[i]
        for k in range(n):
            assert (x[k].rail_id, x[k].offset, x[k].msg_size) == (
                int(xf[i, k, 0]) & 0xFFFF, int(xf[i, k, 1]), int(xf[i, k, 2]))


@pytest.mark.parametrize("rails", [1, 2, 3, 4])
@pytest.mark.parametrize("min_stripe,max_small", [(4096, 64), (131072, 64), (1000, 10), (1, 0)])
def test_against_independent_model(oracle, rails, min_stripe, max_small):
    rng = np.random.default_rng(rails * 1000 + min_stripe)
    sizes = np.concatenate([
        synthetic.stripe_sizes(rails + min_stripe, 3000),
        rng.integers(0, 200, 500).astype(np.uint64),            # around the small threshold
        (rng.integers(0, 6, 500) * min_stripe + rng.integers(-2, 3, 500)).clip(0).astype(np.uint64),
    ])
    rng.shuffle(sizes)
    seeds = (int(rng.integers(0, rails)), int(rng.integers(0, rails)))
    num, xf, st = _oracle.sched_batch(oracle, sizes, rails, min_stripe, max_small, seeds)
    want, small_end, big_end = model_schedule(sizes, rails, min_stripe, max_small, seeds)
    assert rows(num, xf) == want
    assert (st.rr_small_counter, st.rr_counter) == (small_end, big_end)


def test_invariants_default_thresholds(oracle):
    sizes = synthetic.stripe_sizes(3, 200000)
    num, xf, _ = _oracle.sched_batch(oracle, sizes)
    lens = xf[:, :, 2]
    offs = xf[:, :, 1]
    rails = xf[:, :, 0] & np.uint64(0xFFFF)
    assert np.array_equal(lens.sum(axis=1), sizes)                      # sum of stripes = size
    assert set(np.unique(num)) <= {1, 2, 4}                             # divisors of 4 rails
    for k in range(1, 4):
        live = num > k
        assert np.array_equal(offs[live, k], offs[live, k - 1] + lens[live, k - 1])   # contiguous
        assert np.all(lens[live, k - 1] % 128 == 0)                     # all but last are 128-aligned
        assert np.array_equal(rails[live, k], (rails[live, k - 1] + 1) % 4)   # consecutive rails
        dead = ~live
        assert not xf[dead, k, :].any()                                 # unused entries zero
    assert np.all(offs[:, 0] == 0)
    # stripe counts by size class: < 64 B small, <= 128 KiB one, <= 384 KiB two, else four
    big = sizes >= 64
    assert np.all(num[(sizes <= 131072)] == 1)
    assert np.all(num[(sizes > 131072) & (sizes <= 3 * 131072)] == 2)
    assert np.all(num[sizes > 3 * 131072] == 4)
    assert big.any() and (~big).any()


def test_two_independent_counters(oracle):
    # small and large messages interleaved advance different counters
    sizes = np.array([10, 100, 20, 200, 30, 300, 1 << 20, 40], dtype=np.uint64)
    num, xf, st = _oracle.sched_batch(oracle, sizes, 4, 131072, 64, (0, 0))
    got = rows(num, xf)
    assert [g[0][0] for g in got] == [0, 0, 1, 1, 2, 2, 3, 3]
    assert len(got[6]) == 4 and [t[0] for t in got[6]] == [3, 0, 1, 2]
    assert (st.rr_small_counter, st.rr_counter) == (0, 3)


def test_extreme_sizes_wrap_like_the_reference(oracle):
    # size near 2^64: DIV_CEIL avoids overflow (include/nccl_ofi_math.h:23-26); the
    # round-up to the alignment wraps in 64 bits exactly as size_t does in the reference
    for size in [(1 << 63) - 1, 1 << 63, (1 << 64) - 129, (1 << 64) - 1]:
        sizes = np.array([size], dtype=np.uint64)
        num, xf, _ = _oracle.sched_batch(oracle, sizes)
        n = 4
        per = -(-size // n)
        stripe = (-(-per // 128) * 128) & ((1 << 64) - 1)
        left, off, want = size, 0, []
        for k in range(n):
            s = min(left, stripe)
            want.append((k % 4, off, s))
            off = (off + s) & ((1 << 64) - 1)
            left -= s
        assert rows(num, xf)[0] == want


def test_math_helpers_against_reference_header(oracle, ref):
    # NCCL_OFI_DIV_CEIL / ROUND_UP compiled from the reference header
    rng = np.random.default_rng(5)
    for x, y in zip(rng.integers(0, 1 << 62, 2000), rng.integers(1, 1 << 20, 2000)):
        x, y = int(x), int(y)
        assert ref.ref_div_ceil(x, y) == (0 if x == 0 else 1 + (x - 1) // y)
    assert ref.ref_div_ceil(0, 7) == 0
    assert ref.ref_round_up(129, 128) == 256 and ref.ref_round_down(255, 128) == 128
    # num_stripes of the oracle equals the header's DIV_CEIL-based definition
    st = _oracle.Sched(0, 0, 64, 131072, 4, 0)
    for s in [0, 1, 131072, 131073, 262144, 262145, 393216, 393217, 1 << 30]:
        want = max(1, min(ref.ref_div_ceil(s, 131072), 4))
        while want > 1 and 4 % want:
            want -= 1
        assert oracle.oracle_sched_num_stripes(ctypes.byref(st), s) == want
