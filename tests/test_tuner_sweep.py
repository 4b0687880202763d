"""Decision-edge sweep (counterpart of the reference's show-tuner-decisions tool): the
batched, level-by-level bisection must return exactly the edge lists of the reference's
recursive bisection (contrib/python/ofi_nccl/tuner/cli/wrapper.py:186-204) driven one
question at a time.  CPU tests use the oracle as the decision function; the GPU test checks
the product's batched query against it on the same questions."""
import ctypes
import io
import math

import pytest

from aws_ofi_nccl_amd import tuner_sweep as ts


def oracle_backend(oracle):
    calls = {"n": 0, "batches": 0}

    def backend(questions):
        calls["batches"] += 1
        out = []
        for plat, coll, nbytes, nranks, nnodes in questions:
            calls["n"] += 1
            a, p, ch = ctypes.c_int(-1), ctypes.c_int(-1), ctypes.c_int(-1)
            oracle.oracle_region_decide_masked(plat, coll, nbytes, nranks, nnodes, (1 << 21) - 1,
                                               ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
            out.append((a.value, p.value, ch.value))
        return out
    return backend, calls


def recursive_reference(tuner, coll_type, min_size, max_size):
    """The reference's bisect, literally, over single get_coll_info calls."""
    def bisect(lo, hi):
        lo_d, hi_d = tuner.get_coll_info(coll_type, lo), tuner.get_coll_info(coll_type, hi)
        if (lo_d == hi_d and math.log2(hi) - math.log2(lo) <= 1) or hi - lo <= 1:
            return [(lo, lo_d), (hi, hi_d)]
        mid = (lo + hi) // 2
        left, right = bisect(lo, mid), bisect(mid, hi)
        combined = left + right[1:]
        return [combined[0]] + [combined[i] for i in range(1, len(combined))
                                if combined[i][1] != combined[i - 1][1]]
    return bisect(min_size, max_size)


@pytest.mark.parametrize("platform,nranks,nnodes", [
    (ts.TunerPlatform.P5en, 64, 8), (ts.TunerPlatform.P5, 32, 16), (ts.TunerPlatform.P5, 128, 16),
    (ts.TunerPlatform.P6, 16, 16), (ts.TunerPlatform.P6_B300, 256, 32), (ts.TunerPlatform.P5en, 24, 8),
    (ts.TunerPlatform.P5en, 8, 2)])
def test_batched_rounds_give_the_recursive_edges(oracle, platform, nranks, nnodes):
    backend, calls = oracle_backend(oracle)
    batched = ts.Tuner(nranks, nnodes, platform, backend)
    sweep = ts.Sweep([batched], backend)
    rows = sweep.run()
    single = ts.Tuner(nranks, nnodes, platform, backend)
    want = []
    for coll in ts.NCCLFunc:
        want += single._rows(coll, recursive_reference(single, coll, 32, 32 << 30))
    strip = lambda rs: [tuple(str(r[k]) for k in ("collective", "message_size", "algo", "proto",
                                                   "nchannels", "ranks", "nodes")) for r in rs]
    assert strip(rows) == strip(want)
    assert sweep.rounds <= 40                       # one batch per bisection level, not per question
    assert sweep.questions == len(single._cache)    # and not a question more than the recursion asks


def test_edges_are_real_changes_and_bracket_them(oracle):
    backend, _ = oracle_backend(oracle)
    t = ts.Tuner(64, 8, ts.TunerPlatform.P5en, backend)
    rows = [r for r in t.analyze_message_range(ts.NCCLFunc.AllReduce, 32, 32 << 30)]
    sizes = [r["message_size"] for r in rows]
    assert sizes == sorted(sizes) and sizes[0] == 32 and sizes[-1] <= 32 << 30
    decisions = [(r["algo"], r["proto"], r["nchannels"]) for r in rows]
    assert len(set(decisions)) >= 3                 # P5en AllReduce at 8 ranks/node has several regions
    # the list holds the first point and then only points where the answer changes ...
    assert all(a != b for a, b in zip(decisions, decisions[1:]))
    # ... and each change is bracketed to one byte: the size just below still has the old answer
    for (size, new), old in zip(zip(sizes[1:], decisions[1:]), decisions):
        d = t.get_coll_info(ts.NCCLFunc.AllReduce, size - 1)
        assert (d["algo"], d["proto"], d["nchannels"]) == old != new
    # unsupported collectives have no decision anywhere: one row, the start of the range
    rows = t.analyze_message_range(ts.NCCLFunc.Broadcast, 32, 32 << 30)
    assert [r["message_size"] for r in rows] == [32]
    assert all(isinstance(r["algo"], float) and math.isnan(r["algo"]) for r in rows)


def test_show_all_prints_tables(oracle):
    backend, calls = oracle_backend(oracle)
    buf = io.StringIO()
    rows = ts.show_all(min_ranks_per_node=8, max_ranks_per_node=8, min_nnodes=4, max_nnodes=8, inc_nnodes=4,
                       show_channels=True, backend=backend, out=buf)
    text = buf.getvalue()
    assert {r["collective"] for r in rows} == {"AllReduce", "AllGather", "ReduceScatter"}
    assert "Ring" in text and "Simple" in text and "P5en" in text and "P6_B300" in text
    assert calls["batches"] <= 45 and calls["n"] > 1000


@pytest.mark.gpu
def test_gpu_backend_answers_like_the_oracle(lib, oracle, gpu):
    backend, _ = oracle_backend(oracle)
    tuners_gpu = [ts.Tuner(8 * n, n, p) for p in ts.TunerPlatform for n in (4, 16)]
    tuners_cpu = [ts.Tuner(8 * n, n, p, backend) for p in ts.TunerPlatform for n in (4, 16)]
    got = ts.Sweep(tuners_gpu).run()
    want = ts.Sweep(tuners_cpu, backend).run()
    assert [tuple(map(str, r.values())) for r in got] == [tuple(map(str, r.values())) for r in want]
    assert len(got) > 100
