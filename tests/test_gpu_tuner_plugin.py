"""GPU parity of the per-collective tuner entry points: the point-query C ABI and the NCCL plugin
structs (v2 / v3 / v6) against the CPU oracle's restatement of region_get_coll_info_internal_v3/_v2,
model_get_coll_info_internal_v3/_v2 and region_get_chunk_size_internal."""
import ctypes
import os

import numpy as np
import pytest

import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

PLATFORM_NAMES = ["p5.48xlarge", "p5en.48xlarge", "p6-b200.48xlarge", "p6-b300.48xlarge"]
ENV_KEYS = ["OFI_NCCL_FORCE_PRODUCT_NAME", "OFI_NCCL_TUNER_TYPE", "OFI_NCCL_FORCE_NUM_RAILS", "NCCL_ALGO",
            "NCCL_PROTO", "OFI_NCCL_TUNER_NUM_CHANNELS", "OFI_NCCL_TUNER_NET_COMP_OVERHEAD"]
ALL = 0x1FFFFF


@pytest.fixture
def clean_env():
    saved = {k: os.environ.pop(k, None) for k in ENV_KEYS}
    yield
    for k, v in saved.items():
        os.environ.pop(k, None)
        if v is not None:
            os.environ[k] = v


def sizes_for_test(rng, n):
    anchors = [196608, 13107200, 31457280, 3145728, 32768, 131072, 8388608, 4 << 20, 32 << 20, 8 * 65536,
               3 << 30, 5 << 30, 107374182400]
    out = [0, 1] + [a + d for a in anchors for d in (-1, 0, 1)]
    out += [int(2 ** rng.uniform(0, 37)) for _ in range(n)]
    return out


def test_query_batch_matches_oracle(lib, oracle, gpu):
    rng = np.random.default_rng(11)
    qs, want = [], []
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    out = ctypes.c_uint64()
    for size in sizes_for_test(rng, 600):
        plat = int(rng.integers(0, 4))
        coll = int(rng.choice([4, 2, 3, 0]))
        N = int(rng.choice([1, 2, 4, 8, 8, 16, 16, 17, 64, 128, 1024]))
        R = N * int(rng.choice([1, 1, 2, 8, 8])) if rng.random() < 0.95 else N * 8 + 1
        mask = ALL if rng.random() < 0.7 else int(rng.integers(0, ALL + 1))
        kind = int(rng.integers(0, 3))
        pipe = int(rng.integers(1, 5))
        algo, proto = int(rng.choice([0, 6, 1])), int(rng.choice([1, 2, 0]))
        qs.append(m.TunerQuery(plat, kind, coll, pipe, 8, 3, algo, proto, mask, 0, size, R, N))
        if kind == 0:
            ch.value = -1
            oracle.oracle_region_decide_masked(plat, coll, size, R, N, mask, ctypes.byref(a), ctypes.byref(p),
                                               ctypes.byref(ch))
            want.append((a.value, p.value, ch.value, 0))
        elif kind == 1:
            if plat < 2:
                oracle.oracle_model_decide_v2(plat, coll, pipe, size, R, N, 8, 3, (mask >> 17) & 1,
                                              ctypes.byref(a), ctypes.byref(p))
                want.append((a.value, p.value, -1, 0))
            else:
                want.append((-1, -1, -1, 0))
        else:
            out.value = 0
            got = oracle.oracle_region_chunk_size(plat, coll, size, algo, proto, R, N, ctypes.byref(out))
            want.append((-1, -1, -1, out.value if got else 0))
    n = len(qs)
    arr = (m.TunerQuery * n)(*qs)
    ans = (m.TunerAnswer * n)()
    assert lib.ofi_amd_tuner_query(arr, n, ans) == 0
    got = [(x.algo, x.proto, x.nchannels, x.chunk_size) for x in ans]
    bad = [i for i in range(n) if got[i] != want[i]]
    assert not bad, [(i, got[i], want[i]) for i in bad[:5]]
    assert sum(1 for w in want if w[0] >= 0) > 60 and sum(1 for w in want if w[3] > 0) >= 3
    # argument checking
    bad_q = (m.TunerQuery * 1)(m.TunerQuery(9, 0, 4, 1, 8, 3, 0, 0, ALL, 0, 1, 8, 8))
    assert lib.ofi_amd_tuner_query(bad_q, 1, ans) < 0
    assert lib.ofi_amd_tuner_query(None, 0, None) == 0


@pytest.mark.parametrize("plat", [0, 1, 2, 3])
@pytest.mark.parametrize("ranks,nodes", [(64, 8), (16, 16), (32, 16), (1024, 128), (16, 2)])
def test_plugin_v3_region(lib, oracle, gpu, clean_env, plat, ranks, nodes):
    os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = PLATFORM_NAMES[plat]
    v3 = m.NcclTunerV3.in_dll(lib, "ncclTunerPlugin_v3")
    ctx = ctypes.c_void_p()
    assert v3.init(ranks, nodes, None, ctypes.byref(ctx)) == 0 and ctx.value
    rng = np.random.default_rng(plat * 100 + ranks)
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    decided = 0
    for size in sizes_for_test(rng, 120):
        for coll in (4, 2, 3):
            table = np.full((7, 3), 1337.0, dtype=np.float32)    # as the reference's Python sweep does
            ignore = rng.random((7, 3)) < 0.15
            table[ignore] = -1.0
            num_algo = int(rng.choice([7, 7, 6]))
            mask = 0
            for x in range(num_algo):
                for y in range(3):
                    if not ignore[x, y]:
                        mask |= 1 << (x * 3 + y)
            before = table.copy()
            nch = ctypes.c_int(-5)
            assert v3.getCollInfo(ctx, coll, size, 1, table.ctypes.data, num_algo, 3, ctypes.byref(nch)) == 0
            ch.value = -5
            oracle.oracle_region_decide_masked(plat, coll, size, ranks, nodes, mask, ctypes.byref(a),
                                               ctypes.byref(p), ctypes.byref(ch))
            want = before.copy()
            if a.value >= 0:
                want[a.value, p.value] = 0.0
                decided += 1
            assert np.array_equal(table, want), (size, coll)
            assert nch.value == ch.value
            # asking again (now from the plugin's table of answers) gives the same
            table2 = before.copy()
            v3.getCollInfo(ctx, coll, size, 1, table2.ctypes.data, num_algo, 3, ctypes.byref(nch))
            assert np.array_equal(table2, want)
    if nodes > 2 and (ranks == 8 * nodes or ranks == nodes or (plat == 0 and ranks == 2 * nodes)):
        assert decided > 50
    else:
        assert decided == 0
    assert v3.destroy(ctx) == 0


def test_plugin_v3_model_type(lib, oracle, gpu, clean_env):
    os.environ["OFI_NCCL_TUNER_TYPE"] = "Model"
    os.environ["OFI_NCCL_TUNER_NUM_CHANNELS"] = "16"
    os.environ["OFI_NCCL_TUNER_NET_COMP_OVERHEAD"] = "5"
    v3 = m.NcclTunerV3.in_dll(lib, "ncclTunerPlugin_v3")
    a, p = ctypes.c_int(), ctypes.c_int()
    rng = np.random.default_rng(3)
    for plat, ranks, nodes in [(0, 128, 16), (1, 64, 8), (0, 16, 16), (1, 8, 2)]:
        os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = PLATFORM_NAMES[plat]
        ctx = ctypes.c_void_p()
        assert v3.init(ranks, nodes, None, ctypes.byref(ctx)) == 0 and ctx.value
        for size in sizes_for_test(rng, 60):
            for coll, pipe in ((4, 1), (4, 3), (2, 1)):
                table = np.full((7, 3), 1337.0, dtype=np.float32)
                table[1, 2] = -1.0                      # the model tuner ignores NCCL's marks
                nch = ctypes.c_int(-5)
                assert v3.getCollInfo(ctx, coll, size, pipe, table.ctypes.data, 7, 3, ctypes.byref(nch)) == 0
                oracle.oracle_model_decide(plat, coll, pipe, size, ranks, nodes, 16, 5, ctypes.byref(a),
                                           ctypes.byref(p))
                want = np.full((7, 3), 1337.0, dtype=np.float32)
                want[1, 2] = -1.0
                if a.value >= 0:
                    want[a.value, p.value] = 0.0
                assert np.array_equal(table, want), (plat, size, coll, pipe)
                assert nch.value == -5
        v3.destroy(ctx)
    # a platform without a model keeps the region tuner even when Model is forced (:102-107)
    os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = PLATFORM_NAMES[2]
    ctx = ctypes.c_void_p()
    assert v3.init(64, 8, None, ctypes.byref(ctx)) == 0 and ctx.value
    table = np.full((7, 3), 1337.0, dtype=np.float32)
    nch = ctypes.c_int(-5)
    v3.getCollInfo(ctx, 4, 1024, 1, table.ctypes.data, 7, 3, ctypes.byref(nch))
    ch = ctypes.c_int(-5)
    oracle.oracle_region_decide(2, 4, 1024, 64, 8, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
    assert a.value >= 0 and table[a.value, p.value] == 0.0
    v3.destroy(ctx)


def test_plugin_v2(lib, oracle, gpu, clean_env):
    v2 = m.NcclTunerV2.in_dll(lib, "ncclTunerPlugin_v2")
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    rng = np.random.default_rng(8)
    pat_cases = 0
    for plat, ranks, nodes, model in [(1, 64, 8, 0), (2, 8, 8, 0), (3, 64, 64, 0), (0, 128, 16, 1)]:
        os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = PLATFORM_NAMES[plat]
        os.environ["OFI_NCCL_TUNER_TYPE"] = "Model" if model else "Region"
        ctx = ctypes.c_void_p()
        assert v2.init(ranks, nodes, None, ctypes.byref(ctx)) == 0 and ctx.value
        for size in sizes_for_test(rng, 80):
            for coll in (4, 2, 3):
                for nvls in (0, 1):
                    ga, gp, gn = ctypes.c_int(-9), ctypes.c_int(-9), ctypes.c_int(-9)
                    assert v2.getCollInfo(ctx, coll, size, 0, nvls, 1, ctypes.byref(ga), ctypes.byref(gp),
                                          ctypes.byref(gn)) == 0
                    if model:
                        oracle.oracle_model_decide_v2(plat, coll, 1, size, ranks, nodes, 8, 3, nvls,
                                                      ctypes.byref(a), ctypes.byref(p))
                    else:
                        mask = ALL & ~(7 << 18)
                        if not nvls:
                            mask &= ~(7 << 15)
                        oracle.oracle_region_decide_masked(plat, coll, size, ranks, nodes, mask,
                                                           ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
                        v3a, v3p = ctypes.c_int(), ctypes.c_int()
                        oracle.oracle_region_decide(plat, coll, size, ranks, nodes, ctypes.byref(v3a),
                                                    ctypes.byref(v3p), ctypes.byref(ch))
                        pat_cases += v3a.value == 6
                    want = (a.value, p.value) if a.value >= 0 else (-9, -9)
                    assert (ga.value, gp.value) == want, (plat, size, coll, nvls)
                    assert gn.value == -9                 # v2 never sets nChannels (:1995-2062)
        v2.destroy(ctx)
    assert pat_cases > 10        # sizes where v3 would say PAT were exercised


def test_plugin_v6_chunk_size(lib, oracle, gpu, clean_env):
    v6 = m.NcclTunerV6.in_dll(lib, "ncclTunerPlugin_v6")
    out = ctypes.c_uint64()
    rng = np.random.default_rng(5)
    hits = 0
    for plat, ranks, nodes in [(1, 8, 8), (1, 64, 64), (1, 64, 8), (0, 8, 8), (2, 16, 16)]:
        os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = PLATFORM_NAMES[plat]
        ctx = ctypes.c_void_p()
        assert v6.init(ctypes.byref(ctx), 0x1234, ranks, nodes, None, None, None) == 0 and ctx.value
        for size in sizes_for_test(rng, 60):
            for coll, algo, proto in [(4, 0, 1), (2, 6, 2), (4, 1, 2), (3, 6, 2)]:
                chunk = ctypes.c_size_t(777)
                assert v6.getChunkSize(ctx, coll, size, algo, proto, 8, ctypes.byref(chunk)) == 0
                out.value = 0
                if oracle.oracle_region_chunk_size(plat, coll, size, algo, proto, ranks, nodes, ctypes.byref(out)):
                    assert chunk.value == out.value
                    hits += 1
                else:
                    assert chunk.value == 777
        # v6 getCollInfo is v3 with one more argument
        table = np.full((7, 3), 1337.0, dtype=np.float32)
        nch = ctypes.c_int(-5)
        assert v6.getCollInfo(ctx, 4, 4096, 1, table.ctypes.data, 7, 3, 1, ctypes.byref(nch)) == 0
        assert v6.finalize(ctx) == 0
    assert hits > 100


def test_query_heuristic_breakpoints_by_hand(lib, gpu):
    """The hand-derived breakpoints of the nChannels and chunk-size ladders
    (tests/test_oracle_tuner_heuristics.py) asked of the GPU through the point-query C ABI:
    both sides of every breakpoint, no oracle in between."""
    import test_oracle_tuner_heuristics as h
    qs, want = [], []

    def ask(plat, kind, coll, size, ranks, nodes, algo, proto, expect):
        qs.append(m.TunerQuery(plat, kind, coll, 1, 8, 3, algo, proto, ALL, 0, size, ranks, nodes))
        want.append(expect)

    for nodes, log2_nodes in ((8, 3), (32, 5)):
        before = 32
        for cut, after in h.BEST_TREE[log2_nodes]:
            ask(h.P6, 0, h.AR, cut - 1, 8 * nodes, nodes, 0, 0, (h.TREE, h.LL128, before, 0))
            ask(h.P6, 0, h.AR, cut, 8 * nodes, nodes, 0, 0, (h.TREE, h.LL128, after, 0))
            before = after
    for size, ch in ((4 * h.MIB - 1, -1), (4 * h.MIB, 32), (32 * h.MIB, 32), (32 * h.MIB + 1, -1)):
        ask(h.P6, 0, h.AR, size, 64, 8, 0, 0, (h.TREE, h.LL128, ch, 0))
    for nodes in (8, 16, 64):
        for size, ch in ((nodes * 65536, 1), (nodes * 65536 + 1, 2), (nodes * 131072, 2), (nodes * 131072 + 1, 0)):
            ask(h.P6, 0, h.AG, size, nodes, nodes, 0, 0, (h.PAT, h.SIMPLE, ch, 0))
    ask(h.P6, 0, h.AG, 32 * h.MIB, 512, 512, 0, 0, (h.PAT, h.SIMPLE, 1, 0))
    ask(h.P6, 0, h.AG, 32 * h.MIB + 1, 512, 512, 0, 0, (h.PAT, h.SIMPLE, -1, 0))
    for table, coll, algo, proto, floor in ((h.PAT_LADDERS, h.AG, h.PAT, h.SIMPLE, 32768),
                                            (h.TREE_P5EN_LADDERS, h.AR, h.TREE, h.LL128, 18000)):
        for nodes, ladder in table.items():
            before = floor
            for cut, after in ladder:
                ask(h.P5EN, 2, coll, cut - 1, nodes, nodes, algo, proto, (-1, -1, -1, before))
                ask(h.P5EN, 2, coll, cut, nodes, nodes, algo, proto, (-1, -1, -1, after))
                before = after
    n = len(qs)
    ans = (m.TunerAnswer * n)()
    assert lib.ofi_amd_tuner_query((m.TunerQuery * n)(*qs), n, ans) == 0
    got = [(x.algo, x.proto, x.nchannels, x.chunk_size) for x in ans]
    bad = [i for i in range(n) if got[i] != want[i]]
    assert not bad, [(qs[i].nbytes, qs[i].num_nodes, got[i], want[i]) for i in bad[:5]]
    assert n >= 150


def test_init_evaluates_the_size_ladder_ahead(lib, oracle, gpu, clean_env):
    """init prepares everything that allocates and answers the power-of-two ladder of every
    collective in one launch: a job's first getCollInfo calls are table hits; a narrower cost table
    that still allows the chosen cell is a hit as well; an off-ladder size goes to the GPU once."""
    os.environ["OFI_NCCL_FORCE_PRODUCT_NAME"] = PLATFORM_NAMES[2]            # P6: regions for AR, AG, RS
    v3 = m.NcclTunerV3.in_dll(lib, "ncclTunerPlugin_v3")
    ctx = ctypes.c_void_p()
    assert v3.init(64, 8, None, ctypes.byref(ctx)) == 0 and ctx.value
    st = m.TunerCtxStats()
    assert lib.ofi_amd_tuner_ctx_stats(ctx, ctypes.byref(st)) == 0
    assert st.preloaded >= 5 * 37 and (st.hits, st.misses) == (0, 0)
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    nch = ctypes.c_int(-5)
    asked = 0
    for coll in (4, 2, 3):
        for e in range(0, 37):
            table = np.full((7, 3), 1337.0, dtype=np.float32)
            assert v3.getCollInfo(ctx, coll, 1 << e, 1, table.ctypes.data, 7, 3, ctypes.byref(nch)) == 0
            ch.value = -5
            oracle.oracle_region_decide(2, coll, 1 << e, 64, 8, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
            zero = [(int(i), int(j)) for i, j in zip(*np.where(table == 0.0))]
            assert zero == ([(a.value, p.value)] if a.value >= 0 else []), (coll, e)
            asked += 1
    assert lib.ofi_amd_tuner_ctx_stats(ctx, ctypes.byref(st)) == 0
    assert (st.hits, st.misses) == (asked, 0)
    # NCCL rules out a cell the answer does not use (NVLS): still the same first region -> a hit
    table = np.full((7, 3), 1337.0, dtype=np.float32)
    table[4, :] = -1.0
    oracle.oracle_region_decide(2, 4, 1 << 20, 64, 8, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
    assert a.value not in (-1, 4)
    assert v3.getCollInfo(ctx, 4, 1 << 20, 1, table.ctypes.data, 7, 3, ctypes.byref(nch)) == 0
    assert table[a.value, p.value] == 0.0
    # ... and one that rules out the chosen cell itself has to be asked
    table = np.full((7, 3), 1337.0, dtype=np.float32)
    table[a.value, p.value] = -1.0
    mask = 0x1FFFFF & ~(1 << (a.value * 3 + p.value))
    oracle.oracle_region_decide_masked(2, 4, 1 << 20, 64, 8, mask, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
    assert v3.getCollInfo(ctx, 4, 1 << 20, 1, table.ctypes.data, 7, 3, ctypes.byref(nch)) == 0
    if a.value >= 0:
        assert table[a.value, p.value] == 0.0
    # off the ladder: one round trip, then a hit
    for _ in range(2):
        table = np.full((7, 3), 1337.0, dtype=np.float32)
        assert v3.getCollInfo(ctx, 4, (1 << 20) + 3, 1, table.ctypes.data, 7, 3, ctypes.byref(nch)) == 0
    assert lib.ofi_amd_tuner_ctx_stats(ctx, ctypes.byref(st)) == 0
    assert (st.hits, st.misses) == (asked + 2, 2)
    assert v3.destroy(ctx) == 0
    assert lib.ofi_amd_tuner_ctx_stats(None, ctypes.byref(st)) == -22
