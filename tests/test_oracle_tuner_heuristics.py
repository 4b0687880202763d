"""Pins the oracle's nChannels / chunk-size heuristics (src/tuner/nccl_ofi_regions.cpp:1885-1971,
2135-2152, 2159-2306) by the message sizes at which each output changes.

Every expectation below is a literal worked out on paper from the reference's thresholds, not a
second evaluation of the same loops; both sides of every breakpoint are asserted.

calculateChunkSizeTreeLL128(m, C, L)  (:1885-1938)
    start: 120 * 640 * 8 * 8 / 8 = 614,400 B per step, * 15/16 (data words per LL128 line) = 576,000
    nSteps = 1 + L + 0.1 * 8 = L + 1.8
    loop 1 halves while floor(m / (C * chunk)) < nSteps * 64 / 8 = 8L + 14.4 and chunk > 131,072;
           an integer quotient is below 8L + 14.4 exactly when it is <= 8L + 14, so a chunk of
           576,000 / 288,000 / 144,000 survives iff m >= (8L + 15) * C * chunk; else 72,000 is reached
    loop 2 halves while floor(m / (C * chunk)) < nSteps * 16 / 8 = 2L + 3.6 and chunk > 32,768:
           72,000 / 36,000 survive iff m >= (2L + 4) * C * chunk; the floor is 18,000
    grain = 32 * 8 / 16 * 15 * 8 = 1,920 B; chunk rounds down to whole grains g = chunk // 1,920:
           576,000 -> 300, 288,000 -> 150, 144,000 -> 75, 72,000 -> 37, 36,000 -> 18, 18,000 -> 9
    wire size = ceil(g * 480 / 480) * 256 * 8 = g * 2,048:
           614,400 / 307,200 / 153,600 / 75,776 / 36,864 / 18,432
"""
import ctypes

import pytest

import _oracle  # noqa: F401  (fixture `oracle` comes from conftest)

AR, AG, RS = 4, 2, 3
TREE, RING, NVLS_TREE, PAT = 0, 1, 5, 6
LL, LL128, SIMPLE = 0, 1, 2
P5, P5EN, P6, P6_B300 = 0, 1, 2, 3
MIB = 1 << 20

WIRE = {576000: 614400, 288000: 307200, 144000: 153600, 72000: 75776, 36000: 36864, 18000: 18432}

# (nChannels, log2 nodes) -> thresholds from the formulas above, multiplied out by hand:
#   (16, 2): 8L+15 = 31, 2L+4 = 8:  8*16*36,000 = 4,608,000   8*16*72,000 = 9,216,000
#            31*16*144,000 = 71,424,000   31*16*288,000 = 142,848,000   31*16*576,000 = 285,696,000
#   (24, 3): 39 and 10:  10*24*36,000 = 8,640,000   10*24*72,000 = 17,280,000
#            39*24*144,000 = 134,784,000   269,568,000   539,136,000
#   (32, 0): 15 and 4:   4*32*36,000 = 4,608,000   4*32*72,000 = 9,216,000
#            15*32*144,000 = 69,120,000   138,240,000   276,480,000
#   (1, 10): 95 and 24:  24*36,000 = 864,000   24*72,000 = 1,728,000
#            95*144,000 = 13,680,000   27,360,000   54,720,000
TREE_LL128_LADDERS = {
    (16, 2): [4608000, 9216000, 71424000, 142848000, 285696000],
    (24, 3): [8640000, 17280000, 134784000, 269568000, 539136000],
    (32, 0): [4608000, 9216000, 69120000, 138240000, 276480000],
    (1, 10): [864000, 1728000, 13680000, 27360000, 54720000],
}
TREE_LL128_RUNGS = [18432, 36864, 75776, 153600, 307200, 614400]


@pytest.mark.parametrize("shape", sorted(TREE_LL128_LADDERS))
def test_chunk_size_tree_ll128_breakpoints(oracle, shape):
    channels, log2_nodes = shape
    f = lambda m: oracle.oracle_chunk_tree_ll128(m, channels, log2_nodes)
    cuts = TREE_LL128_LADDERS[shape]
    assert f(0) == 18432 and f(1) == 18432
    for k, cut in enumerate(cuts):
        assert f(cut - 1) == TREE_LL128_RUNGS[k], (shape, cut)
        assert f(cut) == TREE_LL128_RUNGS[k + 1], (shape, cut)
    assert f(cuts[-1] * 1000) == 614400


def test_chunk_size_tree_ll128_invariants(oracle):
    """Never decreases with the message size, always one of the six wire sizes reachable by
    halving (each a whole number of 2,048-byte slices), never grows with the channel count."""
    for log2_nodes in range(0, 12):
        for channels in (1, 8, 16, 24, 32):
            last = 0
            m = 1
            while m < 1 << 40:
                got = oracle.oracle_chunk_tree_ll128(m, channels, log2_nodes)
                assert got in TREE_LL128_RUNGS and got % 2048 == 0
                assert got >= last, (m, channels, log2_nodes)
                assert got <= oracle.oracle_chunk_tree_ll128(m, max(1, channels // 2), log2_nodes)
                last = got
                m = m * 5 // 4 + 1


# calculateBestNChannelTree (:1955-1971): channels 16, 24, 32 in turn, keep the larger payload, on
# equal payload the larger channel count.  The payload never grows with the channel count, so the
# answer is the largest of {16, 24, 32} whose payload still equals that of 16 channels.  With
# the thresholds (2L+4) * C * 36,000 and (2L+4) * C * 72,000 (the 144,000 rung starts far above
# the 32 MiB this function is used up to):
#   L = 2 (x8):  C=16: 4,608,000 / 9,216,000   C=24: 6,912,000 / 13,824,000   C=32: 9,216,000 / 18,432,000
#   L = 3 (x10): C=16: 5,760,000 / 11,520,000  C=24: 8,640,000 / 17,280,000   C=32: 11,520,000 / 23,040,000
#   L = 5 (x14): C=16: 8,064,000 / 16,128,000  C=24: 12,096,000 / 24,192,000  C=32: 16,128,000 / 32,256,000
# Between consecutive thresholds t (ascending) the payloads of (16, 24, 32) channels are:
#   below C16a: all 18,432 -> 32;  [C16a, C24a): 36,864 / 18,432 / 18,432 -> 16;
#   [C24a, C32a): 36,864 / 36,864 / 18,432 -> 24;  C32a == C16b: 75,776 / 36,864 / 36,864 -> 16;
#   [C24b, C32b): 75,776 / 75,776 / 36,864 -> 24;  from C32b: all 75,776 -> 32.
BEST_TREE = {
    2: [(4608000, 16), (6912000, 24), (9216000, 16), (13824000, 24), (18432000, 32)],
    3: [(5760000, 16), (8640000, 24), (11520000, 16), (17280000, 24), (23040000, 32)],
    5: [(8064000, 16), (12096000, 24), (16128000, 16), (24192000, 24), (32256000, 32)],
}


@pytest.mark.parametrize("log2_nodes", sorted(BEST_TREE))
def test_best_nchannel_tree_breakpoints(oracle, log2_nodes):
    f = lambda m: oracle.oracle_best_nchannel_tree(m, log2_nodes)
    before = 32                                   # all three payloads equal below the first threshold: tie -> 32
    assert f(4 * MIB) == 32
    for cut, after in BEST_TREE[log2_nodes]:
        assert f(cut - 1) == before, (log2_nodes, cut)
        assert f(cut) == after, (log2_nodes, cut)
        before = after
    assert f(32 * MIB) == 32


def test_best_nchannel_tree_through_the_region_decision(oracle):
    """region_get_coll_info_internal_v3 :2140-2145: P6 only, 4 MiB <= size <= 32 MiB, Tree/LL128,
    8 ranks per node.  The Tree/LL128 polygon of P6 at 8 ranks per node (:1000-1013) spans, at 64
    ranks, sizes from 393,216 to 40,370,176 and at 256 ranks to 72,876,032, so every point below is
    inside it; at 32 ranks it ends at the vertex (18,350,080, 32)."""
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()

    def decide(plat, size, ranks, nodes):
        ch.value = -1
        oracle.oracle_region_decide(plat, AR, size, ranks, nodes, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
        return a.value, p.value, ch.value

    for nodes, log2_nodes in ((8, 3), (32, 5)):
        before = 32
        for cut, after in BEST_TREE[log2_nodes]:
            assert decide(P6, cut - 1, 8 * nodes, nodes) == (TREE, LL128, before)
            assert decide(P6, cut, 8 * nodes, nodes) == (TREE, LL128, after)
            before = after
    for cut, after in BEST_TREE[2][:4]:           # 18,432,000 lies beyond the polygon at 32 ranks
        assert decide(P6, cut, 32, 4) == (TREE, LL128, after)
    # the size window is closed on both ends
    assert decide(P6, 4 * MIB - 1, 64, 8) == (TREE, LL128, -1)
    assert decide(P6, 4 * MIB, 64, 8) == (TREE, LL128, 32)
    assert decide(P6, 32 * MIB, 64, 8) == (TREE, LL128, 32)
    assert decide(P6, 32 * MIB + 1, 64, 8) == (TREE, LL128, -1)
    # other platforms and other ranks-per-node shapes leave nChannels alone
    assert decide(P6_B300, 8 * MIB, 64, 8)[2] == -1
    assert decide(P5EN, 8 * MIB, 64, 8)[2] == -1
    assert decide(P6, 8 * MIB, 64, 64)[2] == -1   # 1 rank per node: Tree/LL128 there (:1194-1201), no override


def test_best_nchannel_pat_breakpoints(oracle):
    """calculateBestNChannelPat (:1943-1953): 1 up to nodes * 64 KiB inclusive, 2 up to
    nodes * 128 KiB inclusive, else 0."""
    for nodes in (1, 3, 8, 16, 64, 512, 1000):
        f = lambda m: oracle.oracle_best_nchannel_pat(m, nodes)
        assert f(0) == 1 and f(nodes * 65536) == 1
        assert f(nodes * 65536 + 1) == 2 and f(nodes * 131072) == 2
        assert f(nodes * 131072 + 1) == 0 and f(1 << 40) == 0


def test_best_nchannel_pat_through_the_region_decision(oracle):
    """:2147-2152: P6, size <= 32 MiB, PAT/Simple, 1 rank per node.  The AllGather PAT/Simple
    polygon of P6 at 1 rank per node (:1243-1254: (0,2) (65536,4) (1048576,4) (4194305,16)
    (12582912,48) (88080384,48) (248512512,128) (34359738368,17137) (0,131072)) holds every point
    used here: at 8 ranks its right edge is near 2 MiB, at 16 ranks at 4 MiB, from 48 ranks up beyond
    88 MB."""
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()

    def decide(plat, coll, size, nodes):
        ch.value = -1
        oracle.oracle_region_decide(plat, coll, size, nodes, nodes, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
        return a.value, p.value, ch.value

    for nodes in (8, 16, 64):
        assert decide(P6, AG, nodes * 65536, nodes) == (PAT, SIMPLE, 1)
        assert decide(P6, AG, nodes * 65536 + 1, nodes) == (PAT, SIMPLE, 2)
        assert decide(P6, AG, nodes * 131072, nodes) == (PAT, SIMPLE, 2)
        assert decide(P6, AG, nodes * 131072 + 1, nodes) == (PAT, SIMPLE, 0)
    # 512 nodes: nodes * 64 KiB is exactly 32 MiB, the last size the override applies to
    assert decide(P6, AG, 32 * MIB, 512) == (PAT, SIMPLE, 1)
    assert decide(P6, AG, 32 * MIB + 1, 512) == (PAT, SIMPLE, -1)
    assert decide(P6_B300, AG, 8 * 65536, 8)[2] == -1


# chunkSizeTuningAllGatherPatSimpleP5en (:2159-2209), n = message size, N = nodes.
#   sat = 1 MiB (N < 16) or 512 KiB; T1 = min(N, 8) + 1 (N < 16) or 32; T2 = min(N, 16); T3 = min(N, 8)
#   step 1: one halving off sat when n // sat < T1          <=> n < T1 * sat
#   step 2: halve while n // c < T2 and c > 64 KiB          c survives <=> n >= T2 * c
#   step 3: halve while n // c < T3 and c > 32 KiB          only ever 64 KiB -> 32 KiB, when n < T3 * 64 KiB
# N = 8  (9, 8, 8):   >= 9 MiB 1 MiB | >= 4 MiB 512 K | >= 2 MiB 256 K | >= 1 MiB 128 K | >= 512 K 64 K | 32 K
# N = 4  (5, 4, 4):   >= 5 MiB 1 MiB | >= 2 MiB 512 K | >= 1 MiB 256 K | >= 512 K 128 K | >= 256 K 64 K | 32 K
# N = 3  (4, 3, 3):   >= 4 MiB 1 MiB | >= 1.5 MiB 512 K | >= 768 K 256 K | >= 384 K 128 K | >= 192 K 64 K | 32 K
# N = 12 (9, 12, 8):  step 1 keeps 1 MiB from 9 MiB, but step 2 wants 12 chunks: 1 MiB only from 12 MiB;
#                     512 K from 6 MiB (9..12 MiB falls back to it); 256 K from 3 MiB; 128 K from 1.5 MiB;
#                     64 K is step 2's floor; step 3 (T3 = 8): 32 K below 512 KiB
# N = 16, 32 (32, 16, 8): sat = 512 K kept from 16 MiB; 256 K from 4 MiB; 128 K from 2 MiB; 64 K floor;
#                     32 K below 512 KiB
KIB = 1 << 10
PAT_LADDERS = {
    8: [(512 * KIB, 65536), (1 * MIB, 131072), (2 * MIB, 262144), (4 * MIB, 524288), (9 * MIB, 1048576)],
    4: [(256 * KIB, 65536), (512 * KIB, 131072), (1 * MIB, 262144), (2 * MIB, 524288), (5 * MIB, 1048576)],
    3: [(192 * KIB, 65536), (384 * KIB, 131072), (768 * KIB, 262144), (1536 * KIB, 524288), (4 * MIB, 1048576)],
    12: [(512 * KIB, 65536), (1536 * KIB, 131072), (3 * MIB, 262144), (6 * MIB, 524288), (12 * MIB, 1048576)],
    16: [(512 * KIB, 65536), (2 * MIB, 131072), (4 * MIB, 262144), (16 * MIB, 524288)],
    32: [(512 * KIB, 65536), (2 * MIB, 131072), (4 * MIB, 262144), (16 * MIB, 524288)],
    1000: [(512 * KIB, 65536), (2 * MIB, 131072), (4 * MIB, 262144), (16 * MIB, 524288)],
}


def _chunk(oracle, plat, coll, size, algo, proto, ranks, nodes):
    out = ctypes.c_uint64(0)
    rc = oracle.oracle_region_chunk_size(plat, coll, size, algo, proto, ranks, nodes, ctypes.byref(out))
    return (rc, out.value)


@pytest.mark.parametrize("nodes", sorted(PAT_LADDERS))
def test_chunk_size_allgather_pat_simple_p5en_breakpoints(oracle, nodes):
    f = lambda n: _chunk(oracle, P5EN, AG, n, PAT, SIMPLE, nodes, nodes)
    before = 32768
    assert f(0) == (1, 32768) and f(1) == (1, 32768)
    for cut, after in PAT_LADDERS[nodes]:
        assert f(cut - 1) == (1, before), (nodes, cut)
        assert f(cut) == (1, after), (nodes, cut)
        before = after
    assert f(1 << 40) == (1, before)


# chunkSizeTuningTreeLL128P5en (:2211-2274), s = 1 + log2(nodes), start 288,000:
#   step 1: halve when n // 288,000 < 2 s^2            <=> n < 2 s^2 * 288,000
#   step 2: halve when n // c < (size_t)(1.5 s)         (truncated: s = 3 -> 4, not 4.5)
#   step 3: halve while n // c < s + 1 and c > 18,000
# step 2 looks at the chunk step 1 left, so once step 1 has fired it tests 144,000.
#   s = 4 (8 nodes):  2 s^2 = 32, trunc 6, s+1 = 5:  288,000 from 9,216,000; 144,000 from 6*144,000 = 864,000
#                     (then 6 >= 5 keeps it); 72,000 from 5*72,000 = 360,000; 36,000 from 180,000; 18,000
#   s = 3 (4 nodes):  18, trunc(4.5) = 4, 4:  288,000 from 5,184,000; 144,000 from 4*144,000 = 576,000;
#                     72,000 from 288,000; 36,000 from 144,000; 18,000
#   s = 6 (32 nodes): 72, 9, 7:  288,000 from 20,736,000; 144,000 from 9*144,000 = 1,296,000;
#                     72,000 from 7*72,000 = 504,000; 36,000 from 252,000; 18,000
#   s = 1 (1 node):   2, trunc(1.5) = 1, 2:  288,000 from 576,000; step 2 fires below 144,000; step 3 halves
#                     144,000 when n // 144,000 < 2: 144,000 from 288,000; 72,000 from 144,000;
#                     36,000 from 72,000; 18,000
TREE_P5EN_LADDERS = {
    8: [(180000, 36000), (360000, 72000), (864000, 144000), (9216000, 288000)],
    4: [(144000, 36000), (288000, 72000), (576000, 144000), (5184000, 288000)],
    32: [(252000, 36000), (504000, 72000), (1296000, 144000), (20736000, 288000)],
    1: [(72000, 36000), (144000, 72000), (288000, 144000), (576000, 288000)],
    # log2i truncates: 12 nodes behave like 8, 63 like 32
    12: [(180000, 36000), (360000, 72000), (864000, 144000), (9216000, 288000)],
    63: [(252000, 36000), (504000, 72000), (1296000, 144000), (20736000, 288000)],
}


@pytest.mark.parametrize("nodes", sorted(TREE_P5EN_LADDERS))
def test_chunk_size_tree_ll128_p5en_breakpoints(oracle, nodes):
    f = lambda n: _chunk(oracle, P5EN, AR, n, TREE, LL128, nodes, nodes)
    before = 18000
    assert f(0) == (1, 18000)
    for cut, after in TREE_P5EN_LADDERS[nodes]:
        assert f(cut - 1) == (1, before), (nodes, cut)
        assert f(cut) == (1, after), (nodes, cut)
        before = after
    assert f(1 << 40) == (1, 288000)
    if nodes == 4:
        # 1.5 * 3 is truncated to 4: five chunks of 144,000 are already enough
        assert f(5 * 144000 - 1) == (1, 144000)


def test_chunk_size_dispatch(oracle):
    """region_get_chunk_size_internal (:2276-2306): only P5en, only 1 rank per node, only
    AllReduce Tree/LL128 and AllGather PAT/Simple; everything else leaves the chunk size alone."""
    for plat in (P5, P6, P6_B300):
        assert _chunk(oracle, plat, AR, MIB, TREE, LL128, 8, 8)[0] == 0
        assert _chunk(oracle, plat, AG, MIB, PAT, SIMPLE, 8, 8)[0] == 0
    assert _chunk(oracle, P5EN, AR, MIB, TREE, LL128, 64, 8)[0] == 0      # 8 ranks per node
    assert _chunk(oracle, P5EN, AG, MIB, PAT, SIMPLE, 16, 8)[0] == 0
    assert _chunk(oracle, P5EN, RS, MIB, PAT, SIMPLE, 8, 8)[0] == 0       # ReduceScatter: no tuning
    assert _chunk(oracle, P5EN, AR, MIB, TREE, LL, 8, 8)[0] == 0
    assert _chunk(oracle, P5EN, AR, MIB, RING, LL128, 8, 8)[0] == 0
    assert _chunk(oracle, P5EN, AG, MIB, PAT, LL128, 8, 8)[0] == 0
    assert _chunk(oracle, P5EN, AG, MIB, RING, SIMPLE, 8, 8)[0] == 0
    assert _chunk(oracle, P5EN, AR, MIB, TREE, LL128, 8, 8) == (1, 144000)
    assert _chunk(oracle, P5EN, AG, MIB, PAT, SIMPLE, 8, 8) == (1, 131072)


def test_chunk_ladders_invariants(oracle):
    """Both P5en ladders never decrease with the message size and only return the rungs reachable
    by halving from their ceilings."""
    for nodes in (1, 2, 3, 5, 8, 12, 15, 16, 17, 100, 1024):
        last_pat = last_tree = 0
        m = 1
        while m < 1 << 38:
            pat = _chunk(oracle, P5EN, AG, m, PAT, SIMPLE, nodes, nodes)[1]
            tree = _chunk(oracle, P5EN, AR, m, TREE, LL128, nodes, nodes)[1]
            assert pat in (32768, 65536, 131072, 262144, 524288, 1048576) and pat >= last_pat
            assert nodes < 16 or pat <= 524288
            assert tree in (18000, 36000, 72000, 144000, 288000) and tree >= last_tree
            last_pat, last_tree = pat, tree
            m = m * 9 // 8 + 1
