"""Pins the tuner oracle.

Regions: the reference's own unit test (tests/unit/region_based_tuner.cpp:20-248) is replayed
point by point, the polygon table is re-derived from the reference source text, and the
decisions over the whole grid are compared with a textbook even-odd point-in-polygon rule.
Model: the reference has no test of its cost function and its object does not build here, so
the oracle is checked against the closed forms in exact rational arithmetic (1e-6 relative, the
tolerance the task states for costs) and against identities a dropped term or a swapped
operand would break.  The exact fp32 bit pattern of the reference binary stays unpinned."""
import ctypes
import math
import os
import subprocess
import sys
from fractions import Fraction as F

import numpy as np
import pytest

import _oracle
from _oracle import Point
from aws_ofi_nccl_amd import synthetic

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_REGIONS = "/root/reference/src/tuner/nccl_ofi_regions.cpp"

AR, AG, RS = 4, 2, 3
TREE, RING, NVLS_TREE, PAT = 0, 1, 5, 6
LL, LL128, SIMPLE = 0, 1, 2
MAX_SIZE = 100.0 * 1024 * 1024 * 1024
MAX_RANKS = 1024.0 * 1024

# src/tuner/nccl_ofi_model.cpp:13-44, as exact rationals
PARAMS = {
    0: dict(net_lat=F(20), ibw=F(125, 10) * 2**30 / 10**6, nbw=F(20) * 2**30 / 10**6, rails=4),
    1: dict(net_lat=F(18), ibw=F(25) * 2**30 / 10**6, nbw=F(20) * 2**30 / 10**6, rails=2),
}
NVLINK_LAT = {TREE: [F(6, 10), F(125, 100), F(28)], RING: [F(6, 10), F(19, 10), F(34, 10)],
              NVLS_TREE: [F(0), F(0), F(23)]}


def exact_cost(plat, algo, proto, pipe, size, R, N, ch=8, ovh=3):
    p = PARAMS[plat]
    net = p["net_lat"] + (ovh if proto == SIMPLE else 0)
    p2p = NVLINK_LAT[algo][proto]
    lg = F(int(math.log2(N)))                       # N is a power of two in these tests
    if algo == RING:
        lat = 2 * N * net + (2 * (R - 1) - 2 * N) * p2p
        bw = p["ibw"] * p["rails"] * ch
    elif algo == TREE:
        lat = 2 * (R // N - 1) * p2p + 2 * lg * net
        bw = p["ibw"] * p["rails"] * ch / 2
    else:
        lat = 2 * (p2p + lg * net)
        bw = min(p["nbw"], p["ibw"] * p["rails"] / 2) * ch
    bw *= {LL: F(1, 2), LL128: F(15, 16), SIMPLE: F(1)}[proto]
    return lat * pipe + F(size) / bw


def test_model_cost_closed_forms(oracle):
    rng = np.random.default_rng(0)
    worst = 0.0
    for plat in (0, 1):
        for algo in (TREE, RING, NVLS_TREE):
            for proto in (LL, LL128, SIMPLE):
                for _ in range(150):
                    N = 1 << int(rng.integers(0, 11))
                    R = N * int(rng.choice([1, 2, 4, 8]))
                    size = int(synthetic.log_uniform_sizes(int(rng.integers(1 << 30)), 1, 0, 35)[0])
                    pipe = int(rng.integers(1, 9))
                    got = oracle.oracle_model_cost(plat, AR, algo, proto, pipe, size, R, N, 8, 3)
                    want = exact_cost(plat, algo, proto, pipe, size, R, N)
                    if want == 0:
                        assert got == 0.0
                        continue
                    rel = abs(F(got) - want) / abs(want)
                    worst = max(worst, float(rel))
                    assert rel < F(1, 10**6), (plat, algo, proto, pipe, size, R, N, got, float(want))
    assert worst < 1e-6


def test_model_unmodelled_cells_are_minus_one(oracle):
    for coll in (AG, RS, 0, 1):
        assert oracle.oracle_model_cost(0, coll, RING, SIMPLE, 1, 1 << 20, 64, 8, 8, 3) == -1.0
    for algo in (2, 3, 4, PAT):
        assert oracle.oracle_model_cost(0, AR, algo, SIMPLE, 1, 1 << 20, 64, 8, 8, 3) == -1.0


def test_model_identities(oracle):
    c = lambda algo, proto, size, R=64, N=8, pipe=1, plat=0: float(
        oracle.oracle_model_cost(plat, AR, algo, proto, pipe, size, R, N, 8, 3))
    # size 0 leaves the latency term; it scales with numPipeOps
    assert c(RING, SIMPLE, 0) == pytest.approx(2 * 8 * 23 + (2 * 63 - 16) * 3.4, rel=1e-6)
    assert c(RING, SIMPLE, 0, pipe=4) == pytest.approx(4 * c(RING, SIMPLE, 0), rel=1e-6)
    # ppn = 1: the intra-node step count goes negative (int arithmetic), the term subtracts
    assert c(RING, LL, 0, R=8, N=8) == pytest.approx(2 * 8 * 20 - 2 * 0.6, rel=1e-6)
    # one node: log2(1) = 0, tree latency is the NVLink part only
    assert c(TREE, LL128, 0, R=8, N=1) == pytest.approx(2 * 7 * 1.25, rel=1e-6)
    # bandwidth term is linear in size and the protocol factors are 1/2 and 15/16
    big, lat = 1 << 33, c(RING, SIMPLE, 0)
    t_simple = c(RING, SIMPLE, big) - lat
    assert c(RING, SIMPLE, 2 * big) - lat == pytest.approx(2 * t_simple, rel=1e-6)
    assert (c(RING, LL, big) - c(RING, LL, 0)) == pytest.approx(2 * t_simple, rel=1e-6)
    assert (c(RING, LL128, big) - c(RING, LL128, 0)) == pytest.approx(t_simple * 16 / 15, rel=1e-6)
    # tree has half the ring bandwidth; P5en has twice the per-rail rate on half the rails
    assert (c(TREE, SIMPLE, big) - c(TREE, SIMPLE, 0)) == pytest.approx(2 * t_simple, rel=1e-6)
    assert (c(RING, SIMPLE, big, plat=1) - c(RING, SIMPLE, 0, plat=1)) == pytest.approx(t_simple, rel=1e-6)
    # (float)size: sizes above 2^24 round to 24 significant bits before the divide
    assert c(RING, SIMPLE, (1 << 30) + 1) == c(RING, SIMPLE, 1 << 30)


def test_model_decision_is_first_strict_minimum(oracle):
    colls, sizes, nodes, ppn, _ = synthetic.tuner_axes()
    a, p = ctypes.c_int(), ctypes.c_int()
    checked = 0
    for plat in (0, 1):
        for coll in (AR, AG):
            for s in sizes[::7]:
                for N in nodes:
                    for q in ppn:
                        R, N_, s_ = int(N) * int(q), int(N), int(s)
                        oracle.oracle_model_decide(plat, coll, 1, s_, R, N_, 8, 3,
                                                   ctypes.byref(a), ctypes.byref(p))
                        best, choice = None, (-1, -1)
                        quirk = (plat == 0 and coll == AR and N_ == 16 and R == 128
                                 and 3 << 30 < s_ <= 5 << 30)
                        if N_ > 2 and quirk:
                            choice = (NVLS_TREE, SIMPLE)
                        elif N_ > 2:
                            for algo in (0, 1, 5, 6):
                                for proto in (0, 1, 2):
                                    if algo == NVLS_TREE and proto != SIMPLE:
                                        continue
                                    cst = oracle.oracle_model_cost(plat, coll, algo, proto, 1, s_, R,
                                                                   N_, 8, 3)
                                    if cst >= 0 and (best is None or cst < best):
                                        best, choice = cst, (algo, proto)
                        assert (a.value, p.value) == choice
                        checked += 1
    assert checked > 3000


def test_model_p5_quirk_and_small_jobs(oracle):
    a, p = ctypes.c_int(), ctypes.c_int()
    oracle.oracle_model_decide(0, AR, 1, 4 << 30, 128, 16, 8, 3, ctypes.byref(a), ctypes.byref(p))
    assert (a.value, p.value) == (NVLS_TREE, SIMPLE)             # nccl_ofi_model.cpp:183-192
    oracle.oracle_model_decide(0, AR, 1, 3 << 30, 128, 16, 8, 3, ctypes.byref(a), ctypes.byref(p))
    assert (a.value, p.value) != (-1, -1)                        # bound is exclusive below
    for N in (1, 2):                                             # :178
        oracle.oracle_model_decide(0, AR, 1, 1 << 20, 8 * N, N, 8, 3, ctypes.byref(a), ctypes.byref(p))
        assert (a.value, p.value) == (-1, -1)
    oracle.oracle_model_decide(0, AG, 1, 1 << 20, 64, 8, 8, 3, ctypes.byref(a), ctypes.byref(p))
    assert (a.value, p.value) == (-1, -1)                        # nothing modelled: no choice


# ------------------------------------------------------------------ regions

def ext(oracle, a, b):
    return oracle.oracle_region_extend(Point(*a), Point(*b), Point(MAX_SIZE, MAX_RANKS))


def test_extend_region_reference_cases(oracle):
    """test_extend_region, tests/unit/region_based_tuner.cpp:20-73"""
    eps = 1e-4
    e = ext(oracle, (2, 8), (4, 8))
    assert abs(e.x - MAX_SIZE) <= eps and e.y == 8
    e = ext(oracle, (8, 2), (8, 4))
    assert e.x == 8 and e.y == MAX_RANKS
    e = ext(oracle, (8, 64), (8290304, 72))
    slope = (math.log2(72.0) - math.log2(64.0)) / (math.log2(8290304.0) - math.log2(8.0))
    projected_y = math.pow(2.0, math.log2(72.0) + slope * (math.log2(MAX_SIZE) - math.log2(8290304.0)))
    assert abs(e.x - MAX_SIZE) <= eps
    assert e.y == pytest.approx(projected_y, rel=1e-12)      # the reference compares with != ;
    # libm's pow/log2 here and CPython's are the same glibc, so the bits agree as well:
    assert e.y == projected_y
    e = ext(oracle, (8, 64), (16, 1024))
    slope = (math.log2(1024.0) - math.log2(64.0)) / (math.log2(16) - math.log2(8.0))
    projected_x = math.pow(2, ((math.log2(MAX_RANKS) - math.log2(1024.0)) / slope) + math.log2(16))
    assert abs(e.x - projected_x) <= eps and e.y == MAX_RANKS


def reference_polygon(oracle):
    M = 1024.0 * 1024
    e = ext(oracle, (48 * M, 16), (288 * M, 128))
    lin = [(e.x, e.y), (288 * M, 128), (48 * M, 16), (4 * M, 2), (MAX_SIZE, 2)]
    verts = (Point * 5)(*[oracle.oracle_region_log2(Point(*v)) for v in lin])
    return e, verts


def test_is_inside_region_reference_cases(oracle):
    """test_is_inside_region, tests/unit/region_based_tuner.cpp:92-248"""
    M, G = 1024.0 * 1024, 1024.0 * 1024 * 1024
    e, verts = reference_polygon(oracle)
    inside = lambda pt: oracle.oracle_region_inside(pt, verts, 5)
    lg = lambda x, y: oracle.oracle_region_log2(Point(x, y))

    for v in verts:                                   # vertices are "on edge" (:121-133)
        assert inside(v) == 0
    for i in range(5):                                # points along the edges (:140-153), same walk
        k = (i + 1) % 5
        if verts[k].x <= verts[i].x:
            continue                                  # the C loop `x < v[k].x` runs zero times
        slope = (verts[k].y - verts[i].y) / (verts[k].x - verts[i].x)
        c = verts[k].y - (slope * verts[i].x)
        x = verts[i].x
        while x < verts[k].x:
            assert inside(Point(x, slope * x + c)) == 0
            x = x * 2
    off = ext(oracle, (48 * M, 16), (288 * M, 128))
    inside_pts = [(16 * M, 4), (128 * M, 4), (1 * G, 4), (4 * G, 4), (16 * G, 4), (32 * G, 4),
                  (64 * M, 16), (1 * G, 16), (4 * G, 16), (16 * G, 16), (32 * G, 16), (64 * G, 16),
                  (512 * M, 128), (4 * G, 128), (16 * G, 128), (32 * G, 128), (64 * G, 128),
                  (64 * G, 256), (MAX_SIZE - 10.0, 128), (off.x - 10.0, off.y - 10.0)]
    for pt in inside_pts:                             # :165-196
        assert inside(lg(*pt)) == 1, pt
    # :201-243 -- these are passed without the log2 transform in the reference test
    outside_raw = [(8 * M, 4), (8 * M, 32), (8 * M, 128), (8 * M, 512), (8 * M, MAX_RANKS),
                   (16 * M, 8), (16 * M, 32), (16 * M, 128), (16 * M, 512), (16 * M, MAX_RANKS),
                   (32 * M, 16), (32 * M, 32), (32 * M, 64), (32 * M, 128), (32 * M, 256),
                   (64 * M, 32), (64 * M, 64), (64 * M, 256), (64 * M, 1024), (256 * M, 256),
                   (256 * M, 1024), (256 * M, 2048), (MAX_SIZE + 1.0, 128), (e.x + 1.0, e.y + 1.0),
                   (2 * M, 2), (64 * M, 64), (200 * M, 128), (1024 * M, 1024), (1024 * M, 2048)]
    for pt in outside_raw:
        assert inside(Point(*pt)) == -1, pt
    # the same byte/rank values given properly in log2 space: those above or left of the
    # sloped edge are outside, the rest of that list actually lie inside
    for pt in [(8 * M, 4), (8 * M, 32), (16 * M, 8), (32 * M, 16), (64 * M, 32), (64 * M, 1024),
               (256 * M, 256), (256 * M, 2048), (2 * M, 4), (MAX_SIZE * 1.01, 128), (64 * M, 1.9)]:
        assert inside(lg(*pt)) == -1, pt
    # just either side of the bottom edge y = 2 and of the sloped edge through (48 MiB,16)-(288 MiB,128)
    assert inside(lg(1 * G, 2.0001)) == 1 and inside(lg(1 * G, 1.9999)) == -1
    slope = (math.log2(128) - math.log2(16)) / (math.log2(288 * M) - math.log2(48 * M))
    y_on = 2.0 ** (math.log2(16) + slope * (math.log2(100 * M) - math.log2(48 * M)))
    assert inside(lg(100 * M, y_on * 0.999)) == 1 and inside(lg(100 * M, y_on * 1.001)) == -1


def test_region_table_matches_reference_source():
    """The committed flat table is what the generator extracts from the reference text."""
    if not os.path.exists(REF_REGIONS):
        pytest.skip("reference tree not available")
    gen = os.path.join(ROOT, "aws_ofi_nccl_amd", "csrc", "gen_region_tables.py")
    out = subprocess.run([sys.executable, gen, REF_REGIONS], check=True, stdout=subprocess.PIPE).stdout
    committed = open(os.path.join(ROOT, "aws_ofi_nccl_amd", "csrc", "region_tables.inc"), "rb").read()
    assert out == committed


def test_region_table_shape(oracle):
    """Which (platform, shape, collective) have regions: the per-platform tables of src/tuner/nccl_ofi_regions.cpp:295-1882."""
    algos, protos, nv = (ctypes.c_int * 16)(), (ctypes.c_int * 16)(), (ctypes.c_int * 16)()
    verts = (Point * (16 * 20))()
    count = lambda plat, R, N, coll: oracle.oracle_region_polys(plat, R, N, coll, algos, protos, nv, verts, 16)
    for plat in range(4):
        for coll in (AR, AG, RS):
            assert count(plat, 64, 8, coll) > 0 or (plat == 0 and coll != AR)     # R == 8N
            assert count(plat, 8, 8, coll) > 0                                     # R == N
            assert count(plat, 32, 8, coll) == 0                                   # R == 4N: none
            assert (count(plat, 16, 8, coll) > 0) == (plat == 0 and coll == AR)    # R == 2N: P5 AR
    # first P5en / 8 ranks per node / AllReduce polygon: Tree-LL, 5 vertices, two of them at 16 ranks
    assert count(1, 64, 8, AR) == 5
    assert (algos[0], protos[0], nv[0]) == (TREE, LL, 5)
    assert verts[0].y == 4.0 and verts[1].x == math.log2(196608) and verts[1].y == 4.0
    assert verts[0].x == math.log2(1e-6)            # x = 0 becomes log2(1e-6)


def test_region_decisions_spot_checks(oracle):
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(-1)
    dec = lambda plat, coll, size, R, N: (oracle.oracle_region_decide(
        plat, coll, size, R, N, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch)), (a.value, p.value))[1]
    # P5en, 8 ranks/node, AllReduce: small -> Tree/LL, mid -> Tree/LL128, huge at 32 ranks -> Ring/Simple
    assert dec(1, AR, 1024, 32, 4) == (TREE, LL)
    assert dec(1, AR, 196608, 32, 4) == (TREE, LL)          # on the shared edge: first region wins
    assert dec(1, AR, 196609, 32, 4) == (TREE, LL128)
    assert dec(1, AR, 64 << 30, 32, 4) == (RING, SIMPLE)
    assert dec(1, AR, 1024, 16, 2) == (-1, -1)              # two nodes or fewer: no decision
    assert dec(1, AR, 1024, 16, 4) == (-1, -1)              # 4 ranks/node: no regions
    assert dec(1, AR, 200 << 30, 64, 8) == (-1, -1)         # beyond TUNER_MAX_SIZE: outside all
    assert dec(0, AG, 1 << 20, 64, 8) == (-1, -1)           # P5 has AllGather regions only at 1 rank/node


def test_channel_and_chunk_heuristics(oracle):
    # calculateChunkSizeTreeLL128 by hand for 8 MiB, 16 channels, 4 nodes (log2 = 2):
    # start 614400*15/16 = 576000; nSteps = 3.8; 8388608/(16*576000) = 0 < 30.4 -> halve to 288000,
    # 144000, then stops at > 131072?  144000 > 131072 so once more: 72000; second loop: 8388608/
    # (16*72000) = 7 < 7.6 -> 36000 (> 32768) -> 14 >= 7.6 stop; grain 1920 -> 34560;
    # nelem = 18*480 = 8640; ceil(8640/480) = 18 slices * 256 words * 8 B = 36864
    assert oracle.oracle_chunk_tree_ll128(8 << 20, 16, 2) == 36864
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(-1)
    # P6, 1 rank per node, PAT/Simple region: nChannels 1 up to nodes*64 KiB, 2 up to twice that, else 0
    # (every breakpoint of these ladders is pinned in test_oracle_tuner_heuristics.py)
    for size, want in [(8 * 65536, 1), (8 * 65536 + 1, 2), (8 * 131072, 2), (8 * 131072 + 1, 0)]:
        ch.value = -1
        oracle.oracle_region_decide(2, AG, size, 8, 8, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
        assert (a.value, p.value, ch.value) == (PAT, SIMPLE, want)
    out = ctypes.c_uint64(0)
    # chunkSizeTuningTreeLL128P5en (:2211-2274): 8 nodes -> nsteps 4; 64 MiB per channel keeps 288000
    assert oracle.oracle_region_chunk_size(1, AR, 64 << 20, TREE, LL128, 8, 8, ctypes.byref(out)) == 1
    assert out.value == 288000
    # 1 MiB: 3 chunks < 32 -> 144000; 7 >= 6; 7 >= 5 -> stays
    oracle.oracle_region_chunk_size(1, AR, 1 << 20, TREE, LL128, 8, 8, ctypes.byref(out))
    assert out.value == 144000
    # tiny message walks the ladder to the floor
    oracle.oracle_region_chunk_size(1, AR, 1000, TREE, LL128, 8, 8, ctypes.byref(out))
    assert out.value == 18000
    # AllGather PAT/Simple (:2159-2209): 8 nodes, 16 MiB -> 16 chunks of 1 MiB >= T1 = 9 -> 1048576
    oracle.oracle_region_chunk_size(1, AG, 16 << 20, PAT, SIMPLE, 8, 8, ctypes.byref(out))
    assert out.value == 1048576
    oracle.oracle_region_chunk_size(1, AG, 1 << 20, PAT, SIMPLE, 8, 8, ctypes.byref(out))
    assert out.value == 131072        # 1 MiB: cap step -> 512 KiB; 2 < 8 -> 256 K (4) -> 128 K (8 >= 8)
    assert oracle.oracle_region_chunk_size(0, AR, 1 << 20, TREE, LL128, 8, 8, ctypes.byref(out)) == 0
    assert oracle.oracle_region_chunk_size(1, AR, 1 << 20, TREE, LL128, 64, 8, ctypes.byref(out)) == 0


def _independent_region_choice(polys, px, py):
    """First polygon in table order that holds (px, py) by the even-odd rule along a horizontal ray
    towards +x -- not the reference's ray to a far corner -- and the distance to the nearest edge of
    any polygon of the set.  polys: [(algo, proto, [(x, y), ...]), ...] in log2 space."""
    nearest = math.inf
    found = None
    for algo, proto, vs in polys:
        crossings = 0
        for i in range(len(vs)):
            (x1, y1), (x2, y2) = vs[i], vs[(i + 1) % len(vs)]
            ex, ey = x2 - x1, y2 - y1
            ee = ex * ex + ey * ey
            t = 0.0 if ee == 0 else max(0.0, min(1.0, ((px - x1) * ex + (py - y1) * ey) / ee))
            nearest = min(nearest, math.hypot(px - (x1 + t * ex), py - (y1 + t * ey)))
            if (y1 > py) != (y2 > py) and x1 + (py - y1) * ex / ey > px:
                crossings += 1
        if found is None and crossings % 2 == 1:
            found = (algo, proto)
    return found or (-1, -1), nearest


def test_region_decisions_against_an_independent_point_in_polygon_rule(oracle):
    """(algorithm, protocol) of the oracle's region decision over the configured grid of every
    platform and over random (size, nodes, ranks per node) points, against a textbook even-odd test
    on the same polygon table (itself compared with the reference text above).  Points closer than
    1e-6 to an edge are left to the reference's own on-edge cases (its unit-test points, replayed
    above): there the answer depends on its epsilon rules, not on geometry."""
    colls, sizes, nodes, ppn, _ = synthetic.tuner_axes()
    algos, protos, nv = (ctypes.c_int * 16)(), (ctypes.c_int * 16)(), (ctypes.c_int * 16)()
    verts = (Point * (16 * 20))()

    def polygons(plat, R, N, coll):
        n = oracle.oracle_region_polys(plat, R, N, coll, algos, protos, nv, verts, 16)
        return [(algos[q], protos[q], [(verts[q * 20 + v].x, verts[q * 20 + v].y) for v in range(nv[q])])
                for q in range(n)]

    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    rng = np.random.default_rng(5)
    checked = skipped = decided = 0
    for plat in range(4):
        points = [(int(c), int(s), int(n) * int(k), int(n)) for c in colls for s in sizes for n in nodes for k in ppn]
        for _ in range(6000):
            n = int(rng.integers(1, 3000))
            points.append((int(rng.choice(colls)), int(2.0 ** rng.uniform(0, 37.5)), n * int(rng.choice([1, 2, 8])), n))
        cache = {}
        for coll, size, R, N in points:
            key = (coll, R // N)
            if key not in cache:
                cache[key] = polygons(plat, R, N, coll)
            oracle.oracle_region_decide(plat, coll, size, R, N, ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
            if N <= 2 or not cache[key]:
                assert (a.value, p.value) == (-1, -1), (plat, coll, size, R, N)
                continue
            at = oracle.oracle_region_log2(Point(float(size), float(R)))
            want, nearest = _independent_region_choice(cache[key], at.x, at.y)
            if nearest < 1e-6:
                skipped += 1
                continue
            assert (a.value, p.value) == want, (plat, coll, size, R, N, nearest)
            checked += 1
            decided += want != (-1, -1)
    print(f"independent rule: {checked} points compared, {decided} of them inside a region, {skipped} within 1e-6 of an edge")
    assert checked > 15000 and decided > 8000 and skipped < checked // 50, (checked, decided, skipped)
