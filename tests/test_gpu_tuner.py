"""GPU parity: batched tuner grids through the C ABI against the CPU oracle.
Costs are compared bit for bit as fp32 (the task's tolerance is 1e-6 relative; the kernels meet
the stricter bar), algorithm / protocol / channel choices exactly."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import _oracle
import aws_ofi_nccl_amd as m
from aws_ofi_nccl_amd import synthetic

pytestmark = pytest.mark.gpu


def make_plan(lib, colls, sizes, nodes, ppn, algos):
    plan = ctypes.c_void_p()
    rc = lib.ofi_amd_tuner_plan_create(colls.ctypes.data, len(colls), sizes.ctypes.data, len(sizes),
                                       nodes.ctypes.data, len(nodes), ppn.ctypes.data, len(ppn),
                                       algos.ctypes.data, len(algos), ctypes.byref(plan))
    assert rc == 0
    return plan


def oracle_model_grid(oracle, variants, colls, sizes, nodes, ppn, algos):
    cost = np.zeros((len(variants), len(colls), len(sizes), len(nodes), len(ppn), len(algos), 3), np.float32)
    choice = np.zeros((len(variants), len(colls), len(sizes), len(nodes), len(ppn), 2), np.int8)
    a, p = ctypes.c_int(), ctypes.c_int()
    for vi, v in enumerate(variants):
        for ci, c in enumerate(colls):
            for si, s in enumerate(sizes):
                for ni, n in enumerate(nodes):
                    for pi, q in enumerate(ppn):
                        R, N, S = int(n) * int(q), int(n), int(s)
                        modelled = v.platform in (0, 1)
                        for ai, al in enumerate(algos):
                            for pr in range(3):
                                cost[vi, ci, si, ni, pi, ai, pr] = oracle.oracle_model_cost(
                                    v.platform, int(c), int(al), pr, v.pipe_ops, S, R, N,
                                    v.num_channels, v.net_comp_overhead) if modelled else -1.0
                        if modelled:
                            oracle.oracle_model_decide(v.platform, int(c), v.pipe_ops, S, R, N,
                                                       v.num_channels, v.net_comp_overhead,
                                                       ctypes.byref(a), ctypes.byref(p))
                            choice[vi, ci, si, ni, pi] = (a.value, p.value)
                        else:
                            choice[vi, ci, si, ni, pi] = (-1, -1)
    return cost, choice


def run_model(lib, plan, variants, shape):
    nv = len(variants)
    cells, points = lib.ofi_amd_tuner_plan_cells(plan), lib.ofi_amd_tuner_plan_points(plan)
    arr = (m.TunerVariant * nv)(*variants)
    d_cost = torch.full((nv * cells,), 7.0, dtype=torch.float64, device="cuda")
    d_choice = torch.full((nv * points * 2,), 99, dtype=torch.int8, device="cuda")
    assert lib.ofi_amd_tuner_model_grid(plan, arr, nv, d_cost.data_ptr(), d_choice.data_ptr(),
                                        _gpu.stream()) == 0
    _gpu.sync()
    return d_cost.cpu().numpy().reshape(shape + (3,)), d_choice.cpu().numpy().reshape(shape[:-1] + (2,))


def test_model_full_grid_both_platforms(lib, oracle, gpu):
    """The configuration grid: {AR, AG, RS} x 140 sizes x 11 node counts x 4 ranks/node x
    {Ring, Tree, PAT} x 3 protocols, P5/P5e and P5en."""
    colls, sizes, nodes, ppn, algos = synthetic.tuner_axes()
    plan = make_plan(lib, colls, sizes, nodes, ppn, algos)
    assert lib.ofi_amd_tuner_plan_points(plan) == 18480 and lib.ofi_amd_tuner_plan_cells(plan) == 166320
    variants = [m.TunerVariant(0, 1, 8, 3), m.TunerVariant(1, 1, 8, 3)]
    want_cost, want_choice = oracle_model_grid(oracle, variants, colls, sizes, nodes, ppn, algos)
    cost, choice = run_model(lib, plan, variants, (2, 3, 140, 11, 4, 3))
    got32 = cost.astype(np.float32)
    assert np.array_equal(got32.astype(np.float64), cost)            # fp64 output holds fp32 values
    assert np.array_equal(got32.view(np.uint32), want_cost.view(np.uint32))
    assert np.array_equal(choice, want_choice)
    # what the grid contains: real costs only for AllReduce x {Ring, Tree}
    assert np.all(cost[:, 1:] == -1.0) and np.all(cost[:, 0, :, :, :, 2] == -1.0)
    assert np.all(cost[:, 0, :, :, :, :2] > 0)
    assert lib.ofi_amd_tuner_plan_destroy(plan) == 0


def test_model_variants_and_odd_axes(lib, oracle, gpu):
    """numPipeOps / channel / overhead variants, non-power-of-two node counts and sizes, the P5
    NVLS-tree quirk point, platforms without a model, and NVLS_TREE in the emitted algorithm list."""
    colls = np.array([4, 0, 2], dtype=np.int32)
    sizes = np.array([0, 1, 1000, 3 << 30, (3 << 30) + 1, 4 << 30, 5 << 30, (5 << 30) + 1,
                      (1 << 40) + 12345, (1 << 24) + 1], dtype=np.uint64)
    nodes = np.array([1, 2, 3, 5, 16, 24, 1000], dtype=np.uint64)
    ppn = np.array([1, 3, 8], dtype=np.uint32)
    algos = np.array([0, 1, 2, 3, 4, 5, 6], dtype=np.int32)
    plan = make_plan(lib, colls, sizes, nodes, ppn, algos)
    variants = [m.TunerVariant(0, 1, 8, 3), m.TunerVariant(1, 4, 16, 0), m.TunerVariant(0, 7, 1, 10),
                m.TunerVariant(2, 1, 8, 3), m.TunerVariant(3, 2, 8, 3)]
    want_cost, want_choice = oracle_model_grid(oracle, variants, colls, sizes, nodes, ppn, algos)
    cost, choice = run_model(lib, plan, variants, (5, 3, 10, 7, 3, 7))
    assert np.array_equal(cost.astype(np.float32).view(np.uint32), want_cost.view(np.uint32))
    assert np.array_equal(choice, want_choice)
    assert tuple(choice[0, 0, 5, 4, 2]) == (5, 2)                    # 16 nodes x 8, 4 GiB on P5: NVLS tree
    assert np.all(choice[3:] == -1) and np.all(cost[3:] == -1.0)     # P6 platforms have no model
    lib.ofi_amd_tuner_plan_destroy(plan)


@pytest.mark.parametrize("n_nodes,n_ppn", [(51, 5), (64, 4), (257, 1), (40, 8), (1, 1)])
def test_model_grid_on_wide_and_narrow_axes(lib, oracle, gpu, n_nodes, n_ppn):
    """Many (node count, ranks per node) pairs per size, or a single one; an algorithm list without
    a PAT column but with NVLS tree; three variants, one on a platform without a model.  The
    oracle's bits, also when only one of the two outputs is asked for."""
    rng = np.random.default_rng(n_nodes * 10 + n_ppn)
    colls = np.array([4, 3], dtype=np.int32)
    sizes = np.unique((2 ** rng.uniform(0, 36, 7)).astype(np.uint64))
    nodes = np.arange(1, n_nodes + 1, dtype=np.uint64) * np.uint64(3)
    ppn = np.array([1, 2, 4, 8, 3, 5, 6, 7][:n_ppn], dtype=np.uint32)
    algos = np.array([1, 0, 5], dtype=np.int32)                      # Ring, Tree, NVLS tree: no PAT column
    plan = make_plan(lib, colls, sizes, nodes, ppn, algos)
    variants = [m.TunerVariant(0, 2, 8, 3), m.TunerVariant(1, 1, 4, 1), m.TunerVariant(3, 1, 8, 3)]
    shape = (3, 2, len(sizes), n_nodes, n_ppn, 3)
    want_cost, want_choice = oracle_model_grid(oracle, variants, colls, sizes, nodes, ppn, algos)
    cost, choice = run_model(lib, plan, variants, shape)
    assert np.array_equal(cost.astype(np.float32).view(np.uint32), want_cost.view(np.uint32))
    assert np.array_equal(choice, want_choice)
    # one output at a time
    nv, cells, points = 3, lib.ofi_amd_tuner_plan_cells(plan), lib.ofi_amd_tuner_plan_points(plan)
    arr = (m.TunerVariant * nv)(*variants)
    d_cost = torch.full((nv * cells,), 7.0, dtype=torch.float64, device="cuda")
    d_choice = torch.full((nv * points * 2,), 99, dtype=torch.int8, device="cuda")
    assert lib.ofi_amd_tuner_model_grid(plan, arr, nv, d_cost.data_ptr(), None, _gpu.stream()) == 0
    assert lib.ofi_amd_tuner_model_grid(plan, arr, nv, None, d_choice.data_ptr(), _gpu.stream()) == 0
    _gpu.sync()
    assert np.array_equal(d_cost.cpu().numpy().reshape(shape + (3,)), cost)
    assert np.array_equal(d_choice.cpu().numpy().reshape(shape[:-1] + (2,)), choice)
    lib.ofi_amd_tuner_plan_destroy(plan)


def oracle_region_grid(oracle, platforms, colls, sizes, nodes, ppn):
    out = np.zeros((len(platforms), len(colls), len(sizes), len(nodes), len(ppn), 3), np.int32)
    a, p, ch = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    for vi, plat in enumerate(platforms):
        for ci, c in enumerate(colls):
            for si, s in enumerate(sizes):
                for ni, n in enumerate(nodes):
                    for pi, q in enumerate(ppn):
                        ch.value = -1
                        oracle.oracle_region_decide(int(plat), int(c), int(s), int(n) * int(q), int(n),
                                                    ctypes.byref(a), ctypes.byref(p), ctypes.byref(ch))
                        out[vi, ci, si, ni, pi] = (a.value, p.value, ch.value)
    return out


def run_region(lib, plan, platforms, shape):
    points = lib.ofi_amd_tuner_plan_points(plan)
    plats = np.asarray(platforms, dtype=np.int32)
    d = torch.full((len(plats) * points * 4,), 99, dtype=torch.int8, device="cuda")
    assert lib.ofi_amd_tuner_region_grid(plan, plats.ctypes.data, len(plats), d.data_ptr(), _gpu.stream()) == 0
    _gpu.sync()
    raw = d.cpu().numpy().reshape(shape + (4,))
    out = np.zeros(shape + (3,), np.int32)
    out[..., 0], out[..., 1] = raw[..., 0], raw[..., 1]
    out[..., 2] = raw[..., 2:4].copy().view(np.int16)[..., 0]
    return out


def test_region_full_grid_four_platforms(lib, oracle, gpu):
    colls, sizes, nodes, ppn, algos = synthetic.tuner_axes()
    plan = make_plan(lib, colls, sizes, nodes, ppn, algos)
    want = oracle_region_grid(oracle, [0, 1, 2, 3], colls, sizes, nodes, ppn)
    got = run_region(lib, plan, [0, 1, 2, 3], (4, 3, 140, 11, 4))
    mism = np.argwhere((got != want).any(axis=-1))
    assert len(mism) == 0, mism[:10]
    decided = (want[..., 0] >= 0)
    assert decided.sum() > 20000 and (want[..., 2] >= 0).sum() > 1000     # not vacuous
    assert not decided[:, :, :, :2].any()                                 # nodes <= 2 never decide
    assert not decided[1:, :, :, :, 1:3].any()                            # 2 / 4 ranks per node: P5 only
    lib.ofi_amd_tuner_plan_destroy(plan)


def test_region_dense_sizes_near_edges(lib, oracle, gpu):
    """Sizes on and next to polygon vertices (196608, 13107200, ...), node counts that are not
    powers of two, all five collectives of the table axis."""
    colls = np.array([4, 2, 3, 0], dtype=np.int32)
    anchors = [196608, 13107200, 29884416, 129499136, 786432, 4718592, 31457280, 31457281, 3145728,
               32768, 131072, 8388608, 107374182400, 65536 * 8, 4 << 20, 32 << 20]
    sizes = np.array(sorted({max(0, a + d) for a in anchors for d in (-1, 0, 1)} | {0, 1}), dtype=np.uint64)
    nodes = np.array([2, 3, 4, 6, 8, 16, 17, 127, 128, 1000, 131072], dtype=np.uint64)
    ppn = np.array([1, 2, 8], dtype=np.uint32)
    plan = make_plan(lib, colls, sizes, nodes, ppn, np.array([1], dtype=np.int32))
    want = oracle_region_grid(oracle, [0, 1, 2, 3], colls, sizes, nodes, ppn)
    got = run_region(lib, plan, [0, 1, 2, 3], (4, 4, len(sizes), len(nodes), 3))
    mism = np.argwhere((got != want).any(axis=-1))
    assert len(mism) == 0, mism[:10]
    lib.ofi_amd_tuner_plan_destroy(plan)


@pytest.mark.parametrize("n_sizes,n_nodes", [(1, 1), (9, 7), (8, 8), (13, 5), (43, 3), (1, 200)])
def test_region_grid_shapes_around_the_workgroup_size(lib, oracle, gpu, n_sizes, n_nodes):
    """Sizes x nodes per (collective, ranks per node) pair of 1, 63, 64, 65, 129 and 200 points:
    workgroups of 64 with a short or an empty tail, one pair only, platform lists with repeats."""
    rng = np.random.default_rng(n_sizes * 1000 + n_nodes)
    sizes = np.sort(np.unique(np.floor(2.0 ** rng.uniform(0, 37, 4 * n_sizes)).astype(np.uint64)))[:n_sizes]
    assert len(sizes) == n_sizes
    nodes = np.sort(rng.choice(np.arange(1, 3000), n_nodes, replace=False)).astype(np.uint64)
    for colls, ppn, platforms in (([2], [8], [1]), ([4, 3], [1, 8, 2], [3, 0, 0, 2, 1])):
        colls, ppn = np.array(colls, dtype=np.int32), np.array(ppn, dtype=np.uint32)
        plan = make_plan(lib, colls, sizes, nodes, ppn, np.array([1], dtype=np.int32))
        want = oracle_region_grid(oracle, platforms, colls, sizes, nodes, ppn)
        got = run_region(lib, plan, platforms, (len(platforms), len(colls), n_sizes, n_nodes, len(ppn)))
        mism = np.argwhere((got != want).any(axis=-1))
        assert len(mism) == 0, mism[:10]
        assert n_nodes < 3 or (want[..., 0] >= 0).any()
        lib.ofi_amd_tuner_plan_destroy(plan)


def test_region_grid_on_changing_platform_lists(lib, oracle, gpu):
    """One plan, platform lists that grow, shrink and change in place: the launch order the plan keeps
    for a list (which entry, chunk and ranks-per-node value each workgroup takes) is rebuilt whenever
    the list differs from the last call's, never reused for another list."""
    colls = np.array([4, 2, 3], dtype=np.int32)
    sizes = np.array(sorted({int(2 ** (k / 2)) for k in range(10, 70)}), dtype=np.uint64)
    nodes = np.array([1, 2, 3, 4, 8, 16, 32, 64, 100], dtype=np.uint64)
    ppn = np.array([1, 2, 4, 8], dtype=np.uint32)
    plan = make_plan(lib, colls, sizes, nodes, ppn, np.array([1], dtype=np.int32))
    cache = {}
    for platforms in ([0, 1, 2, 3], [3], [1, 1, 0], [0, 1, 1], [2, 3, 0, 1, 0, 3, 2], [3], [0, 1, 2, 3]):
        key = tuple(platforms)
        if key not in cache:
            cache[key] = oracle_region_grid(oracle, platforms, colls, sizes, nodes, ppn)
        got = run_region(lib, plan, platforms, (len(platforms), 3, len(sizes), len(nodes), 4))
        mism = np.argwhere((got != cache[key]).any(axis=-1))
        assert len(mism) == 0, (platforms, mism[:10])
    lib.ofi_amd_tuner_plan_destroy(plan)


def test_bad_arguments(lib, gpu):
    colls, sizes, nodes, ppn, algos = synthetic.tuner_axes()
    plan = ctypes.c_void_p()
    bad_coll = np.array([9], dtype=np.int32)
    assert lib.ofi_amd_tuner_plan_create(bad_coll.ctypes.data, 1, sizes.ctypes.data, 140, nodes.ctypes.data,
                                         11, ppn.ctypes.data, 4, algos.ctypes.data, 3, ctypes.byref(plan)) < 0
    zero_nodes = np.array([0], dtype=np.uint64)
    assert lib.ofi_amd_tuner_plan_create(colls.ctypes.data, 3, sizes.ctypes.data, 140, zero_nodes.ctypes.data,
                                         1, ppn.ctypes.data, 4, algos.ctypes.data, 3, ctypes.byref(plan)) < 0
    plan = make_plan(lib, colls, sizes, nodes, ppn, algos)
    v = (m.TunerVariant * 1)(m.TunerVariant(4, 1, 8, 3))
    assert lib.ofi_amd_tuner_model_grid(plan, v, 1, None, None, None) < 0       # unknown platform
    assert lib.ofi_amd_tuner_region_grid(plan, np.array([7], np.int32).ctypes.data, 1, 1, None) < 0
    lib.ofi_amd_tuner_plan_destroy(plan)
