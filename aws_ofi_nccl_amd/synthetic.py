"""Seeded synthetic inputs for the four hot-path workloads (numpy, host side).

These only *generate inputs*; they compute nothing of the hot path.  The same
arrays are handed to the HIP library and, in tests, to the CPU oracle.
"""
import numpy as np

MASK64 = (1 << 64) - 1


def _mix64(z):
    """splitmix64 finaliser on a uint64 array."""
    z = z.copy()
    z ^= z >> np.uint64(30)
    z *= np.uint64(0xBF58476D1CE4E5B9)
    z ^= z >> np.uint64(27)
    z *= np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    return z


def counter_random(seed, n, stream=0):
    """n uint64 values: mix64(seed + golden * (stream * 2^40 + i + 1))."""
    with np.errstate(over="ignore"):
        ctr = np.arange(1, n + 1, dtype=np.uint64) + np.uint64((stream << 40) & MASK64)
        return _mix64(np.uint64(seed & MASK64) + np.uint64(0x9E3779B97F4A7C15) * ctr)


def log_uniform_sizes(seed, n, lo_log2, hi_log2):
    """Integer log-uniform sizes in [2^lo, 2^hi): uniform octave, uniform within the octave."""
    r = counter_random(seed, n, stream=1)
    e = (np.uint64(lo_log2) + (r & np.uint64(0xFF)) % np.uint64(hi_log2 - lo_log2)).astype(np.uint64)
    one = np.uint64(1)
    return (one << e) | ((r >> np.uint64(8)) & ((one << e) - one))


def stripe_sizes(seed, n):
    """Striping workload: n message sizes log-uniform in [1 B, 256 MiB)."""
    return log_uniform_sizes(seed, n, 0, 28)


def bounce_workload(seed, n=65536, max_len=8192, arena_bytes=2 << 30):
    """Eager-buffer batch: lengths uniform in [0, max_len], packed source offsets,
    disjoint 64-byte-aligned destinations scattered over the arena."""
    rng = np.random.Generator(np.random.PCG64(seed))
    length = rng.integers(0, max_len + 1, size=n, dtype=np.uint32)
    src_off = np.zeros(n, dtype=np.uint64)
    np.cumsum(length[:-1], out=src_off[1:], dtype=np.uint64)
    total = int(length.sum(dtype=np.uint64))
    slots = np.maximum(1, (length.astype(np.int64) + 63) // 64)
    arena_slots = arena_bytes // 64
    free = arena_slots - int(slots.sum())
    if free < 0:
        raise ValueError("arena too small for %d buffers" % n)
    order = rng.permutation(n)
    # random gaps before each buffer (in slots), total <= free
    cuts = np.sort(rng.integers(0, free + 1, size=n, dtype=np.int64))
    gaps = np.diff(np.concatenate(([0], cuts)))
    placed = np.cumsum(slots[order] + gaps) - slots[order]
    dst_off = np.empty(n, dtype=np.uint64)
    dst_off[order] = (placed * 64).astype(np.uint64)
    return {"len": length, "src_off": src_off, "dst_off": dst_off, "src_bytes": total,
            "arena_bytes": arena_bytes}


def random_bytes(seed, nbytes):
    rng = np.random.Generator(np.random.PCG64(seed ^ 0x5EED))
    return rng.integers(0, 256, size=nbytes, dtype=np.uint8)


def tuner_axes():
    """Tuner grid axes: 140 sizes round(2^(k/4)), nodes 1..1024, ranks/node {1,2,4,8}."""
    sizes = np.array([int(round(2.0 ** (k / 4.0))) for k in range(140)], dtype=np.uint64)
    nodes = np.array([1 << k for k in range(11)], dtype=np.uint64)
    ppn = np.array([1, 2, 4, 8], dtype=np.uint32)
    colls = np.array([4, 2, 3], dtype=np.int32)   # AllReduce, AllGather, ReduceScatter
    algos = np.array([1, 0, 6], dtype=np.int32)   # Ring, Tree, PAT
    return colls, sizes, nodes, ppn, algos
