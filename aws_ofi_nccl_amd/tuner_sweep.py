"""Tuner decision sweep: where, along the message-size axis, the tuner changes its answer.

Host-side counterpart of the reference's `show-tuner-decisions` tool
(contrib/python/ofi_nccl/tuner/cli/wrapper.py:57-229, main.py:13-69), same classes, method
names, defaults and output columns.  The reference asks the plugin one (collective, size)
question per ctypes call and bisects the size range recursively; here every round of the
bisection -- for all collectives, shapes and platforms at once -- is one batched GPU query
(`ofi_amd_tuner_query`), so a full sweep is a few dozen launches instead of hundreds of
thousands of calls.  The edge lists are the ones the recursive bisection produces.

    python -m aws_ofi_nccl_amd.tuner_sweep show-all [--max-ranks-per-node 8] [--show-channels]
"""
import argparse
import ctypes
import math
import sys
from enum import Enum

import aws_ofi_nccl_amd as _m


class NCCLFunc(int, Enum):          # wrapper.py:23-32
    Broadcast = 0
    Reduce = 1
    AllGather = 2
    ReduceScatter = 3
    AllReduce = 4
    SendRecv = 5
    Send = 6


class NCCLAlgo(int, Enum):          # wrapper.py:35-42
    TREE = 0
    RING = 1
    COLLNET_DIRECT = 2
    COLLNET_CHAIN = 3
    NVLS = 4
    NVLS_TREE = 5
    PAT = 6


class NCCLProto(int, Enum):         # wrapper.py:45-48
    LL = 0
    LL128 = 1
    SIMPLE = 2


class TunerPlatform(str, Enum):     # wrapper.py:50-54
    P5en = "p5en.48xlarge"
    P5 = "p5.48xlarge"
    P6 = "p6-b200.48xlarge"
    P6_B300 = "p6-b300.48xlarge"


# enum nccl_ofi_tuner_platform (include/tuner/nccl_ofi_tuner_common.h:18-25)
_PLATFORM_ID = {TunerPlatform.P5: 0, TunerPlatform.P5en: 1, TunerPlatform.P6: 2, TunerPlatform.P6_B300: 3}
_ALL_CELLS = (1 << (len(NCCLAlgo) * len(NCCLProto))) - 1     # the tool offers every cell (fill 1337)
_NO_DECISION = {"algo": math.nan, "proto": math.nan, "nchannels": math.nan}


def gpu_backend(questions):
    """[(platform id, coll, nbytes, nranks, nnodes)] -> [(algo, proto, nchannels)] on the GPU."""
    lib = _m.load()
    n = len(questions)
    if n == 0:
        return []
    q = (_m.TunerQuery * n)()
    for i, (plat, coll, nbytes, nranks, nnodes) in enumerate(questions):
        q[i] = _m.TunerQuery(plat, 0, coll, 1, 8, 3, 0, 0, _ALL_CELLS, 0, nbytes, nranks, nnodes)
    a = (_m.TunerAnswer * n)()
    _m.check(lib.ofi_amd_tuner_query(ctypes.cast(q, ctypes.c_void_p), n, ctypes.cast(a, ctypes.c_void_p)),
             "ofi_amd_tuner_query")
    return [(a[i].algo, a[i].proto, a[i].nchannels) for i in range(n)]


class Tuner:
    """One communicator shape on one platform (wrapper.py:57-229).  Answers come from a
    cache that `Sweep` fills in batches; `get_coll_info` on its own asks for one."""

    def __init__(self, nranks, nnodes, platform, backend=gpu_backend):
        self.nranks, self.nnodes, self.platform = nranks, nnodes, TunerPlatform(platform)
        self._backend = backend
        self._cache = {}

    def _key(self, coll_type, msg_size):
        return (_PLATFORM_ID[self.platform], int(coll_type), int(msg_size), self.nranks, self.nnodes)

    @staticmethod
    def _decision(answer):
        algo, proto, nchannels = answer
        if algo < 0:
            return dict(_NO_DECISION)
        # the reference reports nChannels as the plugin left it: 0 from the caller's initial value
        return {"algo": NCCLAlgo(algo), "proto": NCCLProto(proto), "nchannels": max(int(nchannels), 0)}

    def get_coll_info(self, coll_type, msg_size, num_pipe_ops=1):
        key = self._key(coll_type, msg_size)
        if key not in self._cache:
            self._cache[key] = self._decision(self._backend([key])[0])
        return self._cache[key]

    def _bisect(self, coll_type, min_size, max_size, missing):
        """wrapper.py:186-204, except that an unanswered question stops the descent and is noted."""
        lo_key, hi_key = self._key(coll_type, min_size), self._key(coll_type, max_size)
        lo, hi = self._cache.get(lo_key), self._cache.get(hi_key)
        if lo is None:
            missing.add(lo_key)
        if hi is None:
            missing.add(hi_key)
        if lo is None or hi is None:
            return None
        if (_same(lo, hi) and math.log2(max_size) - math.log2(min_size) <= 1) or max_size - min_size <= 1:
            return [(min_size, lo), (max_size, hi)]
        mid_size = (min_size + max_size) // 2
        left = self._bisect(coll_type, min_size, mid_size, missing)
        right = self._bisect(coll_type, mid_size, max_size, missing)
        if left is None or right is None:
            return None
        combined = left + right[1:]
        return [combined[0]] + [combined[i] for i in range(1, len(combined))
                                if not _same(combined[i][1], combined[i - 1][1])]

    def _rows(self, coll_type, edges):
        return [{"collective": coll_type.name, "message_size": size, "algo": d["algo"], "proto": d["proto"],
                 "nchannels": d["nchannels"], "ranks": self.nranks, "nodes": self.nnodes,
                 "platform": self.platform} for size, d in edges]

    def analyze_message_range(self, coll_type, min_size, max_size):
        return Sweep([self], self._backend).run([coll_type], min_size, max_size)

    def analyze_all(self, min_size=32, max_size=32 * 1024 * 1024 * 1024):
        return Sweep([self], self._backend).run(list(NCCLFunc), min_size, max_size)


def _same(a, b):
    """Dict equality, as the reference compares decisions: values that are the same object
    compare equal, so two 'no decision' results (the one NaN object) do merge."""
    return a == b


class Sweep:
    """Bisection of many (tuner, collective) ranges in lock step: one batched query per round."""

    def __init__(self, tuners, backend=gpu_backend):
        self.tuners, self.backend = list(tuners), backend
        self.rounds = self.questions = 0

    def run(self, colls=None, min_size=32, max_size=32 * 1024 * 1024 * 1024):
        colls = list(NCCLFunc) if colls is None else colls
        open_tasks = [(t, c) for t in self.tuners for c in colls]
        edges = {}
        while open_tasks:
            missing, still_open = set(), []
            for t, c in open_tasks:
                e = t._bisect(c, min_size, max_size, missing)
                if e is None:
                    still_open.append((t, c))
                else:
                    edges[(id(t), c)] = e
            if missing:
                keys = sorted(missing)
                answers = self.backend(keys)
                self.rounds += 1
                self.questions += len(keys)
                by_shape = {}
                for t in self.tuners:
                    by_shape.setdefault((_PLATFORM_ID[t.platform], t.nranks, t.nnodes), []).append(t)
                for key, ans in zip(keys, answers):
                    for t in by_shape[(key[0], key[3], key[4])]:
                        t._cache[key] = Tuner._decision(ans)
            open_tasks = still_open
        rows = []
        for t in self.tuners:
            for c in colls:
                rows += t._rows(c, edges[(id(t), c)])
        return rows


def show_all(min_ranks_per_node=1, max_ranks_per_node=64, inc_ranks_per_node=1, min_nnodes=2,
             max_nnodes=int(math.log2(2048)), inc_nnodes=2, show_channels=False, backend=gpu_backend,
             out=sys.stdout):
    """main.py:28-69: every platform x node count x ranks per node; prints one table per collective."""
    tuners = [Tuner(rpn * nodes, nodes, platform, backend)
              for nodes in range(min_nnodes, max_nnodes + 1, inc_nnodes)
              for rpn in range(min_ranks_per_node, max_ranks_per_node + 1, inc_ranks_per_node)
              for platform in TunerPlatform]
    sweep = Sweep(tuners, backend)
    rows = [r for r in sweep.run() if not (isinstance(r["algo"], float) and math.isnan(r["algo"]))]  # dropna
    index = ["nodes", "ranks", "message_size"] + (["nchannels"] if show_channels else [])
    rows.sort(key=lambda r: tuple(r[k] for k in index))
    cols = index + [c for c in ("collective", "algo", "proto", "nchannels", "platform") if c not in index]
    for collective in sorted({r["collective"] for r in rows}):
        print(" ".join("%-14s" % c for c in cols), file=out)
        for r in rows:
            if r["collective"] != collective:
                continue
            shown = dict(r, algo=r["algo"].name.title(), proto=r["proto"].name.title(),
                         platform=r["platform"].name)
            print(" ".join("%-14s" % shown[c] for c in cols), file=out)
    print("# %d questions in %d batched rounds" % (sweep.questions, sweep.rounds), file=out)
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(prog="show-tuner-decisions")
    sub = ap.add_subparsers(dest="cmd", required=True)
    sa = sub.add_parser("show-all")
    sa.add_argument("--min-ranks-per-node", type=int, default=1)
    sa.add_argument("--max-ranks-per-node", type=int, default=64)
    sa.add_argument("--inc-ranks-per-node", type=int, default=1)
    sa.add_argument("--min-nnodes", type=int, default=2)
    sa.add_argument("--max-nnodes", type=int, default=int(math.log2(2048)))
    sa.add_argument("--inc-nnodes", type=int, default=2)
    sa.add_argument("--show-channels", action="store_true")
    args = ap.parse_args(argv)
    _m.check(_m.load().ofi_amd_gpu_init(), "ofi_amd_gpu_init")
    show_all(args.min_ranks_per_node, args.max_ranks_per_node, args.inc_ranks_per_node, args.min_nnodes,
             args.max_nnodes, args.inc_nnodes, args.show_channels)
    return 0


if __name__ == "__main__":
    sys.exit(main())
