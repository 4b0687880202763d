"""Launches one kernel of the library on one named input shape, a fixed number of times.

For profilers: `rocprofv3 --kernel-trace --stats -- python3 -m aws_ofi_nccl_amd.kernel_shapes
--kernel bounce --shape configured --launches 30` sees 30 dispatches of bounce_scatter_kernel and
nothing else of interest, which keeps counter runs short.  The shapes:

  bounce    configured   65,536 buffers, lengths uniform 0..8,192 B, packed source (any byte
                         alignment), 64-byte-aligned destinations scattered over 2 GiB
            aligned8k    --buffers (default 65,536) buffers of exactly 8,192 B, sources 8 KiB
                         apart, the same kind of scattered destinations (what the length and
                         alignment mix costs); 32,768 buffers move the configured batch's bytes
            dense8k      the same with destination i right behind destination i-1 (what the
                         scatter costs)
  copy      payload      a plain device-to-device copy of the configured payload (268,444,074 B):
                         the reference point that scales FETCH_SIZE / WRITE_SIZE
  fill      <MiB>        torch's fill of that many MiB (default 100): what the chip sustains when a
                         kernel only writes
  table     <MiB>        --buffers (default 64) copies of that many MiB each (default 16), sources and
                         destinations 4 KiB-aligned and apart: whole entries through
                         ofi_amd_copy_table_pieces (a wavefront per 8 KiB), or with --cut the same
                         bytes as 256 KiB entries through ofi_amd_copy_table (a wavefront per entry)
  striping  1m | 16m     1,000,000 / 16,000,000 message sizes, 4 rails
  model     64 | 256     tuner cost-model grids per launch
  region    64           tuner region grids per launch
  eager     configured   65,536 rx buffers of 8,320 B, payloads 0..8,184 B, taken in a random
                         order of slots, destinations at any byte alignment
            slots        the same with the rx buffers taken in slot order
            align<N>     the same as configured with every destination a multiple of N bytes
                         (N = 16, 64 or 128); "slots+align<N>" combines the two
"""
import argparse
import ctypes
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 1234


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--kernel", required=True, choices=["bounce", "copy", "fill", "table", "striping", "model", "region", "eager"])
    ap.add_argument("--shape", default=None)
    ap.add_argument("--launches", type=int, default=30)
    ap.add_argument("--buffers", type=int, default=None,
                    help="bounce aligned8k / dense8k: buffer count (default 65,536); table: entries (default 64)")
    ap.add_argument("--cut", action="store_true", help="table: 256 KiB entries, one wavefront each")
    ap.add_argument("--no-flush", action="store_true", help="bounce / eager: no read-back")
    ap.add_argument("--graph", action="store_true",
                    help="record one call into a HIP graph and replay it --launches times")
    ap.add_argument("--busy-seconds", type=float, default=0.0,
                    help="before the launches, keep the device busy this long with plain device copies of 256 MiB "
                         "(another kernel, so that a profiler filtering by kernel name counts only the launches)")
    ap.add_argument("--per-launch", action="store_true",
                    help="an event between every two launches: prints the median launch period of the first 100, "
                         "of every tenth of the run and of the last 1,000 (how the rate moves while the device "
                         "stays busy)")
    args = ap.parse_args()

    import numpy as np
    import torch
    sys.path.insert(0, ROOT)
    import aws_ofi_nccl_amd as m
    from aws_ofi_nccl_amd import synthetic

    lib = m.load()
    m.check(lib.ofi_amd_gpu_init(), "ofi_amd_gpu_init")
    torch.cuda.init()
    side = torch.cuda.Stream()
    torch.cuda.set_stream(side)  # a stream of its own: graphs cannot be recorded on the default one
    stream = ctypes.c_void_p(side.cuda_stream)

    def dev(a):
        signed = {np.dtype(np.uint8): np.uint8, np.dtype(np.uint32): np.int32, np.dtype(np.uint64): np.int64}
        a = np.ascontiguousarray(a)
        return torch.from_numpy(a.view(signed.get(a.dtype, a.dtype))).cuda()

    keep = []
    if args.kernel in ("bounce", "copy"):
        shape = args.shape or ("payload" if args.kernel == "copy" else "configured")
        w = synthetic.bounce_workload(SEED)
        n = len(w["len"])
        if shape in ("aligned8k", "dense8k"):
            n = args.buffers or 65536
            if not 0 < n <= (2 << 30) // 8192:
                ap.error("--buffers out of range")
            length = np.full(n, 8192, dtype=np.uint32)
            src_off = np.arange(n, dtype=np.uint64) * np.uint64(8192)
            if shape == "dense8k":
                dst_off = np.arange(n, dtype=np.uint64) * np.uint64(8192)
            else:
                rng = np.random.Generator(np.random.PCG64(SEED))
                slots = rng.permutation((2 << 30) // 8192)[:n].astype(np.uint64)
                dst_off = slots * np.uint64(8192)
            w = {"len": length, "src_off": src_off, "dst_off": dst_off, "src_bytes": n * 8192,
                 "arena_bytes": 2 << 30}
        elif shape not in ("configured", "payload"):
            ap.error("unknown shape")
        d_src = torch.randint(0, 255, (w["src_bytes"] + 64,), dtype=torch.uint8, device="cuda")
        if args.kernel == "copy":
            d_dst = torch.empty(w["src_bytes"], dtype=torch.uint8, device="cuda")
            step = lambda: d_dst.copy_(d_src[:w["src_bytes"]])
        else:
            d_arena = torch.zeros(w["arena_bytes"], dtype=torch.uint8, device="cuda")
            d_so, d_do, d_len = dev(w["src_off"]), dev(w["dst_off"]), dev(w["len"])
            d_flush = torch.zeros(n, dtype=torch.int32).pin_memory()
            keep += [d_arena, d_so, d_do, d_len, d_flush]
            flush = None if args.no_flush else d_flush.data_ptr()
            step = lambda: m.check(lib.ofi_amd_bounce_scatter(
                d_src.data_ptr(), d_src.numel(), d_arena.data_ptr(), w["arena_bytes"], d_so.data_ptr(),
                d_do.data_ptr(), d_len.data_ptr(), n, flush, stream), "bounce_scatter")
        print("payload bytes per launch: %d, buffers: %d" % (w["src_bytes"], n))
    elif args.kernel == "fill":
        d_fill = torch.empty(int(args.shape or "100") << 20, dtype=torch.uint8, device="cuda")
        step = lambda: d_fill.fill_(7)
        print("bytes written per launch: %d" % d_fill.numel())
    elif args.kernel == "table":
        entries, each = args.buffers or 64, int(args.shape or "16") << 20
        if not 0 < entries * each <= 64 << 30:
            ap.error("--buffers x --shape out of range")
        d_from = torch.randint(0, 255, (entries * each,), dtype=torch.uint8, device="cuda")
        d_to = torch.zeros(entries * each, dtype=torch.uint8, device="cuda")
        piece = (256 << 10) if args.cut else each
        starts = np.arange(0, entries * each, piece, dtype=np.uint64)
        d_s, d_d = dev(starts + np.uint64(d_from.data_ptr())), dev(starts + np.uint64(d_to.data_ptr()))
        d_l = dev(np.full(len(starts), piece, dtype=np.uint32))
        if args.cut:
            step = lambda: m.check(lib.ofi_amd_copy_table(d_s.data_ptr(), d_d.data_ptr(), d_l.data_ptr(), len(starts),
                                                          stream), "copy_table")
        else:
            step = lambda: m.check(lib.ofi_amd_copy_table_pieces(d_s.data_ptr(), d_d.data_ptr(), d_l.data_ptr(),
                                                                 len(starts), piece, stream), "copy_table_pieces")
        print("bytes copied per launch: %d in %d table entries" % (entries * each, len(starts)))
    elif args.kernel == "eager":
        n, stride = 65536, 8320
        rng = np.random.default_rng(SEED)
        recv_len = rng.integers(0, 8185, n).astype(np.uint32)
        rx_off = rng.permutation(n).astype(np.uint64) * np.uint64(stride)
        dst_off = (np.sort(rng.permutation((2 << 30) // 8448)[:n]).astype(np.uint64) * np.uint64(8448) +
                   rng.integers(0, 64, n).astype(np.uint64))
        for word in (args.shape or "configured").split("+"):
            if word == "slots":
                rx_off = np.arange(n, dtype=np.uint64) * np.uint64(stride)
            elif word in ("align16", "align64", "align128"):
                dst_off &= ~np.uint64(int(word[5:]) - 1)
            elif word != "configured":
                ap.error("unknown shape")
        d_rx = torch.randint(0, 255, (n * stride,), dtype=torch.uint8, device="cuda")
        d_dst = torch.zeros(2 << 30, dtype=torch.uint8, device="cuda")
        d = [dev(x) for x in (rx_off, recv_len, dst_off, recv_len)]
        d_copied = torch.zeros(n, dtype=torch.int32, device="cuda")
        d_flush = torch.zeros(n, dtype=torch.int32, device="cuda")
        flush = None if args.no_flush else d_flush.data_ptr()
        step = lambda: m.check(lib.ofi_amd_eager_copy_batch(
            d_rx.data_ptr(), d[0].data_ptr(), d[1].data_ptr(), d_dst.data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
            n, d_copied.data_ptr(), flush, stream), "eager_copy_batch")
        print("payload bytes per launch: %d" % int(recv_len.sum()))
    elif args.kernel == "striping":
        n = {"1m": 1_000_000, "16m": 16_000_000}[args.shape or "1m"]
        sizes = synthetic.stripe_sizes(SEED, n)
        st = m.SchedState(0, 0, 64, 131072, 4, 0)
        d_state = dev(np.frombuffer(bytes(st), dtype=np.uint8).copy())
        d_sizes = dev(sizes)
        d_num = torch.zeros(n, dtype=torch.int32, device="cuda")
        d_xf = torch.zeros(n * 12, dtype=torch.int64, device="cuda")
        step = lambda: m.check(lib.ofi_amd_sched_batch(d_state.data_ptr(), d_sizes.data_ptr(), n, 128,
                                                       d_num.data_ptr(), d_xf.data_ptr(), stream), "sched_batch")
    else:
        colls, sizes, nodes, ppn, algos = synthetic.tuner_axes()
        plan = ctypes.c_void_p()
        m.check(lib.ofi_amd_tuner_plan_create(colls.ctypes.data, len(colls), sizes.ctypes.data, len(sizes),
                                              nodes.ctypes.data, len(nodes), ppn.ctypes.data, len(ppn),
                                              algos.ctypes.data, len(algos), ctypes.byref(plan)), "plan_create")
        points, cells = lib.ofi_amd_tuner_plan_points(plan), lib.ofi_amd_tuner_plan_cells(plan)
        nv = int(args.shape or "64")
        if args.kernel == "model":
            variants = (m.TunerVariant * nv)(*[m.TunerVariant(i % 2, 1 + (i // 2) % 32, 8 + i // 64, 3)
                                               for i in range(nv)])
            d_cost = torch.zeros(nv * cells, dtype=torch.float64, device="cuda")
            d_choice = torch.zeros(nv * points * 2, dtype=torch.int8, device="cuda")
            step = lambda: m.check(lib.ofi_amd_tuner_model_grid(plan, variants, nv, d_cost.data_ptr(),
                                                                d_choice.data_ptr(), stream), "model_grid")
        else:
            plats = np.array([i % 4 for i in range(nv)], dtype=np.int32)
            d_reg = torch.zeros(nv * points * 4, dtype=torch.int8, device="cuda")
            step = lambda: m.check(lib.ofi_amd_tuner_region_grid(plan, plats.ctypes.data, nv, d_reg.data_ptr(),
                                                                 stream), "region_grid")
        print("grids per launch: %d, cost cells per grid: %d, decision points per grid: %d" % (nv, cells, points))

    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    step()  # the first call on a stream may allocate its scratch
    torch.cuda.synchronize()
    if args.graph:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        step = graph.replay
        step()
        torch.cuda.synchronize()
    if args.busy_seconds > 0:
        import time
        d_a = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        d_b = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < args.busy_seconds:
            for _ in range(200):
                d_b.copy_(d_a)
            torch.cuda.synchronize()
    if args.per_launch:
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.launches + 1)]
        marks[0].record()
        for k in range(args.launches):
            step()
            marks[k + 1].record()
        torch.cuda.synchronize()
        us = np.array([marks[k].elapsed_time(marks[k + 1]) * 1e3 for k in range(args.launches)])
        print("%s %s: %d launches back to back, %.2f s; median launch period in us:" % (
            args.kernel, args.shape or "", args.launches, us.sum() / 1e6))
        print("  first %d: %.2f" % (min(100, len(us)), np.median(us[:100])))
        for t in range(10):
            part = us[len(us) * t // 10:len(us) * (t + 1) // 10]
            print("  tenth %d: %.2f (min %.2f, mean %.2f)" % (t + 1, np.median(part), part.min(), part.mean()))
        print("  last %d: %.2f" % (min(1000, len(us)), np.median(us[-1000:])))
        return 0
    e0.record()
    for _ in range(args.launches):
        step()
    e1.record()
    torch.cuda.synchronize()
    print("%s %s%s: %d launches, %.2f us each by HIP events" % (
        args.kernel, args.shape or "", " (graph replays)" if args.graph else "", args.launches,
        e0.elapsed_time(e1) * 1e3 / args.launches))
    return 0


if __name__ == "__main__":
    sys.exit(main())
