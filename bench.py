"""Benchmark of the hot path on one MI355X.

Default workload: ring all-reduce, sum, fp32, 8 simulated ranks x 256 MiB per rank, out of place
(BASELINE.json configs[1] at its largest size).  A "step" is one complete collective (one call per
rank).  Prints one JSON line.

The headline (`value`, `ms_per_step`, `roofline`) is the library's default mode: the fused single pass (one
launch of TeamChainKernel<float, sum>: the workgroups of an XCD read their tiles together, hold the results in LDS
and write them together) that reads every rank's input once, combines in the ring schedule's order and writes
every rank's output once -- 2 * p * S algorithmic bytes per collective, bit for bit the schedule's result.
The schedule run step by step (library setting fuse=0: one launch per phase of copy / reduce steps, replayed from a
HIP graph, 5 * (p - 1) * S bytes, 1.9 times slower per collective) is timed in the same run and reported under
`config.step_by_step` and `roofline_steps`; part of what its phases read comes out of the 256 MB memory-side cache,
so its rate is not a DRAM rate.

    python bench.py [--steps K] [--warmup W] [--size-mib M] [--sweep] [--suite] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
METRIC = "achieved HBM GB/s & % of peak, 8-rank fp32 ring AllReduce 256MiB/rank"

PROFILE_FUSED = os.path.join(ROOT, "profiles", "TeamChainKernel_fp32_sum__ring_allreduce_8ranks_256MiB.txt")
PROFILE_STEPS = os.path.join(ROOT, "profiles", "StepKernel_fp32_sum__ring_allreduce_8ranks_256MiB.txt")


def profiled_traffic(path):
    """Bytes per launch between L2 and the fabric that the committed rocprofv3 --pmc summary of the default workload
    reports (its line `traffic_bytes_per_launch = N`: FETCH_SIZE and WRITE_SIZE scaled by a plain copy of known
    size in the same runs).  None when the summary is absent or has no such line."""
    try:
        with open(path) as f:
            for line in f:
                if line.strip().startswith("traffic_bytes_per_launch"):
                    return int(line.split("=", 1)[1].split()[0].replace("_", ""))
    except (OSError, ValueError, IndexError):
        pass
    return None


def run_mode(pkg, torch, comms, stream, sends, recvs, n, fuse, steps, warmup):
    pkg.set_param(comms[0], "fuse", fuse)
    sp = [t.data_ptr() for t in sends]
    rp = [t.data_ptr() for t in recvs]
    dt, op = pkg.HCCL_DATA_TYPE_FP32, pkg.HCCL_REDUCE_SUM
    for _ in range(warmup):
        pkg.all_reduce(comms, sp, rp, n, dt, op, stream.cuda_stream)
    stream.synchronize()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        e0.record(stream)
        for _ in range(steps):
            pkg.all_reduce(comms, sp, rp, n, dt, op, stream.cuda_stream)
        e1.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = e0.elapsed_time(e1) / steps
    info = pkg.last_op_info(comms[0])
    return wall_ms, dev_ms, info


def per_launch_times(pkg, torch, comms, stream, sends, recvs, n, fuse, steps):
    """Median and minimum device time of single collectives (one event pair each), in ms."""
    pkg.set_param(comms[0], "fuse", fuse)
    sp = [t.data_ptr() for t in sends]
    rp = [t.data_ptr() for t in recvs]
    dt, op = pkg.HCCL_DATA_TYPE_FP32, pkg.HCCL_REDUCE_SUM
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    with torch.cuda.stream(stream):
        for e0, e1 in pairs:
            e0.record(stream)
            pkg.all_reduce(comms, sp, rp, n, dt, op, stream.cuda_stream)
            e1.record(stream)
    stream.synchronize()
    ts = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return ts[len(ts) // 2], ts[0]


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def time_calls(torch, stream, call, steps, warmup):
    for _ in range(warmup):
        call()
    stream.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(steps):
        call()
    e1.record(stream)
    stream.synchronize()
    return e0.elapsed_time(e1) / steps


def run_suite(pkg, torch, steps, warmup, only="", settings=()):
    """The other configurations of BASELINE.json (reduce-scatter op x type matrix, 16-rank all-to-all-v,
    halving-doubling all-reduce in bf16 at 32 and 24 ranks, all-gather) and the rest of the API (mesh and
    halving-doubling all-reduce, rooted collectives, uniform all-to-all, send / receive), fused and step-by-step:
    a table on stderr."""
    import numpy as np
    stream = torch.cuda.Stream()
    out = sys.stderr
    out.write("%-46s %-6s %9s %10s %9s %8s\n" % ("configuration", "mode", "launches", "time_us", "GB/s", "%peak"))

    def report(name, comms, call):
        if only and not any(part in name for part in only.split(",")):
            return
        for kv in settings:
            k, v = kv.split("=", 1)
            pkg.set_param(comms[0], k, v)
        for fuse in (1, 0):
            pkg.set_param(comms[0], "fuse", fuse)
            ms = time_calls(torch, stream, call, steps, warmup)
            info = pkg.last_op_info(comms[0])
            moved = info["bytesRead"] + info["bytesWritten"]
            gbps = moved / (ms * 1e-3) / 1e9
            out.write("%-46s %-6s %9d %10.1f %9.1f %8.1f\n" % (name, "fused" if info["fused"] else "steps", info["launches"],
                                                              ms * 1e3, gbps, 100 * gbps / HBM_PEAK_GBPS))

    dtypes = {"fp16": (pkg.HCCL_DATA_TYPE_FP16, torch.float16), "bf16": (pkg.HCCL_DATA_TYPE_BFP16, torch.bfloat16),
              "int8": (pkg.HCCL_DATA_TYPE_INT8, torch.int8), "int32": (pkg.HCCL_DATA_TYPE_INT32, torch.int32),
              "int64": (pkg.HCCL_DATA_TYPE_INT64, torch.int64), "fp32": (pkg.HCCL_DATA_TYPE_FP32, torch.float32)}
    ops = {"sum": 0, "prod": 1, "max": 2, "min": 3}

    def rand(n, tdt):
        if tdt.is_floating_point:
            return torch.randn(n, dtype=torch.float32, device="cuda").to(tdt)
        if tdt == torch.int64:
            return torch.randint(-(1 << 40), 1 << 40, (n,), dtype=tdt, device="cuda")
        info = torch.iinfo(tdt)
        return torch.randint(info.min, info.max, (n,), dtype=tdt, device="cuda")

    # reduce-scatter, 8 ranks, 64 MiB per rank send buffer
    p = 8
    comms = pkg.comm_init_all(p)
    for tname in ("fp16", "bf16", "int8", "int32", "int64"):
        hdt, tdt = dtypes[tname]
        unit = pkg.DTYPE_SIZE[hdt]
        n = (64 << 20) // unit // p
        sends = [rand(n * p, tdt) for _ in range(p)]
        recvs = [torch.empty(n, dtype=tdt, device="cuda") for _ in range(p)]
        sp, rp = [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs]
        torch.cuda.synchronize()
        for oname, op in ops.items():
            report("reduce-scatter ring p=8 64MiB/rank %s %s" % (tname, oname), comms,
                   lambda: pkg.reduce_scatter(comms, sp, rp, n, hdt, op, stream.cuda_stream))
        del sends, recvs
    # all-gather, 8 ranks, 32 MiB per rank in, 256 MiB per rank out
    n = (32 << 20)
    sends = [rand(n, torch.int8) for _ in range(p)]
    recvs = [torch.empty(n * p, dtype=torch.int8, device="cuda") for _ in range(p)]
    sp, rp = [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs]
    torch.cuda.synchronize()
    report("all-gather ring p=8 32MiB/rank in", comms,
           lambda: pkg.all_gather(comms, sp, rp, n, pkg.HCCL_DATA_TYPE_INT8, stream.cuda_stream))
    del sends, recvs
    pkg.comm_destroy(comms)

    # all-to-all-v, 16 ranks, lognormal counts
    p = 16
    rng = np.random.default_rng(2024)
    cnt = np.clip(np.rint(np.exp(np.log(65536.0) + rng.standard_normal((p, p)))), 0, 4 << 20).astype(np.uint64)
    sdis, rdis = np.zeros((p, p), np.uint64), np.zeros((p, p), np.uint64)
    sl, rl = [], []
    for r in range(p):
        pos = 0
        for j in rng.permutation(p):
            pos += int(rng.integers(0, 1024))
            sdis[r, j] = pos
            pos += int(cnt[r, j])
        sl.append(pos)
        pos = 0
        for i in rng.permutation(p):
            pos += int(rng.integers(0, 1024))
            rdis[r, i] = pos
            pos += int(cnt[i, r])
        rl.append(pos)
    comms = pkg.comm_init_all(p)
    sends = [rand(max(x, 1), torch.int32) for x in sl]
    recvs = [torch.empty(max(x, 1), dtype=torch.int32, device="cuda") for x in rl]
    sp, rp = [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs]
    torch.cuda.synchronize()
    tables = pkg.a2av_tables(cnt, sdis, cnt.T.copy(), rdis)
    report("all-to-all-v pairwise p=16 int32 lognormal (%.0f MB)" % (4 * cnt.sum() / 1e6), comms,
           lambda: pkg.all_to_all_v(comms, sp, None, None, rp, None, None, pkg.HCCL_DATA_TYPE_INT32, stream.cuda_stream,
                                    tables=tables))
    # the same exchange when the tables change on every call (an expert-parallel layer): nothing can be reused, so
    # this is wall time per call, from the first rank's call to completion, one call at a time
    name = "all-to-all-v pairwise p=16 lognormal, new tables every call"
    if not only or any(part in name for part in only.split(",")):
        import time
        sets = []
        for k in range(24):
            rng_k = np.random.default_rng(3000 + k)
            c = np.clip(np.rint(np.exp(np.log(65536.0) + rng_k.standard_normal((p, p)))), 0, 4 << 20).astype(np.uint64)
            sd = np.concatenate([np.zeros((p, 1), np.uint64), np.cumsum(c, axis=1)[:, :-1]], axis=1).astype(np.uint64)
            rc = c.T.copy()
            rd = np.concatenate([np.zeros((p, 1), np.uint64), np.cumsum(rc, axis=1)[:, :-1]], axis=1).astype(np.uint64)
            sets.append((pkg.a2av_tables(c, sd, rc, rd), int(max(c.sum(axis=1).max(), rc.sum(axis=1).max()))))
        longest = max(n for _, n in sets)
        sends2 = [torch.zeros(longest, dtype=torch.int32, device="cuda") for _ in range(p)]
        recvs2 = [torch.zeros(longest, dtype=torch.int32, device="cuda") for _ in range(p)]
        sp2, rp2 = [t.data_ptr() for t in sends2], [t.data_ptr() for t in recvs2]
        for fuse in (1, 0):
            pkg.set_param(comms[0], "fuse", fuse)
            walls = []
            for tabs, _ in sets:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                pkg.all_to_all_v(comms, sp2, None, None, rp2, None, None, pkg.HCCL_DATA_TYPE_INT32, stream.cuda_stream, tables=tabs)
                stream.synchronize()
                walls.append(time.perf_counter() - t0)
            if len(walls) > 4:
                info = pkg.last_op_info(comms[0])
                out.write("%-46s %-6s %9d %10.1f %9s %8s   (wall, median of %d calls, all cache misses: hit=%d)\n" % (
                    name, "fused" if info["fused"] else "steps", info["launches"], 1e6 * float(np.median(walls[2:])), "-", "-",
                    len(walls) - 2, info["cacheHit"]))
        del sends2, recvs2
    pkg.set_param(comms[0], "servers", 2)
    report("all-to-all-v staged 2x8 p=16 int32 lognormal (%.0f MB)" % (4 * cnt.sum() / 1e6), comms,
           lambda: pkg.all_to_all_v(comms, sp, None, None, rp, None, None, pkg.HCCL_DATA_TYPE_INT32, stream.cuda_stream,
                                    tables=tables))
    del sends, recvs
    pkg.comm_destroy(comms)

    # the same with segments below a KiB: counts lognormal(ln 64, 1) elements, ragged displacements
    for p in (16, 64):
        rng = np.random.default_rng(2025 + p)
        cnt = np.clip(np.rint(np.exp(np.log(64.0) + rng.standard_normal((p, p)))), 0, 4 << 20).astype(np.uint64)
        sdis, rdis = np.zeros((p, p), np.uint64), np.zeros((p, p), np.uint64)
        sl, rl = [], []
        for r in range(p):
            pos = 0
            for j in rng.permutation(p):
                pos += int(rng.integers(0, 16))
                sdis[r, j] = pos
                pos += int(cnt[r, j])
            sl.append(pos)
            pos = 0
            for i in rng.permutation(p):
                pos += int(rng.integers(0, 16))
                rdis[r, i] = pos
                pos += int(cnt[i, r])
            rl.append(pos)
        comms = pkg.comm_init_all(p)
        sends = [rand(max(x, 1), torch.int32) for x in sl]
        recvs = [torch.empty(max(x, 1), dtype=torch.int32, device="cuda") for x in rl]
        sp, rp = [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs]
        torch.cuda.synchronize()
        tables = pkg.a2av_tables(cnt, sdis, cnt.T.copy(), rdis)
        report("all-to-all-v pairwise p=%d int32 small segments (%.0f KB)" % (p, 4 * cnt.sum() / 1e3), comms,
               lambda: pkg.all_to_all_v(comms, sp, None, None, rp, None, None, pkg.HCCL_DATA_TYPE_INT32, stream.cuda_stream,
                                        tables=tables))
        del sends, recvs
        pkg.comm_destroy(comms)

    # halving-doubling all-reduce, bf16, 128 MiB per rank, 32 and 24 ranks
    for p in (32, 24):
        comms = pkg.comm_init_all(p)
        pkg.set_param(comms[0], "algo", "rhd")
        n = (128 << 20) // 2
        sends = [rand(n, torch.bfloat16) for _ in range(p)]
        recvs = [torch.empty(n, dtype=torch.bfloat16, device="cuda") for _ in range(p)]
        sp, rp = [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs]
        torch.cuda.synchronize()
        report("all-reduce rhd p=%d bf16 sum 128MiB/rank" % p, comms,
               lambda: pkg.all_reduce(comms, sp, rp, n, pkg.HCCL_DATA_TYPE_BFP16, 0, stream.cuda_stream))
        del sends, recvs
        pkg.comm_destroy(comms)

    # the widened API: mesh / halving-doubling all-reduce, rooted collectives, uniform all-to-all, send / receive
    p = 8
    n = (256 << 20) // 4
    sends = [rand(n, torch.float32) for _ in range(p)]
    recvs = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(p)]
    sp, rp = [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs]
    FP32 = pkg.HCCL_DATA_TYPE_FP32
    for algo, det in (("mesh", 1), ("mesh", 0), ("rhd", 0)):
        comms = pkg.comm_init_all(p)
        pkg.set_param(comms[0], "algo", algo)
        pkg.set_param(comms[0], "deterministic", det)
        torch.cuda.synchronize()
        label = algo + (" (piece cut)" if (algo, det) == ("mesh", 1) else " (uncut)" if algo == "mesh" else "")
        report("all-reduce %s p=8 fp32 sum 256MiB/rank" % label, comms,
               lambda: pkg.all_reduce(comms, sp, rp, n, FP32, 0, stream.cuda_stream))
        for ralgo in (("ring", "mesh", "rhd") if (algo, det) == ("mesh", 0) else ()):
            pkg.set_param(comms[0], "algo", ralgo)
            report("reduce %s p=8 fp32 sum 256MiB/rank root 3" % ralgo, comms,
                   lambda: pkg.reduce(comms, sp, rp, n, FP32, 0, 3, stream.cuda_stream))
            if ralgo != "rhd":
                report("broadcast %s p=8 256MiB root 3" % ralgo, comms,
                       lambda: pkg.broadcast(comms, rp, n, FP32, 3, stream.cuda_stream))
        pkg.comm_destroy(comms)
    # in place (send buffer == receive buffer on every rank).  max rather than sum: replays feed on their own
    # output, which a sum would drive to infinity; after the first call the buffers hold full-entropy data
    comms = pkg.comm_init_all(p)
    for r in range(p):
        recvs[r].copy_(sends[r])
    torch.cuda.synchronize()
    report("all-reduce ring p=8 fp32 max 256MiB/rank in place", comms,
           lambda: pkg.all_reduce(comms, rp, rp, n, FP32, 2, stream.cuda_stream))
    report("all-reduce ring p=8 fp32 max 256MiB/rank out of place", comms,
           lambda: pkg.all_reduce(comms, sp, rp, n, FP32, 2, stream.cuda_stream))
    pkg.comm_destroy(comms)
    for servers, level0, level1 in ((2, "mesh", "ring"), (2, "mesh", "rhd"), (4, "mesh", "rhd"), (2, "ring", "rhd"), (1, "ring4", "rhd")):
        comms = pkg.comm_init_all(p)
        pkg.set_param(comms[0], "servers", servers)
        pkg.set_param(comms[0], "level0", level0)
        pkg.set_param(comms[0], "algo", level1)
        torch.cuda.synchronize()
        report("all-reduce two-level %dx%d %s+%s fp32 sum 256MiB/rank" % (servers, p // servers, level0, level1), comms,
               lambda: pkg.all_reduce(comms, sp, rp, n, FP32, 0, stream.cuda_stream))
        pkg.comm_destroy(comms)
    comms = pkg.comm_init_all(p)
    pkg.set_param(comms[0], "servers", 2)
    report("reduce-scatter two-level 2x4 rhd+mesh fp32 sum 256MiB/rank in", comms,
           lambda: pkg.reduce_scatter(comms, sp, rp, n // p, FP32, 0, stream.cuda_stream))
    pkg.comm_destroy(comms)
    comms = pkg.comm_init_all(p)
    pkg.set_param(comms[0], "servers", 2)
    report("all-gather two-level 2x4 mesh+rhd 32MiB/rank in", comms,
           lambda: pkg.all_gather(comms, sp, rp, n // p, FP32, stream.cuda_stream))
    pkg.comm_destroy(comms)
    comms = pkg.comm_init_all(p)
    pkg.set_param(comms[0], "servers", 2)
    report("reduce two-level 2x4 mesh+rhd fp32 sum 256MiB/rank root 3", comms,
           lambda: pkg.reduce(comms, sp, rp, n, FP32, 0, 3, stream.cuda_stream))
    pkg.comm_destroy(comms)
    comms = pkg.comm_init_all(p)
    m = n // p
    report("scatter mesh p=8 32MiB/rank root 3", comms,
           lambda: pkg.scatter(comms, sp, rp, m, FP32, 3, stream.cuda_stream))
    report("all-to-all uniform p=8 32MiB/pair", comms,
           lambda: pkg.all_to_all(comms, sp, rp, m, FP32, stream.cuda_stream))

    def sendrecv():
        pkg.send(comms[1], sp[1], n, FP32, 5, stream.cuda_stream)
        pkg.recv(comms[5], rp[5], n, FP32, 1, stream.cuda_stream)
    report("send/recv rank 1 -> 5 256MiB", comms, sendrecv)
    del sends, recvs
    pkg.comm_destroy(comms)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size-mib", type=float, default=256.0, help="bytes per rank, MiB")
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--sweep", action="store_true", help="also time 8 KiB .. 256 MiB per rank (x2), table on stderr")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--suite-filter", default="", help="with --suite: only configurations whose name contains this (several alternatives separated by commas)")
    ap.add_argument("--suite", action="store_true", help="time the other BASELINE.json configurations (table on stderr) and exit")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain 1 GiB int32 copy (one-rank all-reduce, out of place) three times, so that a "
                         "counter profile of this command holds a copy of known size to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--set", action="append", default=[], metavar="KEY=VALUE",
                    help="library setting for the run (see HcclAmdSetParam), e.g. --set blocks_per_cu=4")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path is built and measured on one GPU (the ranks of the communicator are "
                 "simulated inside it); --gpus %d is not supported" % args.gpus)

    import numpy as np
    import torch
    from __graft_entry__ import load_package

    pkg = load_package()
    pkg.lib()                                  # raises if the HIP library is not built
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if args.suite:
        run_suite(pkg, torch, args.steps, args.warmup, args.suite_filter, args.set)
        return
    p = args.ranks
    n = int(args.size_mib * (1 << 20)) // 4
    S = n * 4
    threads = min(16, os.cpu_count() or 1)

    # synthetic inputs, uniform in [-1, 1), made on the device
    gen = torch.Generator(device="cuda")
    gen.manual_seed(20240611)
    sends = [torch.rand(n, dtype=torch.float32, device="cuda", generator=gen) * 2.0 - 1.0 for _ in range(p)]
    recvs = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(p)]
    oracle, ins = None, None
    if not args.no_cpu:
        # the CPU checker is loaded for the cpu_baseline leg only (and the bit-for-bit comparison that goes with it)
        from oracle import oracle
        ins = [t.cpu().numpy() for t in sends]
    comms = pkg.comm_init_all(p)
    stream = torch.cuda.Stream()
    for kv in args.set:
        k, v = kv.split("=", 1)
        pkg.set_param(comms[0], k, v)
    torch.cuda.synchronize()

    wall_ms, dev_ms, info = run_mode(pkg, torch, comms, stream, sends, recvs, n, 1, args.steps, args.warmup)
    fused_out = recvs[0].cpu().numpy()
    med_ms, min_ms = per_launch_times(pkg, torch, comms, stream, sends, recvs, n, 1, args.steps)
    s_wall_ms, s_dev_ms, s_info = run_mode(pkg, torch, comms, stream, sends, recvs, n, 0, args.steps, args.warmup)
    step_out = recvs[0].cpu().numpy()
    same_all = all(torch.equal(recvs[0], recvs[r]) for r in range(1, p))

    actual = info["bytesRead"] + info["bytesWritten"]
    s_actual = s_info["bytesRead"] + s_info["bytesWritten"]
    achieved = actual / (dev_ms * 1e-3) / 1e9
    s_achieved = s_actual / (s_dev_ms * 1e-3) / 1e9

    cpu = None
    bit_exact = None
    if not args.no_cpu:
        best, touched = None, 0
        outs = [np.empty(n, np.float32) for _ in range(p)]
        for _ in range(3):
            work = [x.copy() for x in ins]
            t0 = time.perf_counter()
            _, touched = oracle.allreduce(work, oracle.FP32, oracle.SUM, flags=oracle.DIRECT | oracle.ZERO_STAGING,
                                          threads=threads, outs=outs, return_touched=True)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        bit_exact = bool(np.array_equal(outs[0], fused_out) and np.array_equal(outs[0], step_out))
        work = [x.copy() for x in ins]
        t0 = time.perf_counter()
        oracle.allreduce(work, oracle.FP32, oracle.SUM, flags=oracle.DIRECT | oracle.ZERO_STAGING, threads=1, outs=outs)
        single = time.perf_counter() - t0
        # same byte basis as `value`: every input read once, every output written once (2 * p * S) per collective
        cpu = {"value": round(actual / best / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": "the full workload once per timing (%d ranks x %.0f MiB fp32, out of place), the checker's ring "
                         "schedule in direct zero-staging mode on %d threads, best of 3 = %.3f s; value = 2*p*S bytes "
                         "(the headline's basis) / that time; the checker itself read and wrote %d bytes per "
                         "collective" % (p, args.size_mib, threads, best, touched),
               "bytes_touched_GBps": round(touched / best / 1e9, 3),
               "single_thread_value": round(actual / single / 1e9, 3), "single_thread_s": round(single, 3),
               "host_cpus_visible": os.cpu_count(), "cpu_model": cpu_model()}

    if args.calibrate:
        one = pkg.comm_init_all(1)
        m = 256 << 20
        src = torch.ones(m, dtype=torch.int32, device="cuda")
        dst = torch.zeros(m, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        for _ in range(3):
            pkg.all_reduce(one, [src.data_ptr()], [dst.data_ptr()], m, pkg.HCCL_DATA_TYPE_INT32, pkg.HCCL_REDUCE_SUM,
                           stream.cuda_stream)
        stream.synchronize()
        assert bool(torch.equal(src, dst))
        pkg.comm_destroy(one)
        del src, dst

    if args.sweep:
        sys.stderr.write("bytes/rank  fused_us  fused_GB/s(actual)  steps_us  steps_GB/s(actual)  sched_GB/s(fused)"
                         "  cpu_us(%d threads)  cpu_sched_GB/s  note\n" % threads)
        size = 8 << 10
        while size <= int(args.size_mib * (1 << 20)):
            m = size // 4
            _, f_ms, fi = run_mode(pkg, torch, comms, stream, sends, recvs, m, 1, args.steps, args.warmup)
            _, g_ms, gi = run_mode(pkg, torch, comms, stream, sends, recvs, m, 0, args.steps, args.warmup)
            fa = (fi["bytesRead"] + fi["bytesWritten"]) / (f_ms * 1e-3) / 1e9
            ga = (gi["bytesRead"] + gi["bytesWritten"]) / (g_ms * 1e-3) / 1e9
            cpu_us = float("nan")
            if not args.no_cpu:
                small = [x[:m] for x in ins]
                outs = [np.empty(m, np.float32) for _ in range(p)]
                best = None
                for _ in range(3):
                    work = [x.copy() for x in small]
                    t0 = time.perf_counter()
                    oracle.allreduce(work, oracle.FP32, oracle.SUM, flags=oracle.DIRECT | oracle.ZERO_STAGING, threads=threads,
                                     outs=outs)
                    dt = time.perf_counter() - t0
                    best = dt if best is None else min(best, dt)
                cpu_us = best * 1e6
            # send and receive buffers of all ranks together against the 256 MB memory-side cache: below it the replays
            # run out of cache and the rates say nothing about HBM
            note = "cache-resident" if 2 * p * size <= (256 << 20) else ""
            sys.stderr.write("%10d %9.1f %12.1f %9.1f %12.1f %12.1f %12.1f %12.1f  %s\n"
                             % (size, f_ms * 1e3, fa, g_ms * 1e3, ga, (5 * p - 3) * size / (f_ms * 1e-3) / 1e9, cpu_us,
                                (5 * p - 3) * size / (cpu_us * 1e-6) / 1e9, note))
            size *= 2

    headline = p == 8 and args.size_mib == 256.0 and not args.set and info["algo"] == 0
    sched_name = {0: "ring", 1: "mesh", 2: "halving-doubling", 4: "mesh"}.get(info["algo"], "?")
    launches = max(1, s_info["launches"])
    fused_kernel = ("Team" if info.get("teamLaunches") else "") + ("TreeKernel" if info["algo"] == 2 else "ChainKernel")
    # The headline is what a caller of HcclAllReduce gets with the library's defaults (fuse=1): one fused launch.
    line = {
        "metric": METRIC,
        "value": round(actual / (wall_ms * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "%s all-reduce sum fp32, %d simulated ranks x %.0f MiB per rank, out of place, one GPU%s"
                        % (sched_name, p, args.size_mib, " (BASELINE.json configs[1] at its largest size)" if headline else ""),
            "issue": "library default (fuse=1): one %s launch per collective reads every rank's input once, combines in "
                     "the %s schedule's order and writes every rank's output; same bits as the schedule run step by step"
                     % (fused_kernel, sched_name),
            "team_kernel": bool(info.get("teamLaunches")),
            "default_mode": "fused single pass",
            "launches_per_step": info["launches"],
            "graph": info["graph"],
            "bytes_per_step": actual,
            "pct_of_hbm_peak": round(100.0 * achieved / HBM_PEAK_GBPS, 2),
            "ms_per_step_device": round(dev_ms, 4),
            "launch_ms_median": round(med_ms, 4),
            "launch_ms_min": round(min_ms, 4),
            "schedule_bytes_per_second_GBps": round(s_actual / (dev_ms * 1e-3) / 1e9, 1),
            "bit_exact_vs_host_reference": bit_exact,
            "all_ranks_identical": bool(same_all),
            "step_by_step": {
                "note": "library setting fuse=0: the schedule's %d phases of copy / reduce steps, one StepKernel launch "
                        "each, replayed from a HIP graph; same bits; not the default (%.2fx the time per collective)"
                        % (s_info["launches"], s_dev_ms / dev_ms),
                "launches_per_step": s_info["launches"],
                "graph": s_info["graph"],
                "ms_per_step": round(s_wall_ms, 4),
                "ms_per_step_device": round(s_dev_ms, 4),
                "bytes_per_step": s_actual,
            },
        },
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": profiled_traffic(PROFILE_FUSED) if headline else None,
            "traffic_source": "profiles/" + os.path.basename(PROFILE_FUSED) + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)"
                              if headline else None,
            "kernel": "%s<float, sum> (fused %s all-reduce, the library default): %d algorithmic bytes per launch "
                      "(%d x %.0f MiB read + the same written), average launch %.4f ms over %d launches, HIP events on "
                      "the launching stream" % (fused_kernel, sched_name, actual, p, args.size_mib, dev_ms, args.steps),
        },
        "roofline_steps": {
            "bound": "hbm", "achieved": round(s_achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(s_achieved / HBM_PEAK_GBPS, 4),
            "traffic": profiled_traffic(PROFILE_STEPS) if headline else None,
            "kernel": "StepKernel<float, sum>, library setting fuse=0: %d launches per collective (one per phase), %.1f MB "
                      "per launch on average, average launch %.1f us = %.4f ms per graph replay / %d, gaps between the "
                      "graph's nodes included, over %d replays.  Includes memory-side-cache hits: from the second phase "
                      "on, part of what a phase reads was written by the phase before and comes out of the 256 MB "
                      "memory-side cache, so this is a rate between L2 and the fabric, not a DRAM rate (the one phase "
                      "with cold inputs runs about 16 %% slower, see profiles/)"
                      % (s_info["launches"], s_actual / launches / 1e6, s_dev_ms * 1e3 / launches, s_dev_ms, launches, args.steps),
        },
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))
    pkg.comm_destroy(comms)


if __name__ == "__main__":
    main()
