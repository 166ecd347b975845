"""Seeded random configurations through the C ABI against the CPU checker: ranks, sizes (whole tiles,
ragged ends, a few elements), types, operations, schedules, misaligned and in-place buffers, fused and
step-by-step issue.  Every case must match bit for bit (16-bit floats included: both sides round after
every step)."""
import os

import numpy as np
import pytest
import torch

import closed_forms as cf
import gpu_harness as gh
from closed_forms import ALL_TYPES, INT64, PROD

pytestmark = pytest.mark.gpu
# other random cases without touching the file: HCCL_AMD_TEST_SEED_SHIFT=1000 python -m pytest ...
SEED_SHIFT = int(os.environ.get("HCCL_AMD_TEST_SEED_SHIFT", "0"))
H = gh.H
RING, MESH, RHD, MESH_ATOMIC = 0, 1, 2, 4
NAMES = {RING: "ring", MESH: "mesh", RHD: "rhd", MESH_ATOMIC: "mesh"}


@pytest.fixture(scope="module")
def orc():
    from oracle import oracle
    oracle.build()
    return oracle


def _size(rng):
    kind = rng.integers(0, 5)
    if kind == 0:
        return int(rng.integers(1, 40))                       # a few elements
    if kind == 1:
        return int(rng.integers(1, 9)) * 4096 * 8             # whole tiles for every type and rank count up to 8
    if kind == 2:
        return int(rng.integers(1, 9)) * 4096 * 8 + int(rng.integers(1, 4096))   # tiles plus a ragged end
    return int(rng.integers(40, 300000))


def _expected(algo, dt, op):
    return MESH if (algo == MESH_ATOMIC and (dt == INT64 or op == PROD)) else algo


@pytest.mark.parametrize("seed", range(6))
def test_random_allreduce(orc, seed):
    rng = np.random.default_rng(9000 + SEED_SHIFT + seed)
    for case in range(12):
        p = int(rng.choice([2, 3, 4, 5, 7, 8, 12, 16]))
        algo = int(rng.choice([RING, MESH, RHD, MESH_ATOMIC]))
        dt = int(rng.choice(ALL_TYPES))
        op = int(rng.integers(0, 4))
        n = _size(rng)
        fuse = int(rng.integers(0, 2))
        in_place = bool(rng.integers(0, 2))
        unit = H.DTYPE_SIZE[dt]
        pad = int(rng.choice([0, 0, unit, 16, 4 if unit <= 4 else 8]))
        ccl = int(rng.choice([200 << 20, 200 << 20, 1 << 16, 3000 * unit]))
        ins = [cf.random_input(dt, n, rng) for _ in range(p)]
        want = orc.allreduce(ins, dt, op, algo=_expected(algo, dt, op), ccl_bytes=ccl)
        print("random allreduce seed", seed, "case", case, "p", p, "algo", algo, "type", dt, "op", op, "n", n, "fuse", fuse,
              "in place", in_place, "pad", pad, "ccl", ccl, flush=True)
        g = gh.Group(p, algo=NAMES[algo], deterministic=0 if algo == MESH_ATOMIC else 1, fuse=fuse, buffsize_bytes=ccl)
        try:
            outs, keep = gh.all_reduce(g, ins, dt, op, in_place=in_place, pad=pad)
            for r in range(p):
                assert gh.same(dt, outs[r], want[r]), (seed, case, r)
                if keep is not None:
                    assert np.array_equal(keep[r], ins[r])
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(4))
def test_random_reducescatter_allgather(orc, seed):
    rng = np.random.default_rng(9100 + SEED_SHIFT + seed)
    for case in range(10):
        p = int(rng.choice([2, 3, 4, 6, 8, 12]))
        algo = int(rng.choice([RING, MESH, RHD, MESH_ATOMIC]))
        dt = int(rng.choice(ALL_TYPES))
        op = int(rng.integers(0, 4))
        n = max(1, _size(rng) // p)
        fuse = int(rng.integers(0, 2))
        unit = H.DTYPE_SIZE[dt]
        pad = int(rng.choice([0, unit, 16]))
        print("random rs/ag seed", seed, "case", case, "p", p, "algo", algo, "type", dt, "op", op, "n", n, "fuse", fuse, "pad", pad,
              flush=True)
        g = gh.Group(p, algo=NAMES[algo], deterministic=0 if algo == MESH_ATOMIC else 1, fuse=fuse)
        try:
            ins = [cf.random_input(dt, n * p, rng) for _ in range(p)]
            want = orc.reducescatter(ins, dt, op, algo=_expected(algo, dt, op))
            outs, keep = gh.reduce_scatter(g, ins, dt, op, pad=pad)
            for r in range(p):
                assert gh.same(dt, outs[r], want[r]), (seed, case, "rs", r)
                assert np.array_equal(keep[r], ins[r])
            small = [x[:n] for x in ins]
            outs = gh.all_gather(g, small, dt, pad=pad)
            whole = np.concatenate(small)
            for r in range(p):
                assert np.array_equal(outs[r], whole), (seed, case, "ag", r)
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_rooted(orc, seed):
    rng = np.random.default_rng(9200 + SEED_SHIFT + seed)
    for case in range(8):
        p = int(rng.choice([2, 3, 5, 8, 12]))
        algo = int(rng.choice([RING, MESH, RHD, MESH_ATOMIC]))
        dt = int(rng.choice(ALL_TYPES))
        op = int(rng.integers(0, 4))
        n = _size(rng)
        fuse = int(rng.integers(0, 2))
        root = int(rng.integers(0, p))
        print("random rooted seed", seed, "case", case, "p", p, "algo", algo, "type", dt, "op", op, "n", n, "fuse", fuse, "root", root,
              flush=True)
        g = gh.Group(p, algo=NAMES[algo], deterministic=0 if algo == MESH_ATOMIC else 1, fuse=fuse)
        try:
            ins = [cf.random_input(dt, n, rng) for _ in range(p)]
            want = orc.reduce_to_root(ins, dt, op, root, algo=_expected(algo, dt, op))
            sends = [gh.to_dev(x) for x in ins]
            recvs = [gh.empty_dev(n * H.DTYPE_SIZE[dt], fill=0x33) for _ in range(p)]
            torch.cuda.synchronize()
            H.reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, root, g.stream_ptr)
            g.stream.synchronize()
            assert gh.same(dt, gh.to_host(recvs[root], dt), want), (seed, case, "reduce")
            bufs = [gh.to_dev(x) for x in ins]
            torch.cuda.synchronize()
            H.broadcast(g.comms, [t.data_ptr() for t in bufs], n, dt, root, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert np.array_equal(gh.to_host(bufs[r], dt), ins[root]), (seed, case, "broadcast", r)
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_allreduce_some_ranks_in_place_and_rank_groups(orc, seed):
    # a random subset of the ranks passes one buffer for both arguments; half the cases run on rank groups
    # (two-level schedules, mesh or rings inside a group)
    rng = np.random.default_rng(9300 + SEED_SHIFT + seed)
    for case in range(10):
        p = int(rng.choice([4, 6, 8, 12, 16]))
        dt = int(rng.choice(ALL_TYPES))
        op = int(rng.integers(0, 4))
        n = _size(rng)
        fuse = int(rng.integers(0, 2))
        mask = int(rng.integers(0, 1 << p))
        level1 = int(rng.choice([RING, RHD]))
        servers, level0 = 1, "mesh"
        if rng.random() < 0.5:
            servers = int(rng.choice([s for s in range(2, p + 1) if p % s == 0]))
            level0 = str(rng.choice(["mesh", "ring", "ring4"])) if p // servers == 8 else str(rng.choice(["mesh", "ring"]))
        unit = H.DTYPE_SIZE[dt]
        pad = int(rng.choice([0, 0, unit, 16, 4 if unit <= 4 else 8]))      # buffers off their natural alignment
        ins = [cf.random_input(dt, n, rng) for _ in range(p)]
        if servers > 1:
            atomic = level0 == "mesh" and dt != INT64 and op != PROD
            want = orc.allreduce_two_level(ins, dt, op, servers, level1=level1, atomic=atomic, level0=level0)
        else:
            want = orc.allreduce(ins, dt, op, algo=level1)
        print("random allreduce seed", seed, "case", case, "p", p, "type", dt, "op", op, "n", n, "fuse", fuse, "mask", bin(mask),
              "servers", servers, level0, "level1", level1, "pad", pad, flush=True)
        g = gh.Group(p, algo=NAMES[level1], fuse=fuse, servers=servers, level0=level0)
        try:
            sends = [gh.to_dev(x, pad) for x in ins]
            recvs = [sends[r] if (mask >> r) & 1 else gh.empty_dev(n * unit, pad if r % 2 else 0) for r in range(p)]
            torch.cuda.synchronize()
            H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert gh.same(dt, gh.to_host(recvs[r], dt), want[r]), (seed, case, r)
                if not (mask >> r) & 1:
                    assert np.array_equal(gh.to_host(sends[r], dt), ins[r]), (seed, case, r, "send buffer changed")
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_reducescatter_and_reduce_on_rank_groups(orc, seed):
    # two-level reduce-scatter and rooted reduce: random group shapes, types, sizes, misaligned buffers, both issue modes
    rng = np.random.default_rng(9400 + SEED_SHIFT + seed)
    for case in range(8):
        p = int(rng.choice([4, 6, 8, 12, 16, 16, 24, 32]))
        servers = int(rng.choice([s for s in range(2, p + 1) if p % s == 0]))
        if p >= 16 and p % 8 == 0 and int(rng.integers(0, 2)):
            servers = p // 8                                  # servers of 8 devices: the four-ring topology is allowed
        level1 = int(rng.choice([RING, RHD]))
        det = int(rng.integers(0, 2))
        dt = int(rng.choice(ALL_TYPES))
        op = int(rng.integers(0, 4))
        n = max(1, _size(rng) // p)
        fuse = int(rng.integers(0, 2))
        root = int(rng.integers(0, p))
        unit = H.DTYPE_SIZE[dt]
        pad = int(rng.choice([0, 0, unit, 16]))
        atomic = det == 0 and dt != INT64 and op != PROD
        level0 = str(rng.choice(["mesh", "mesh", "ring", "ring4"] if p // servers == 8 else ["mesh", "mesh", "ring"]))
        print("random grouped seed", seed, "case", case, "p", p, "servers", servers, level0, "level1", level1, "deterministic", det,
              "type", dt, "op", op, "n", n, "fuse", fuse, "root", root, "pad", pad, flush=True)
        g = gh.Group(p, algo=NAMES[level1], deterministic=det, fuse=fuse, servers=servers)
        try:
            ins = [cf.random_input(dt, n * p, rng) for _ in range(p)]
            g.set(level0=level0)
            # four rings inside, a ring between the servers: on some cases only a few devices of a server have a network port
            nic = ([[0, 4], [5], [1, 2, 3, 7], None][int(rng.integers(0, 4))]
                   if level0 == "ring4" and level1 == RING and servers > 1 else None)
            if nic is not None:
                print("    network ports on devices", nic, flush=True)
                g.set(nic_ranks=",".join(str(d) for d in nic))
                want = orc.reducescatter_two_level_pruned([x.copy() for x in ins], dt, op, servers, nic)
            else:
                want = orc.reducescatter_two_level(ins, dt, op, servers, level1=level1, atomic=atomic, level0=level0)
            sends = [gh.to_dev(x, pad) for x in ins]
            recvs = [gh.empty_dev(n * unit, pad if r % 2 else 0) for r in range(p)]
            torch.cuda.synchronize()
            H.reduce_scatter(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert gh.same(dt, gh.to_host(recvs[r], dt), want[r]), (seed, case, "reduce-scatter", r)
                assert np.array_equal(gh.to_host(sends[r], dt), ins[r]), (seed, case, "send buffer changed", r)
            if nic is not None:
                g.set(nic_ranks="all")
            want_root = orc.reduce_to_root_two_level(ins, dt, op, root, servers, level1=level1, atomic=atomic, level0=level0)
            outs = [gh.empty_dev(n * p * unit, 0 if r % 2 else pad, fill=0x33) for r in range(p)]
            torch.cuda.synchronize()
            H.reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in outs], n * p, dt, op, root, g.stream_ptr)
            g.stream.synchronize()
            assert gh.same(dt, gh.to_host(outs[root], dt), want_root), (seed, case, "reduce")
            for r in range(p):
                if r != root:
                    assert bool((outs[r] == 0x33).all()), (seed, case, "a rank other than the root was written", r)
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_alltoallv_flat_and_staged(orc, seed):
    """All-to-all-v with random tables: element sizes 1, 2, 4 and 8 bytes (displacements then fall on every byte
    alignment), counts from zero to tens of thousands, over one server or several, fused and step by step,
    against the checker's staged or flat schedule; bytes outside the addressed blocks must stay as they were."""
    from closed_forms import INT8, INT16, INT32
    rng = np.random.default_rng(5200 + SEED_SHIFT + seed)
    carriers = {INT8: np.int8, INT16: np.int16, INT32: np.int32, INT64: np.int64}
    for case in range(8):
        p = int(rng.choice([2, 3, 4, 6, 8, 12, 16]))
        servers = int(rng.choice([s for s in range(1, p + 1) if p % s == 0]))
        dt = int(rng.choice(list(carriers)))
        fuse = int(rng.integers(0, 2))
        big = int(rng.choice([50, 3000, 40000]))
        cnt = rng.integers(0, big, (p, p)).astype(np.uint64)
        cnt[rng.random((p, p)) < 0.2] = 0
        sdis, rdis = np.zeros((p, p), np.uint64), np.zeros((p, p), np.uint64)
        sl, rl = [], []
        for r in range(p):
            pos = 0
            for j in rng.permutation(p):
                pos += int(rng.integers(0, 37))
                sdis[r, j] = pos
                pos += int(cnt[r, j])
            sl.append(pos + 7)
            pos = 0
            for i in rng.permutation(p):
                pos += int(rng.integers(0, 37))
                rdis[r, i] = pos
                pos += int(cnt[i, r])
            rl.append(pos + 7)
        info = np.iinfo(carriers[dt])
        ins = [rng.integers(info.min, info.max, n, dtype=carriers[dt]) for n in sl]
        want = [np.full(n, 0x5A, carriers[dt]) for n in rl]
        if servers > 1:
            assert orc.alltoallv_staged(ins, cnt, sdis, want, cnt.T.copy(), rdis, dt, servers) == 0
        else:
            assert orc.alltoallv(ins, cnt, sdis, want, cnt.T.copy(), rdis, dt) == 0
        ccl = int(rng.choice([200 << 20, 1 << 16, 4096]))          # small buffers: blocks and runs travel in pieces
        print("random all-to-all-v seed", seed, "case", case, "p", p, "servers", servers, "dt", dt, "fuse", fuse, "max", big,
              "buffer", ccl, flush=True)
        g = gh.Group(p, fuse=fuse, servers=servers, buffsize_bytes=ccl)
        try:
            outs = gh.all_to_all_v(g, ins, cnt, sdis, rl, cnt.T.copy(), rdis, dt, fill=0x5A)
            for r in range(p):
                assert np.array_equal(outs[r], want[r]), (seed, case, r)
            assert g.info()["fused"] == fuse
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(2))
def test_random_two_level_reducescatter_with_random_network_ports(orc, seed):
    """Servers of 8 devices with four rings inside and a ring between them, 1, 2, 4 or all 8 devices of every server with a
    network port, chosen at random: the branch that all-reduces inside a server first, against the checker, on random
    types, reductions, counts, staging-buffer sizes and both issue modes."""
    rng = np.random.default_rng(9700 + SEED_SHIFT + seed)
    for case in range(6):
        servers = int(rng.choice([2, 2, 3, 4]))
        p = servers * 8
        ports = int(rng.choice([1, 2, 4, 8]))
        nic = sorted(int(d) for d in rng.choice(8, size=ports, replace=False))
        dt = int(rng.choice(ALL_TYPES))
        op = int(rng.integers(0, 4))
        n = max(1, _size(rng) // (4 * p))
        fuse = int(rng.integers(0, 2))
        ccl = int(rng.choice([200 << 20, 1 << 18]))
        unit = H.DTYPE_SIZE[dt]
        pad = int(rng.choice([0, unit, 16]))
        print("random pruned two-level seed", seed, "case", case, "servers", servers, "ports", nic, "type", dt, "op", op, "n", n,
              "fuse", fuse, "buffer", ccl, "pad", pad, flush=True)
        g = gh.Group(p, algo="ring", servers=servers, level0="ring4", fuse=fuse, buffsize_bytes=ccl)
        try:
            g.set(nic_ranks=",".join(str(d) for d in nic))
            ins = [cf.random_input(dt, n * p, rng) for _ in range(p)]
            want = (orc.reducescatter_two_level_pruned([x.copy() for x in ins], dt, op, servers, nic, ccl_bytes=ccl) if ports < 8
                    else orc.reducescatter_two_level(ins, dt, op, servers, level1=RING, level0="ring4", ccl_bytes=ccl))
            sends = [gh.to_dev(x, pad) for x in ins]
            recvs = [gh.empty_dev(n * unit, pad if r % 2 else 0) for r in range(p)]
            torch.cuda.synchronize()
            H.reduce_scatter(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert gh.same(dt, gh.to_host(recvs[r], dt), want[r]), (seed, case, r)
                assert np.array_equal(gh.to_host(sends[r], dt), ins[r]), (seed, case, "send buffer changed", r)
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_scatter_and_broadcast_over_rank_groups(orc, seed):
    """Scatter and broadcast with random roots, rank groups and schedule settings (auto, ring, star, ...): whatever the route,
    rank r ends with the root's block r / with the root's buffer, the root's input stays as it was."""
    rng = np.random.default_rng(5300 + SEED_SHIFT + seed)
    for case in range(8):
        p = int(rng.choice([2, 3, 4, 6, 8, 12, 16]))
        servers = int(rng.choice([s for s in range(1, p + 1) if p % s == 0]))
        setting = str(rng.choice(["auto", "ring", "star", "mesh", "rhd", "hd_blocks"]))
        dt = int(rng.choice(ALL_TYPES))
        n = _size(rng) // 4 + 1
        fuse = int(rng.integers(0, 2))
        root = int(rng.integers(0, p))
        ccl = int(rng.choice([200 << 20, 1 << 16]))
        level0 = str(rng.choice(["mesh", "ring", "ring4"] if p // servers == 8 else ["mesh", "ring"]))
        print("random scatter / broadcast seed", seed, "case", case, "p", p, "servers", servers, level0, "algo", setting, "type", dt,
              "n", n, "fuse", fuse, "root", root, "buffer", ccl, flush=True)
        g = gh.Group(p, algo=setting, fuse=fuse, servers=servers, buffsize_bytes=ccl)
        try:
            g.set(level0=level0)
            src = cf.random_input(dt, n * p, rng)
            sends = [gh.to_dev(src) if r == root else None for r in range(p)]
            recvs = [gh.empty_dev(n * H.DTYPE_SIZE[dt], fill=0x33) for _ in range(p)]
            torch.cuda.synchronize()
            H.scatter(g.comms, [t.data_ptr() if t is not None else None for t in sends], [t.data_ptr() for t in recvs],
                      n, dt, root, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert np.array_equal(gh.to_host(recvs[r], dt), src[r * n:(r + 1) * n]), (seed, case, "scatter", r)
            assert np.array_equal(gh.to_host(sends[root], dt), src)
            ins = [cf.random_input(dt, n, rng) for _ in range(p)]
            bufs = [gh.to_dev(x) for x in ins]
            torch.cuda.synchronize()
            H.broadcast(g.comms, [t.data_ptr() for t in bufs], n, dt, root, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert np.array_equal(gh.to_host(bufs[r], dt), ins[root]), (seed, case, "broadcast", r)
        finally:
            g.close()


@pytest.mark.parametrize("seed", range(3))
def test_random_sequence_of_calls_on_one_group(orc, seed):
    # What a training or serving loop does to one communicator: collectives of every kind with sizes and tables that
    # change from call to call, repeats of earlier calls, the issue mode switched in between.  The library answers
    # from its caches where it can (prepared collectives, plans, plans derived from earlier plans) and grows its
    # scratch memory on the way; every result is the checker's.
    rng = np.random.default_rng(5400 + SEED_SHIFT + seed)
    p = int(rng.choice([4, 8, 16]))
    algo = int(rng.choice([RING, MESH_ATOMIC, RHD]))
    dt = int(rng.choice([cf.FP32, cf.BF16, cf.INT32, cf.FP16]))
    op = 0
    unit = H.DTYPE_SIZE[dt]
    top = 48 * 1024
    pool = [cf.random_input(dt, top * p, rng) for _ in range(p)]          # every call reads a prefix of these
    sends = [gh.to_dev(x) for x in pool]
    recvs = [gh.empty_dev(top * p * unit) for _ in range(p)]
    ptr = lambda ts: [t.data_ptr() for t in ts]
    g = gh.Group(p, algo=NAMES[algo], deterministic=0 if algo == MESH_ATOMIC else 1, cache_entries=16)
    seen = []
    try:
        torch.cuda.synchronize()
        for call in range(60):
            if call % 7 == 3:
                g.set(fuse=int(rng.integers(0, 2)))
            kind = str(rng.choice(["ar", "ar", "rs", "rsv", "ag", "agv", "red", "bc"]))
            if seen and rng.random() < 0.25:
                kind, n, counts = seen[int(rng.integers(0, len(seen)))]      # an earlier call again
            else:
                n = int(rng.choice([int(rng.integers(1, 64)), int(rng.integers(1, 6)) * p * 32 * 16, int(rng.integers(64, top))]))
                counts = rng.integers(1, top // 2, p) if rng.random() < 0.8 else rng.integers(0, 50, p)
                seen.append((kind, n, counts))
            displs = np.concatenate(([0], np.cumsum(counts)[:-1])).astype(np.int64)
            print("sequence seed", seed, "call", call, kind, "p", p, "algo", algo, "type", dt, "n", n, flush=True)
            if kind == "ar":
                ins = [x[:n] for x in pool]
                want = orc.allreduce(ins, dt, op, algo=algo)
                H.all_reduce(g.comms, ptr(sends), ptr(recvs), n, dt, op, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[r], dt)[:n] for r in range(p)]
            elif kind == "rs":
                m = max(1, n // p)
                want = orc.reducescatter([x[:m * p] for x in pool], dt, op, algo=algo)
                H.reduce_scatter(g.comms, ptr(sends), ptr(recvs), m, dt, op, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[r], dt)[:m] for r in range(p)]
            elif kind == "rsv":
                extent = int(counts.sum())
                want = orc.reducescatter_v([x[:extent] for x in pool], counts, displs, dt, op, algo=algo)
                H.reduce_scatter_v(g.comms, ptr(sends), counts, displs, ptr(recvs), dt, op, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[r], dt)[:int(counts[r])] for r in range(p)]
            elif kind == "ag":
                m = max(1, n // p)
                want = [np.concatenate([x[:m] for x in pool])] * p
                H.all_gather(g.comms, ptr(sends), ptr(recvs), m, dt, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[r], dt)[:m * p] for r in range(p)]
            elif kind == "agv":
                want = [np.concatenate([pool[r][:int(counts[r])] for r in range(p)])] * p
                H.all_gather_v(g.comms, ptr(sends), ptr(recvs), counts, displs, dt, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[r], dt)[:int(counts.sum())] for r in range(p)]
            elif kind == "red":
                root = n % p
                want = [orc.reduce_to_root([x[:n] for x in pool], dt, op, root, algo=algo)]
                H.reduce(g.comms, ptr(sends), ptr(recvs), n, dt, op, root, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[root], dt)[:n]]
            else:
                root = n % p
                for r in range(p):
                    recvs[r][:n * unit].copy_(sends[r][:n * unit])
                torch.cuda.synchronize()
                want = [pool[root][:n]] * p
                H.broadcast(g.comms, ptr(recvs), n, dt, root, g.stream_ptr)
                g.stream.synchronize()
                got = [gh.to_host(recvs[r], dt)[:n] for r in range(p)]
            for r in range(len(want)):
                assert gh.same(dt, got[r], want[r]), (seed, call, kind, r)
        for r in range(p):
            assert np.array_equal(gh.to_host(sends[r], dt), pool[r]), ("send buffer changed", r)
    finally:
        g.close()
