"""The team form of the fused kernels (an XCD's workgroups read together, park their results in LDS, write together)
against the CPU checker, through the C ABI: every kernel family (chain, copy, tree, stack), sizes that run for several
rounds and end in the shrinking tail of regions, ragged and unaligned buffers, in place, repeated launches on the same
buffers (the launch's counters must come back to zero), replays from a caller's graph, and the library's own choice of
the team form for large write-heavy collectives.  Same bars as the plain kernels: bit for bit."""
import numpy as np
import pytest
import torch

import closed_forms as cf
import gpu_harness as gh
from closed_forms import BF16, FP16, FP32, INT8, INT32, INT64, MAX, MIN, PROD, SUM

pytestmark = pytest.mark.gpu
H = gh.H
RING, MESH, RHD = 0, 1, 2
ALGO_NAME = {RING: "ring", MESH: "mesh", RHD: "rhd"}


@pytest.fixture(scope="module")
def orc():
    from oracle import oracle
    oracle.build()
    return oracle


def _ins(dt, p, n, seed):
    rng = np.random.default_rng(seed)
    return [cf.random_input(dt, n, rng) for _ in range(p)]


def test_team_chain_allreduce_types_ops_sizes(orc):
    # ring all-reduce through TeamChainKernel: one tile, a ragged tail, several rounds with the shrinking tail of regions
    p = 8
    g = gh.Group(p, algo="ring", team=1)
    try:
        for dt, op, n in ((FP32, SUM, 5), (FP32, SUM, 100003), (FP32, MAX, 3 * 1024 * 1024 + 17), (BF16, SUM, 2 * 1024 * 1024 + 5),
                          (INT8, MIN, 9 * 1024 * 1024 + 3), (INT64, PROD, 524288 + 1), (FP16, PROD, 300001),
                          (FP32, SUM, 24 * 1024 * 1024 + 64)):
            print("team chain", dt, op, n, flush=True)
            ins = _ins(dt, p, n, 7000 + dt + n % 97)
            want = orc.allreduce(ins, dt, op)
            for rep in range(2):         # the second launch finds the counters as the first left them
                outs, keep = gh.all_reduce(g, ins, dt, op)
                info = g.info()
                assert info["fused"] == 1 and info["teamLaunches"] >= 1, info
                for r in range(p):
                    assert gh.same(dt, outs[r], want[r]), (dt, op, n, rep, r)
                    assert np.array_equal(keep[r], ins[r])
    finally:
        g.close()


def test_team_chain_in_place_and_unaligned(orc):
    p, n = 8, 1500007
    g = gh.Group(p, algo="ring", team=1)
    try:
        for pad in (0, 4, 20):
            for in_place in (False, True):
                ins = _ins(FP32, p, n, 7100 + pad)
                want = orc.allreduce(ins, FP32, SUM)
                print("team chain pad", pad, "in place", in_place, flush=True)
                outs, _ = gh.all_reduce(g, ins, FP32, SUM, in_place=in_place, pad=pad)
                assert g.info()["teamLaunches"] >= 1
                for r in range(p):
                    assert np.array_equal(outs[r], want[r]), (pad, in_place, r)
    finally:
        g.close()


def test_team_chain_whole_rounds_read_source_by_source(orc):
    # Slices of 4 MiB and more: a workgroup's round is then 8 (in the tail of regions 4) whole tiles of one item, and
    # the chain kernel reads such a round source by source with the partial results in LDS.  Even and odd numbers of
    # sources, 2 and 3 of them, more than 8; element widths of 1 to 8 bytes; float max / min over NaNs with payloads,
    # signed zeros, infinities and denormals, where a swapped operand in any fold changes the bits; in place.
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.0, -1.0, 3.4e38], np.float32)
    nan2 = np.array([0x7fc00001, 0xffc00002, 0x7fa00003], np.uint32).view(np.float32)
    pool = np.concatenate([specials, nan2])
    mib = 1 << 20
    for p, dt, op, slice_bytes, special, in_place in ((8, FP32, MAX, 8 * mib, True, False), (8, FP32, MIN, 4 * mib, True, True),
                                                      (7, FP16, SUM, 8 * mib, False, False), (5, INT8, SUM, 8 * mib, False, False),
                                                      (4, INT64, PROD, 8 * mib, False, False), (16, FP32, SUM, 4 * mib, False, False),
                                                      (3, BF16, MIN, 8 * mib, False, True), (2, FP32, MAX, 16 * mib, True, False),
                                                      (6, BF16, SUM, 8 * mib, False, False)):
        n = p * slice_bytes // H.DTYPE_SIZE[dt]
        rng = np.random.default_rng(7300 + p + dt)
        print("team chain by source p", p, "type", dt, "op", op, "slice", slice_bytes, "specials", special, "in place", in_place, flush=True)
        ins = [rng.choice(pool, n).astype(np.float32) if special else cf.random_input(dt, n, rng) for _ in range(p)]
        want = orc.allreduce([x.copy() for x in ins], dt, op, threads=8)
        g = gh.Group(p, algo="ring", team=1)
        try:
            for rep in range(2):
                outs, keep = gh.all_reduce(g, ins, dt, op, in_place=in_place)
                info = g.info()
                assert info["fused"] == 1 and info["teamLaunches"] >= 1, info
                for r in range(p):
                    if special:
                        assert np.array_equal(outs[r].view(np.uint32), want[r].view(np.uint32)), (p, dt, op, rep, r)
                    else:
                        assert gh.same(dt, outs[r], want[r]), (p, dt, op, rep, r)
                    assert in_place or np.array_equal(keep[r].view(np.uint8), ins[r].view(np.uint8))
        finally:
            g.close()


@pytest.mark.parametrize("algo", [MESH, RHD])
def test_team_mesh_and_tree_allreduce(orc, algo):
    # the halving-doubling schedule fuses into trees (TeamTreeKernel), with a fold for rank counts that are no power of
    # two; the mesh into chains
    for p in (8, 6, 16, 12):
        g = gh.Group(p, algo=ALGO_NAME[algo], deterministic=1, team=1)
        try:
            for dt, op, n in ((FP32, SUM, 2 * 1024 * 1024 + 11), (BF16, SUM, 1024 * 1024 + 3), (INT32, MAX, 70001)):
                print("team", ALGO_NAME[algo], "p", p, dt, op, n, flush=True)
                ins = _ins(dt, p, n, 7200 + p + dt)
                want = orc.allreduce(ins, dt, op, algo=algo)
                outs, _ = gh.all_reduce(g, ins, dt, op)
                info = g.info()
                assert info["fused"] == 1 and info["teamLaunches"] >= 1, info
                for r in range(p):
                    assert gh.same(dt, outs[r], want[r]), (algo, p, dt, r)
        finally:
            g.close()


def test_team_stack_two_level_allreduce(orc):
    # mesh inside a group, ring between the groups: chains inside chains, the stack kernel's team form
    servers, D = 2, 4
    p = servers * D
    g = gh.Group(p, algo="ring", servers=servers, deterministic=1, team=1)
    try:
        for dt, op, n in ((FP32, SUM, 3 * 1024 * 1024 + 7), (BF16, PROD, 500001), (FP32, MIN, 100003)):
            print("team stack", dt, op, n, flush=True)
            ins = _ins(dt, p, n, 7300 + dt)
            want = orc.allreduce_two_level(ins, dt, op, servers, level1=RING)
            outs, _ = gh.all_reduce(g, ins, dt, op)
            info = g.info()
            assert info["fused"] == 1 and info["teamLaunches"] >= 1, info
            for r in range(p):
                assert gh.same(dt, outs[r], want[r]), (dt, op, r)
    finally:
        g.close()


def test_team_copy_allgather_and_broadcast(orc):
    p = 8
    g = gh.Group(p, algo="ring", team=1)
    try:
        # (the 16 MiB blocks give rounds of 8 whole tiles, which are read with all their loads issued at once)
        for dt, n, pad in ((INT32, 1000003, 0), (INT8, 5 * 1024 * 1024 + 1, 0), (BF16, 700001, 6), (INT32, 4 * 1024 * 1024, 0)):
            print("team copy all-gather", dt, n, pad, flush=True)
            ins = _ins(dt, p, n, 7400 + dt)
            outs = gh.all_gather(g, ins, dt, pad=pad)
            assert g.info()["teamLaunches"] >= 1
            whole = np.concatenate(ins)
            for r in range(p):
                assert np.array_equal(outs[r], whole), (dt, n, r)
        for n, root in ((3 * 1024 * 1024 + 9, 5), (16 * 1024 * 1024, 2)):
            print("team copy broadcast", n, root, flush=True)
            bufs_np = _ins(INT32, p, n, 7450)
            bufs = [gh.to_dev(x) for x in bufs_np]
            torch.cuda.synchronize()
            H.broadcast(g.comms, [t.data_ptr() for t in bufs], n, INT32, root, g.stream_ptr)
            g.stream.synchronize()
            assert g.info()["teamLaunches"] >= 1
            for r in range(p):
                assert np.array_equal(gh.to_host(bufs[r], INT32), bufs_np[root]), r
    finally:
        g.close()


def test_team_reducescatter_and_reduce_when_forced(orc):
    # many sources into one destination: not what the library picks the team form for, but it must give the same bits
    p = 8
    g = gh.Group(p, algo="ring", team=1)
    try:
        n = (2 * 1024 * 1024 + 40) // p * p
        ins = _ins(FP32, p, n, 7500)
        want = orc.reducescatter(ins, FP32, SUM)
        outs, _ = gh.reduce_scatter(g, ins, FP32, SUM)
        assert g.info()["teamLaunches"] >= 1
        for r in range(p):
            assert np.array_equal(outs[r], want[r]), r
    finally:
        g.close()


def test_team_kernels_replayed_from_a_callers_graph(orc):
    # the launch's counters are put back by the kernel itself, so a captured launch can be replayed as it is
    p, n = 8, 2 * 1024 * 1024 + 3
    g = gh.Group(p, team=1)
    try:
        rng = np.random.default_rng(7600)
        sends = [torch.from_numpy(rng.standard_normal(n).astype(np.float32)).cuda() for _ in range(p)]
        recvs = [torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(p)]
        gath = [torch.zeros(n * p, dtype=torch.float32, device="cuda") for _ in range(p)]
        torch.cuda.synchronize()

        def both():
            H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, FP32, SUM, g.stream_ptr)
            assert g.info()["teamLaunches"] == 1
            H.all_gather(g.comms, [t.data_ptr() for t in recvs], [t.data_ptr() for t in gath], n, FP32, g.stream_ptr)
            assert g.info()["teamLaunches"] == 1

        both()
        g.stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(g.stream):
            graph.capture_begin()
            try:
                both()
            finally:
                graph.capture_end()
        for replay in range(3):
            for t in sends:
                t.mul_(1.25)
            torch.cuda.synchronize()
            want = orc.allreduce([t.cpu().numpy() for t in sends], FP32, SUM)
            for t in recvs + gath:
                t.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            if replay == 1:              # an eager launch of the same prepared collectives between two replays
                both()
                g.stream.synchronize()
            for r in range(p):
                assert np.array_equal(recvs[r].cpu().numpy(), want[r]), (replay, r)
                assert np.array_equal(gath[r].cpu().numpy(), np.concatenate(want)), (replay, r)
    finally:
        g.close()


def test_library_picks_the_team_form_for_large_write_heavy_collectives(orc):
    # default settings: an all-reduce of 64 MiB per rank runs for two full rounds and more and writes eight destinations
    # per tile -> team kernel; a small one, and a reduce-scatter (one destination per tile) -> the plain kernels
    p = 8
    g = gh.Group(p, algo="ring", team="auto")
    try:
        n = 16 * 1024 * 1024
        ins = _ins(FP32, p, n, 7700)
        want = orc.allreduce(ins, FP32, SUM)
        outs, _ = gh.all_reduce(g, ins, FP32, SUM)
        assert g.info()["teamLaunches"] == 1, g.info()
        for r in range(p):
            assert np.array_equal(outs[r], want[r]), r
        small = [x[:100003] for x in ins]
        outs, _ = gh.all_reduce(g, small, FP32, SUM)
        assert g.info()["teamLaunches"] == 0
        want = orc.allreduce(small, FP32, SUM)
        for r in range(p):
            assert np.array_equal(outs[r], want[r]), r
        outs, _ = gh.reduce_scatter(g, ins, FP32, SUM)
        assert g.info()["teamLaunches"] == 0
        want = orc.reducescatter(ins, FP32, SUM)
        for r in range(p):
            assert np.array_equal(outs[r], want[r]), r
        g.set(team=0)
        outs, _ = gh.all_reduce(g, ins, FP32, SUM)
        assert g.info()["teamLaunches"] == 0
        want = orc.allreduce(ins, FP32, SUM)
        for r in range(p):
            assert np.array_equal(outs[r], want[r]), r
    finally:
        g.close()
