"""The reduce-scatter that allocates nothing (HcclAmdReduceScatterNoAlloc) against HcclReduceScatter, through
the C ABI: same bits, on two calls in a row of which the second is smaller, fused and step by step, and the
size limit of the fixed workspace."""
import numpy as np
import pytest
import torch

import closed_forms as cf
import gpu_harness as gh
from closed_forms import BF16, FP32, INT32, MAX, SUM

pytestmark = pytest.mark.gpu
H = gh.H


def _ins(dt, p, n, seed):
    rng = np.random.default_rng(seed)
    return [cf.random_input(dt, n, rng) for _ in range(p)]


def _both(g, ins, dt, op):
    """Runs the ordinary entry point, then the one under test, on the same device inputs; returns both outputs."""
    unit = H.DTYPE_SIZE[dt]
    n = ins[0].size // g.p
    sends = [gh.to_dev(x) for x in ins]
    ref = [gh.empty_dev(n * unit) for _ in ins]
    got = [gh.empty_dev(n * unit, fill=0x5A) for _ in ins]
    torch.cuda.synchronize()
    sp = [t.data_ptr() for t in sends]
    H.reduce_scatter(g.comms, sp, [t.data_ptr() for t in ref], n, dt, op, g.stream_ptr)
    H.reduce_scatter_no_alloc(g.comms, sp, [t.data_ptr() for t in got], n, dt, op, g.stream_ptr)
    info = g.info()
    g.stream.synchronize()
    for r in range(g.p):
        assert np.array_equal(gh.to_host(sends[r], dt), ins[r])          # send buffers are left alone
    return [gh.to_host(t, dt) for t in ref], [gh.to_host(t, dt) for t in got], info


@pytest.mark.parametrize("fuse", [1, 0])
def test_reduce_scatter_no_alloc_matches_reduce_scatter(orc, fuse):
    p = 8
    g = gh.Group(p, fuse=fuse)
    try:
        # two calls in a row on the same workspace, the second with a smaller input; then other types
        for dt, op, n in ((FP32, SUM, 100003), (FP32, SUM, 4099), (BF16, SUM, 30011), (INT32, MAX, 7), (FP32, SUM, 131072)):
            print("reduce-scatter without allocation: fuse", fuse, "type", dt, "op", op, "n", n, flush=True)
            ins = _ins(dt, p, n * p, 17 * n + dt)
            ref, got, info = _both(g, ins, dt, op)
            want = orc.reducescatter(ins, dt, op)
            for r in range(p):
                assert gh.same(dt, got[r], ref[r]), (fuse, dt, op, n, r)
                assert gh.same(dt, got[r], want[r]), (fuse, dt, op, n, r)
            assert info["fused"] == fuse and info["graph"] == 0 and info["cacheHit"] == 0
    finally:
        g.close()


def test_reduce_scatter_no_alloc_rejects_what_does_not_fit(orc):
    p = 8
    g = gh.Group(p, fuse=0)
    try:
        # step by step the schedule keeps p * n * 4 bytes of partial results per rank; the workspace has 4 MiB per rank
        n = (4 << 20) // 4 // p + 64
        sends = [torch.zeros(n * p, dtype=torch.float32, device="cuda") for _ in range(p)]
        recvs = [torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(p)]
        torch.cuda.synchronize()
        with pytest.raises(H.HcclError) as e:
            H.reduce_scatter_no_alloc(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, FP32, SUM,
                                      g.stream_ptr)
        assert e.value.code == H.HCCL_E_PARA
        # the same size through the fused form needs tables only and goes through
        g.set(fuse=1)
        H.reduce_scatter_no_alloc(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, FP32, SUM,
                                  g.stream_ptr)
        g.stream.synchronize()
        assert all(float(t.abs().max()) == 0.0 for t in recvs)
    finally:
        g.close()


def test_reduce_scatter_no_alloc_on_a_group_assembled_rank_by_rank(orc):
    # communicators made with HcclCommInitRootInfo: the device is set up when the last rank joins, so the first
    # collective of the group may be the one that allocates nothing
    p, n = 8, 20011
    comms = H.comm_init_root_info(p, H.comm_config_init())
    stream = torch.cuda.Stream()
    try:
        ins = _ins(FP32, p, n * p, 4242)
        want = orc.reducescatter(ins, FP32, SUM)
        sends = [gh.to_dev(x) for x in ins]
        got = [gh.empty_dev(n * 4, fill=0x5A) for _ in ins]
        torch.cuda.synchronize()
        H.reduce_scatter_no_alloc(comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in got], n, FP32, SUM,
                                  stream.cuda_stream)
        stream.synchronize()
        for r in range(p):
            assert np.array_equal(gh.to_host(got[r], FP32), want[r]), r
    finally:
        torch.cuda.synchronize()
        H.comm_destroy(comms)


@pytest.mark.parametrize("fuse", [1, 0])
def test_reduce_scatter_no_alloc_calls_on_two_streams_are_ordered(orc, fuse):
    # two groups on two streams share the GPU's one workspace: the second call is queued behind the first call's work
    # by the library (an event made at set-up), so each gets its own result although nothing orders the streams otherwise
    p = 8
    ga, gb = gh.Group(p, fuse=fuse), gh.Group(p, fuse=fuse)
    try:
        na, nb = 120011, 4099
        ins_a, ins_b = _ins(FP32, p, na * p, 5151), _ins(FP32, p, nb * p, 5152)
        want_a, want_b = orc.reducescatter(ins_a, FP32, SUM), orc.reducescatter(ins_b, FP32, SUM)
        sa, sb = [gh.to_dev(x) for x in ins_a], [gh.to_dev(x) for x in ins_b]
        oa = [gh.empty_dev(na * 4, fill=0x5A) for _ in range(p)]
        ob = [gh.empty_dev(nb * 4, fill=0x5A) for _ in range(p)]
        torch.cuda.synchronize()
        for rep in range(3):
            H.reduce_scatter_no_alloc(ga.comms, [t.data_ptr() for t in sa], [t.data_ptr() for t in oa], na, FP32, SUM, ga.stream_ptr)
            H.reduce_scatter_no_alloc(gb.comms, [t.data_ptr() for t in sb], [t.data_ptr() for t in ob], nb, FP32, SUM, gb.stream_ptr)
        ga.stream.synchronize()
        gb.stream.synchronize()
        for r in range(p):
            assert np.array_equal(gh.to_host(oa[r], FP32), want_a[r]), (fuse, "a", r)
            assert np.array_equal(gh.to_host(ob[r], FP32), want_b[r]), (fuse, "b", r)
    finally:
        ga.close()
        gb.close()


@pytest.mark.parametrize("fuse", [1, 0])
def test_reduce_scatter_no_alloc_recorded_into_a_callers_graph(orc, fuse):
    # the call under stream capture: the table uploads and the kernels become nodes of the caller's graph; every replay
    # rewrites the workspace's tables, also after an ordinary collective and another call of this kind ran in between
    p, n = 8, 30011
    g = gh.Group(p, fuse=fuse)
    try:
        rng = np.random.default_rng(6161 + fuse)
        sends = [torch.from_numpy(rng.standard_normal(n * p).astype(np.float32)).cuda() for _ in range(p)]
        got = [torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(p)]
        other = [torch.zeros(n * p, dtype=torch.float32, device="cuda") for _ in range(p)]
        small = [torch.zeros(16, dtype=torch.float32, device="cuda") for _ in range(p)]
        torch.cuda.synchronize()
        sp, gp = [t.data_ptr() for t in sends], [t.data_ptr() for t in got]
        H.reduce_scatter_no_alloc(g.comms, sp, gp, n, FP32, SUM, g.stream_ptr)        # eager, once
        g.stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(g.stream):
            graph.capture_begin()
            try:
                H.reduce_scatter_no_alloc(g.comms, sp, gp, n, FP32, SUM, g.stream_ptr)
            finally:
                graph.capture_end()
        for replay in range(3):
            for t in sends:
                t.mul_(1.5)
            torch.cuda.synchronize()
            want = orc.reducescatter([t.cpu().numpy() for t in sends], FP32, SUM)
            for t in got:
                t.zero_()
            # other users of the library and of the workspace between the replays
            H.all_reduce(g.comms, sp, [t.data_ptr() for t in other], n * p, FP32, SUM, g.stream_ptr)
            H.reduce_scatter_no_alloc(g.comms, sp, [t.data_ptr() for t in small], 16, FP32, SUM, g.stream_ptr)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for r in range(p):
                assert np.array_equal(got[r].cpu().numpy(), want[r]), (fuse, replay, r)
    finally:
        g.close()
