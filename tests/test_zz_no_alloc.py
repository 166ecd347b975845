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
