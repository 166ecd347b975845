"""The headline configuration at its real size on the GPU: 8 ranks, fp32 sum, 256 MiB per rank,
ring all-reduce.  Checked bit for bit against the CPU checker and through size-independent properties."""
import numpy as np
import pytest
import torch

import gpu_harness as gh
from closed_forms import FP32, SUM

pytestmark = pytest.mark.gpu
H = gh.H


def test_ring_allreduce_256mib_per_rank():
    from oracle import oracle as orc
    orc.build()
    p, n = 8, 64 << 20
    ins = [orc.fill_uniform_f32(n, 1234, r, threads=16) for r in range(p)]
    sends = [torch.from_numpy(x).cuda() for x in ins]
    torch.cuda.synchronize()
    results = {}
    for fuse in (1, 0):
        g = gh.Group(p, fuse=fuse)
        try:
            recvs = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(p)]
            torch.cuda.synchronize()
            print("full size all-reduce fuse", fuse, flush=True)
            H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, FP32, SUM, g.stream_ptr)
            g.stream.synchronize()
            info = g.info()
            S = n * 4
            if fuse:
                assert info["bytesRead"] == p * S and info["bytesWritten"] == p * S
            else:
                assert info["bytesRead"] + info["bytesWritten"] == 5 * (p - 1) * S
            # property: every rank holds the same bits
            for r in range(1, p):
                assert torch.equal(recvs[0], recvs[r]), (fuse, r)
            # property: send buffers untouched
            assert torch.equal(sends[3], torch.from_numpy(ins[3]).cuda())
            results[fuse] = recvs[0].cpu().numpy()
            del recvs
        finally:
            g.close()
    assert np.array_equal(results[1], results[0])            # fused and step-by-step agree bit for bit
    # the checker at full size (direct messages, no staging, 16 threads); its inputs are clobbered
    work = [x.copy() for x in ins]
    outs = [np.empty(n, np.float32) for _ in range(p)]
    orc.allreduce(work, FP32, SUM, flags=orc.DIRECT | orc.ZERO_STAGING, threads=16, outs=outs)
    assert np.array_equal(results[1], outs[0])
    assert np.array_equal(outs[0], outs[5])
    # property: all-reduce == all-gather of reduce-scatter (done with the library itself on a 1/8 sample)
    m = n // 8
    g = gh.Group(p)
    try:
        rs_out = [torch.empty(m // p, dtype=torch.float32, device="cuda") for _ in range(p)]
        ag_out = [torch.empty(m, dtype=torch.float32, device="cuda") for _ in range(p)]
        ar_out = [torch.empty(m, dtype=torch.float32, device="cuda") for _ in range(p)]
        part = [t[:m].contiguous() for t in sends]
        torch.cuda.synchronize()
        H.set_param(g.comms[0], "align", m * 4 // p)     # make the all-reduce slices equal the scatter blocks
        H.all_reduce(g.comms, [t.data_ptr() for t in part], [t.data_ptr() for t in ar_out], m, FP32, SUM, g.stream_ptr)
        H.reduce_scatter(g.comms, [t.data_ptr() for t in part], [t.data_ptr() for t in rs_out], m // p, FP32, SUM, g.stream_ptr)
        H.all_gather(g.comms, [t.data_ptr() for t in rs_out], [t.data_ptr() for t in ag_out], m // p, FP32, g.stream_ptr)
        g.stream.synchronize()
        for r in range(p):
            assert torch.equal(ar_out[r], ag_out[r]), r
    finally:
        g.close()


@pytest.mark.parametrize("p", [32, 24])
def test_rhd_allreduce_bf16_128mib_per_rank(p):
    """Recursive halving-doubling all-reduce, bf16 sum, 128 MiB per rank, 32 ranks (power of two) and 24 ranks
    (block of 16 plus 8 folded pairs): the fused tree kernel and the step-by-step schedule against the
    checker at full size, bit for bit (fp32 accumulation, one rounding per stored step in all three)."""
    from closed_forms import BF16
    from oracle import oracle as orc
    orc.build()
    n = 64 << 20                                     # bf16 elements per rank
    rng = np.random.default_rng(99 + p)
    # bf16 bit patterns with exponents near 1.0 (no Inf / NaN), every rank a different rotation of one block
    base = (rng.integers(0, 2, n, dtype=np.uint16) << 15) | (rng.integers(118, 132, n, dtype=np.uint16) << 7) | \
        rng.integers(0, 128, n, dtype=np.uint16)
    ins = [np.roll(base, 1237 * r + 1) ^ np.uint16(r & 0x7f) for r in range(p)]
    sends = [torch.from_numpy(x.view(np.int16)).cuda() for x in ins]
    torch.cuda.synchronize()
    results = {}
    for fuse in (1, 0):
        g = gh.Group(p, algo="rhd", fuse=fuse)
        try:
            recvs = [torch.empty(n, dtype=torch.int16, device="cuda") for _ in range(p)]
            torch.cuda.synchronize()
            print("full size rhd all-reduce p", p, "fuse", fuse, flush=True)
            H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, BF16, SUM, g.stream_ptr)
            g.stream.synchronize()
            assert g.info()["fused"] == fuse
            for r in range(1, p):
                assert torch.equal(recvs[0], recvs[r]), (fuse, r)      # every rank holds the same bits
            results[fuse] = recvs[0].cpu().numpy().view(np.uint16)
            del recvs
        finally:
            g.close()
    assert torch.equal(sends[p - 1], torch.from_numpy(ins[p - 1].view(np.int16)).cuda())   # inputs untouched
    assert np.array_equal(results[1], results[0])                      # fused and step-by-step agree bit for bit
    del sends
    print("checker at full size", flush=True)
    outs = [np.empty(n, np.uint16) for _ in range(p)]
    orc.allreduce(ins, BF16, SUM, algo=orc.RHD, flags=orc.DIRECT | orc.ZERO_STAGING, threads=16, outs=outs)   # clobbers ins
    assert np.array_equal(results[1], outs[0])
    assert np.array_equal(outs[0], outs[p - 1])


def test_buffers_larger_than_4_gib():
    """Two ranks with 5 GiB each: byte offsets inside a buffer go beyond 32 bits.  Integer sum, checked on the GPU
    against torch's own addition, fused and step by step, plus the all-gather of the same buffers' first GiB."""
    from closed_forms import INT32
    p, n = 2, (5 << 30) // 4
    sends = [torch.arange(n, dtype=torch.int32, device="cuda") * (3 + 4 * r) + r for r in range(p)]
    want = sends[0] + sends[1]
    torch.cuda.synchronize()
    for fuse in (1, 0):
        g = gh.Group(p, fuse=fuse)
        try:
            recvs = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(p)]
            torch.cuda.synchronize()
            print("5 GiB per rank all-reduce fuse", fuse, flush=True)
            H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, INT32, SUM, g.stream_ptr)
            g.stream.synchronize()
            for r in range(p):
                assert torch.equal(recvs[r], want), (fuse, r)
            del recvs
        finally:
            g.close()
    del want
    g = gh.Group(p)
    try:
        m = (3 << 30) // 4                      # 3 GiB in per rank: the second block of the output starts beyond 2^31 bytes
        outs = [torch.zeros(m * p, dtype=torch.int32, device="cuda") for _ in range(p)]
        torch.cuda.synchronize()
        H.all_gather(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in outs], m, INT32, g.stream_ptr)
        g.stream.synchronize()
        for r in range(p):
            for j in range(p):
                assert torch.equal(outs[r][j * m:(j + 1) * m], sends[j][:m]), (r, j)
    finally:
        g.close()
