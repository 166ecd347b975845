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


def _device_inputs(dt, p, n, seed):
    """Inputs of BASELINE.json's reduce-scatter configuration, made on the device: fp16 / bf16 ~ N(0, 1), int8 / int32
    uniform over the full range, int64 uniform in [-2^40, 2^40).  Returns device tensors and their host copies as
    carrier arrays."""
    from closed_forms import BF16, CARRIER, FP16, INT8, INT32, INT64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    dev = []
    for _ in range(p):
        if dt in (FP16, BF16):
            t = torch.randn(n, dtype=torch.float32, device="cuda", generator=gen).to(torch.float16 if dt == FP16 else torch.bfloat16)
        elif dt == INT64:
            t = torch.randint(-(1 << 40), 1 << 40, (n,), dtype=torch.int64, device="cuda", generator=gen)
        elif dt == INT32:
            t = torch.randint(-(1 << 31), 1 << 31, (n,), dtype=torch.int64, device="cuda", generator=gen).to(torch.int32)
        else:
            assert dt == INT8
            t = torch.randint(-128, 128, (n,), dtype=torch.int16, device="cuda", generator=gen).to(torch.int8)
        dev.append(t)
    torch.cuda.synchronize()
    host = [t.view(torch.int16).cpu().numpy().view(CARRIER[dt]) if dt in (FP16, BF16) else t.cpu().numpy() for t in dev]
    return dev, host


def test_reducescatter_64mib_per_rank_every_op_and_type():
    """BASELINE.json configs[2] in full: ring reduce-scatter over 8 ranks, 64 MiB per rank, {sum, prod, max, min} x
    {fp16, bf16, int8, int32, int64}, fused and step by step, against the checker at full size.  Integers bit-exact;
    fp16 / bf16 within 1 ulp (they come out bit-equal: both sides accumulate in fp32 and round once per stored step)."""
    from closed_forms import BF16, CARRIER, FP16, INT8, INT32, INT64, MAX, MIN, PROD
    from oracle import oracle as orc
    from test_gpu_parity import _ulp_close
    orc.build()
    p = 8
    bit_equal_16 = 0
    for dt in (FP16, BF16, INT8, INT32, INT64):
        unit = H.DTYPE_SIZE[dt]
        n = (64 << 20) // unit // p                          # elements each rank receives
        sends, ins = _device_inputs(dt, p, n * p, 4242 + dt)
        for op in (SUM, PROD, MAX, MIN):
            print("reduce-scatter 64 MiB per rank: type", dt, "op", op, flush=True)
            want = orc.reducescatter(ins, dt, op, flags=orc.DIRECT, threads=16)
            for fuse in (1, 0):
                g = gh.Group(p, fuse=fuse)
                try:
                    recvs = [gh.empty_dev(n * unit) for _ in range(p)]
                    torch.cuda.synchronize()
                    H.reduce_scatter(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, g.stream_ptr)
                    g.stream.synchronize()
                    assert g.info()["fused"] == fuse
                    for r in range(p):
                        got = gh.to_host(recvs[r], dt)
                        if dt in (FP16, BF16):
                            assert _ulp_close(dt, got, want[r]), (dt, op, fuse, r)       # the bar: within 1 ulp
                            bit_equal_16 += int(gh.same(dt, got, want[r]))
                        else:
                            assert np.array_equal(got, want[r]), (dt, op, fuse, r)
                    del recvs
                finally:
                    g.close()
        # the inputs are still what they were
        assert np.array_equal(sends[p - 1].view(torch.int16).cpu().numpy().view(CARRIER[dt]) if dt in (FP16, BF16)
                              else sends[p - 1].cpu().numpy(), ins[p - 1])
        del sends, ins
    assert bit_equal_16 == 2 * 4 * 2 * p                      # and in fact every 16-bit float result was bit-equal


def test_ring_allreduce_size_sweep_8kib_to_256mib():
    """BASELINE.json configs[1]: ring all-reduce, sum, fp32, 8 ranks, every size of the sweep (8 KiB ... 256 MiB per
    rank, doubling), fused and step by step, bit for bit against the checker; inputs uniform in [-1, 1) from a seed."""
    from oracle import oracle as orc
    orc.build()
    p, nmax = 8, 64 << 20
    ins = [orc.fill_uniform_f32(nmax, 77, r, threads=16) for r in range(p)]
    sends = [torch.from_numpy(x).cuda() for x in ins]
    recvs = [torch.empty(nmax, dtype=torch.float32, device="cuda") for _ in range(p)]
    torch.cuda.synchronize()
    groups = {fuse: gh.Group(p, fuse=fuse) for fuse in (1, 0)}
    try:
        size = 8 << 10
        sizes = []
        while size <= (256 << 20):
            sizes.append(size)
            size *= 2
        assert len(sizes) == 16
        for size in sizes:
            n = size // 4
            work = [x[:n].copy() for x in ins]
            outs = [np.empty(n, np.float32) for _ in range(p)]
            orc.allreduce(work, FP32, SUM, flags=orc.DIRECT | orc.ZERO_STAGING, threads=16, outs=outs)
            for fuse in (1, 0):
                g = groups[fuse]
                print("all-reduce sweep: bytes per rank", size, "fuse", fuse, flush=True)
                for t in recvs:
                    t[:n].zero_()
                torch.cuda.synchronize()
                H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, FP32, SUM, g.stream_ptr)
                g.stream.synchronize()
                assert g.info()["fused"] == fuse
                for r in (0, 3, p - 1):
                    assert np.array_equal(recvs[r][:n].cpu().numpy(), outs[r]), (size, fuse, r)
                for r in range(1, p):
                    assert torch.equal(recvs[0][:n], recvs[r][:n]), (size, fuse, r)
    finally:
        for g in groups.values():
            g.close()
