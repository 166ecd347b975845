"""Moves numpy rank buffers to the GPU, calls the library through its C ABI, brings results back.
torch is used for device memory and streams only."""
import numpy as np
import torch

import closed_forms as cf
from hccl_loader import load

H = load()


class Group:
    def __init__(self, p, **params):
        self.p = p
        self.comms = H.comm_init_all(p)
        self.stream = torch.cuda.Stream()
        for k, v in params.items():
            H.set_param(self.comms[0], k, v)

    def set(self, **params):
        for k, v in params.items():
            H.set_param(self.comms[0], k, v)

    def close(self):
        torch.cuda.synchronize()
        H.comm_destroy(self.comms)

    def info(self):
        return H.last_op_info(self.comms[0])

    @property
    def stream_ptr(self):
        return self.stream.cuda_stream


def to_dev(arr, pad_front=0):
    """numpy array -> uint8 device tensor; pad_front bytes shift the data off its natural alignment."""
    raw = torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).copy())
    if pad_front == 0:
        return raw.cuda()
    t = torch.empty(raw.numel() + 256, dtype=torch.uint8, device="cuda")
    t[pad_front:pad_front + raw.numel()].copy_(raw)
    return t[pad_front:pad_front + raw.numel()]


def empty_dev(nbytes, pad_front=0, fill=0xA5):
    t = torch.full((nbytes + 256,), fill, dtype=torch.uint8, device="cuda")
    return t[pad_front:pad_front + nbytes]


def to_host(t, dt):
    return t.cpu().numpy().view(cf.CARRIER[dt])


def same(dt, got, want):
    if dt in (cf.FP16, cf.BF16, cf.FP32, cf.FP64):
        g, w = cf.widen(dt, got).astype(np.float64), cf.widen(dt, want).astype(np.float64)
        nn = np.isnan(g) & np.isnan(w)
        return np.array_equal(got[~nn], want[~nn])
    return np.array_equal(got, want)


def all_reduce(g, ins, dt, op, in_place=False, pad=0):
    unit = H.DTYPE_SIZE[dt]
    n = ins[0].size
    sends = [to_dev(x, pad) for x in ins]
    recvs = sends if in_place else [empty_dev(n * unit, pad) for _ in ins]
    torch.cuda.synchronize()
    H.all_reduce(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, g.stream_ptr)
    g.stream.synchronize()
    outs = [to_host(t, dt) for t in recvs]
    keep = None if in_place else [to_host(t, dt) for t in sends]
    return outs, keep


def reduce_scatter(g, ins, dt, op, pad=0):
    unit = H.DTYPE_SIZE[dt]
    n = ins[0].size // g.p
    sends = [to_dev(x, pad) for x in ins]
    recvs = [empty_dev(n * unit, pad) for _ in ins]
    torch.cuda.synchronize()
    H.reduce_scatter(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, op, g.stream_ptr)
    g.stream.synchronize()
    return [to_host(t, dt) for t in recvs], [to_host(t, dt) for t in sends]


def all_gather(g, ins, dt, pad=0):
    unit = H.DTYPE_SIZE[dt]
    n = ins[0].size
    sends = [to_dev(x, pad) for x in ins]
    recvs = [empty_dev(n * unit * g.p, pad) for _ in ins]
    torch.cuda.synchronize()
    H.all_gather(g.comms, [t.data_ptr() for t in sends], [t.data_ptr() for t in recvs], n, dt, g.stream_ptr)
    g.stream.synchronize()
    return [to_host(t, dt) for t in recvs]


def all_to_all_v(g, sends_np, cnt, sdis, recv_lens, rcnt, rdis, dt, fill=-1):
    sends = [to_dev(x) for x in sends_np]
    recvs = [to_dev(np.full(n, fill, cf.CARRIER[dt])) for n in recv_lens]
    torch.cuda.synchronize()
    H.all_to_all_v(g.comms, [t.data_ptr() for t in sends], cnt, sdis, [t.data_ptr() for t in recvs], rcnt, rdis, dt,
                   g.stream_ptr)
    g.stream.synchronize()
    return [to_host(t, dt) for t in recvs]
