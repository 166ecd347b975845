"""ctypes front end of the CPU checker (oracle/hccl_oracle.cc).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py.  The product library never loads it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhccl_oracle.so")

# HcclDataType / HcclReduceOp values (inc/hccl/hccl_types.h:58-87 of the reference).
INT8, INT16, INT32, FP16, FP32, INT64, UINT64, UINT8, UINT16, UINT32, FP64, BF16 = range(12)
SUM, PROD, MAX, MIN = range(4)
RING, MESH, RHD = range(3)
MESH_ATOMIC = 4   # mesh reduce phases without the piece cut, streams in index order
DIRECT = 1        # flags bit0: messages are pointers, not snapshots
ZERO_STAGING = 2  # flags bit1: templates run on the caller's buffers (input clobbered)

# numpy carrier type per HcclDataType (fp16 / bf16 travel as raw uint16 bit patterns)
NP_CARRIER = {
    INT8: np.int8, INT16: np.int16, INT32: np.int32, FP16: np.uint16, FP32: np.float32, INT64: np.int64,
    UINT64: np.uint64, UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32, FP64: np.float64, BF16: np.uint16,
}


def build(force=False):
    """Compile the checker with g++ (a few seconds)."""
    import fcntl
    src = os.path.join(_HERE, "hccl_oracle.cc")
    # one builder at a time (test workers start together): the others wait and then find the library up to date
    with open(os.path.join(_HERE, ".build.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
            subprocess.check_call(["make", "-C", _HERE, "-B", "libhccl_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        u64, u32, i32, vp = ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int, ctypes.c_void_p
        pu64 = ctypes.POINTER(ctypes.c_uint64)
        L.orc_dtype_size.restype = u64
        L.orc_dtype_size.argtypes = [i32]
        L.orc_ring_slices.argtypes = [u64, u32, u64, pu64, pu64]
        L.orc_rhd_params.argtypes = [u32, ctypes.POINTER(u32), ctypes.POINTER(u32)]
        L.orc_rhd_slices.argtypes = [u64, u32, u64, pu64, pu64]
        L.orc_cut_pieces.argtypes = [u32, pu64, pu64, u32, u64, pu64, pu64]
        L.orc_chunk_plan.restype = u32
        L.orc_chunk_plan.argtypes = [i32, u64, u64, u32, u64, u64, u32, pu64]
        L.orc_reduce.argtypes = [i32, i32, vp, vp, vp, u64]
        for name in ("orc_f32_to_bf16", "orc_bf16_to_f32", "orc_f32_to_fp16", "orc_fp16_to_f32"):
            getattr(L, name).argtypes = [vp, vp, u64]
        L.orc_allreduce.argtypes = [i32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, i32, u64, u64, i32, i32, pu64]
        L.orc_reducescatter.argtypes = [i32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, i32, u64, u64, i32, i32]
        L.orc_allgather.argtypes = [i32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, u64, u64, i32, i32]
        L.orc_allgather_two_level.argtypes = [i32, i32, u32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, u64, u64, i32, i32]
        L.orc_allgather_two_level.restype = i32
        L.orc_reducescatter_v.argtypes = [i32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), pu64, pu64, i32, i32, u64, i32, i32]
        L.orc_allgather_v.argtypes = [i32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), pu64, pu64, i32, i32, i32]
        L.orc_broadcast.argtypes = [u32, ctypes.POINTER(vp), u64, i32, u32, u64, u64, i32, i32]
        L.orc_reduce_to_root.argtypes = [u32, ctypes.POINTER(vp), vp, u64, i32, i32, u32, u64, i32, i32]
        L.orc_reduce_to_root_rhd.argtypes = [u32, ctypes.POINTER(vp), vp, u64, i32, i32, u32, u64, u64, i32, i32]
        L.orc_allreduce_two_level.argtypes = [i32, i32, u32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, i32, u64, u64,
                                              i32, i32]
        L.orc_reducescatter_two_level.argtypes = [i32, i32, u32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, i32, u64, u64,
                                                  i32, i32]
        L.orc_reducescatter_two_level_pruned.argtypes = [u32, u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, i32,
                                                         ctypes.POINTER(u32), u32, u64, u64, i32, i32]
        L.orc_reduce_to_root_two_level.argtypes = [i32, i32, u32, u32, ctypes.POINTER(vp), vp, u64, i32, i32, u32, u64, u64, i32, i32]
        L.orc_broadcast_rhd.argtypes = [u32, ctypes.POINTER(vp), u64, i32, u32, u64, u64, i32, i32]
        L.orc_broadcast_hd_blocks.argtypes = [u32, ctypes.POINTER(vp), u64, i32, u32, u64, i32, i32, ctypes.POINTER(u64)]
        L.orc_broadcast_hd_blocks_route.argtypes = [u32, u32, ctypes.POINTER(u32), u32]
        L.orc_broadcast_mesh.argtypes = [u32, ctypes.POINTER(vp), u64, i32, u32, u64, u64, i32, i32]
        L.orc_broadcast_star.argtypes = [u32, ctypes.POINTER(vp), u64, i32, u32, i32, i32, ctypes.POINTER(u64)]
        L.orc_broadcast_star.restype = i32
        L.orc_allreduce_ring_pruned.argtypes = [u32, ctypes.POINTER(vp), ctypes.POINTER(vp), u64, i32, i32, ctypes.POINTER(u32), u32,
                                                u64, u64, i32, i32]
        L.orc_broadcast_two_level_ring.argtypes = [u32, u32, u32, ctypes.POINTER(vp), u64, i32, u32, u64, u64, i32, i32, ctypes.POINTER(u64)]
        L.orc_broadcast_two_level.argtypes = [u32, u32, ctypes.POINTER(vp), u64, i32, u32, u64, u64, i32, i32, ctypes.POINTER(u64)]
        L.orc_reduce_to_root_mesh.argtypes = [u32, ctypes.POINTER(vp), vp, u64, i32, i32, u32, u64, u64, i32, i32, i32]
        L.orc_scatter.argtypes = [u32, vp, ctypes.POINTER(vp), u64, i32, u32, i32, i32]
        L.orc_scatter_ring.argtypes = [u32, vp, ctypes.POINTER(vp), u64, i32, u32, i32, i32]
        L.orc_scatter_ring.restype = i32
        L.orc_scatter_two_level.argtypes = [u32, u32, vp, ctypes.POINTER(vp), u64, i32, u32, u64, u64, i32, i32, ctypes.POINTER(u64), i32]
        L.orc_scatter_two_level.restype = i32
        L.orc_alltoallv.argtypes = [u32, ctypes.POINTER(vp), pu64, pu64, ctypes.POINTER(vp), pu64, pu64, i32, u64, i32, i32]
        L.orc_alltoallv_staged.argtypes = [u32, u32, ctypes.POINTER(vp), pu64, pu64, ctypes.POINTER(vp), pu64, pu64, i32, i32, i32]
        L.orc_alltoallv_staged.restype = i32
        L.orc_alltoallv_rounds.argtypes = [u32, pu64, pu64, i32, u64, pu64, pu64, pu64]
        L.orc_alltoallv_rounds.restype = i32
        L.orc_alltoallv_staged_rounds.argtypes = [u32, u32, pu64, i32, u64, pu64, pu64, pu64]
        L.orc_alltoallv_staged_rounds.restype = i32
        L.orc_fill_uniform_f32.argtypes = [vp, u64, u64, u32, i32]
        _lib = L
    return _lib


DEFAULT_CCL_BYTES = 200 << 20   # HCCL_COMM_DEFAULT_BUFFSIZE MiB (inc/hccl/hccl_types.h:112)
DEFAULT_ALIGN = 128


def dtype_size(dt):
    return int(lib().orc_dtype_size(dt))


def _u64arr(n):
    return (ctypes.c_uint64 * n)()


def ring_slices(total, p, align=DEFAULT_ALIGN):
    off, size = _u64arr(p), _u64arr(p)
    lib().orc_ring_slices(total, p, align, off, size)
    return list(off), list(size)


def rhd_params(p):
    b, q = ctypes.c_uint32(), ctypes.c_uint32()
    lib().orc_rhd_params(p, ctypes.byref(b), ctypes.byref(q))
    return b.value, q.value


def rhd_slices(total, block, align=DEFAULT_ALIGN):
    off, size = _u64arr(block), _u64arr(block)
    lib().orc_rhd_slices(total, block, align, off, size)
    return list(off), list(size)


def cut_pieces(offs, sizes, n, align=DEFAULT_ALIGN):
    k = len(offs)
    oi, si = _u64arr(k), _u64arr(k)
    oi[:] = offs
    si[:] = sizes
    oo, so = _u64arr(k * n), _u64arr(k * n)
    lib().orc_cut_pieces(k, oi, si, n, align, oo, so)
    return [[(oo[t * k + r], so[t * k + r]) for r in range(k)] for t in range(n)]


def chunk_plan(kind, count, unit, p, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN):
    buf = _u64arr(4096)
    n = lib().orc_chunk_plan(kind, count, unit, p, ccl_bytes, align, 4096, buf)
    return [int(buf[i]) for i in range(min(n, 4096))]


def _ptrs(arrs):
    a = (ctypes.c_void_p * len(arrs))()
    for i, x in enumerate(arrs):
        assert x.flags["C_CONTIGUOUS"]
        a[i] = x.ctypes.data
    return a


def reduce(dt, op, a, b):
    out = np.empty_like(a)
    rc = lib().orc_reduce(dt, op, out.ctypes.data, a.ctypes.data, b.ctypes.data, a.size)
    assert rc == 0
    return out


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16(x.ctypes.data, out.ctypes.data, x.size)
    return out


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().orc_bf16_to_f32(x.ctypes.data, out.ctypes.data, x.size)
    return out


def f32_to_fp16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_fp16(x.ctypes.data, out.ctypes.data, x.size)
    return out


def fp16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().orc_fp16_to_f32(x.ctypes.data, out.ctypes.data, x.size)
    return out


def allreduce(ins, dt, op, algo=RING, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1,
              outs=None, return_touched=False):
    """ins: list of p equal-length numpy arrays (carrier dtype).  Returns the p outputs."""
    p = len(ins)
    if outs is None:
        outs = [np.empty_like(x) for x in ins]
    touched = ctypes.c_uint64(0)
    rc = lib().orc_allreduce(algo, p, _ptrs(ins), _ptrs(outs), ins[0].size, dt, op, ccl_bytes, align, flags, threads,
                             ctypes.byref(touched))
    if rc != 0:
        raise RuntimeError("oracle allreduce failed rc=%d" % rc)
    return (outs, touched.value) if return_touched else outs


def allreduce_ring_pruned(ins, dt, op, nic_ranks, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1):
    """Ring all-reduce over 8 ranks of which only nic_ranks (1, 2 or 4, ascending) own a network port."""
    assert len(ins) == 8
    outs = [np.empty_like(x) for x in ins]
    nic = (ctypes.c_uint32 * len(nic_ranks))(*[int(x) for x in nic_ranks])
    rc = lib().orc_allreduce_ring_pruned(8, _ptrs(ins), _ptrs(outs), ins[0].size, dt, op, nic, len(nic_ranks), ccl_bytes, align,
                                         flags, threads)
    if rc != 0:
        raise RuntimeError("oracle port-pruned ring allreduce failed rc=%d" % rc)
    return outs


def allreduce_two_level(ins, dt, op, servers, level1=RING, atomic=False, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0,
                        threads=1, level0="mesh"):
    """`servers` groups of consecutive ranks; inside a group `level0`: "mesh" (piece cut, or uncut when `atomic`),
    "ring" (one ring in rank order) or "ring4" (the four rings of the 8-device ring topology, groups of 8);
    `level1` (RING or RHD) between the groups."""
    outs = [np.empty_like(x) for x in ins]
    mode = {"mesh": 1 if atomic else 0, "ring": 2, "ring4": 3}[level0]
    rc = lib().orc_allreduce_two_level(level1, mode, servers, len(ins), _ptrs(ins), _ptrs(outs), ins[0].size, dt, op,
                                       ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle two-level allreduce failed rc=%d" % rc)
    return outs


def reducescatter(ins, dt, op, algo=RING, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1):
    p = len(ins)
    assert ins[0].size % p == 0
    n = ins[0].size // p
    outs = [np.empty(n, dtype=ins[0].dtype) for _ in range(p)]
    rc = lib().orc_reducescatter(algo, p, _ptrs(ins), _ptrs(outs), n, dt, op, ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle reducescatter failed rc=%d" % rc)
    return outs


def reducescatter_two_level(ins, dt, op, servers, level1=RING, atomic=False, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN,
                            flags=0, threads=1, level0="mesh"):
    """`servers` groups of consecutive ranks: `level1` (RING or RHD) between the groups first, then inside a group
    `level0`: "mesh" (piece cut, or uncut when `atomic`), "ring" or "ring4"."""
    p = len(ins)
    assert ins[0].size % p == 0
    n = ins[0].size // p
    outs = [np.empty(n, dtype=ins[0].dtype) for _ in range(p)]
    mode = {"mesh": 1 if atomic else 0, "ring": 2, "ring4": 3}[level0]
    rc = lib().orc_reducescatter_two_level(level1, mode, servers, p, _ptrs(ins), _ptrs(outs), n, dt, op,
                                           ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle two-level reducescatter failed rc=%d" % rc)
    return outs


def reducescatter_two_level_pruned(ins, dt, op, servers, nic, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1):
    """Two-level ring reduce-scatter over servers of 8 devices of which only the devices in `nic` have a network port
    (the isMultiNic branch of coll_reduce_scatter_ring_executor.cc): all-reduce inside the servers, ring between the
    servers on the port devices, scatter inside the servers."""
    p = len(ins)
    n = ins[0].size // p
    outs = [np.empty(n, dtype=ins[0].dtype) for _ in range(p)]
    nic = sorted(nic)
    arr = (ctypes.c_uint32 * len(nic))(*nic)
    rc = lib().orc_reducescatter_two_level_pruned(servers, p, _ptrs(ins), _ptrs(outs), n, dt, op, arr, len(nic),
                                                  ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle port-pruned two-level reducescatter failed rc=%d" % rc)
    return outs


def allgather(ins, dt, algo=RING, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1):
    p = len(ins)
    n = ins[0].size
    outs = [np.empty(n * p, dtype=ins[0].dtype) for _ in range(p)]
    rc = lib().orc_allgather(algo, p, _ptrs(ins), _ptrs(outs), n, dt, ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle allgather failed rc=%d" % rc)
    return outs


def allgather_two_level(ins, dt, servers, level1=RING, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1,
                        level0="mesh"):
    """`servers` groups of consecutive ranks: the all-gather inside a group first (`level0`: "mesh", "ring" or
    "ring4"), then `level1` (RING or RHD) between the groups."""
    p = len(ins)
    n = ins[0].size
    outs = [np.empty(n * p, dtype=ins[0].dtype) for _ in range(p)]
    mode = {"mesh": 0, "ring": 2, "ring4": 3}[level0]
    rc = lib().orc_allgather_two_level(level1, mode, servers, p, _ptrs(ins), _ptrs(outs), n, dt, ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle two-level allgather failed rc=%d" % rc)
    return outs


def reducescatter_v(ins, counts, displs, dt, op, algo=RING, align=DEFAULT_ALIGN, flags=0, threads=1):
    """ins: p arrays holding the blocks {displs[i], counts[i]}; returns p arrays, rank r gets block r reduced."""
    p = len(ins)
    c, d = _u64arr(p), _u64arr(p)
    c[:] = [int(x) for x in counts]
    d[:] = [int(x) for x in displs]
    outs = [np.empty(int(counts[r]), dtype=ins[0].dtype) for r in range(p)]
    rc = lib().orc_reducescatter_v(algo, p, _ptrs(ins), _ptrs(outs), c, d, dt, op, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle reducescatter_v failed rc=%d" % rc)
    return outs


def allgather_v(ins, counts, displs, out_len, dt, algo=RING, flags=0, threads=1, fill=0):
    p = len(ins)
    c, d = _u64arr(p), _u64arr(p)
    c[:] = [int(x) for x in counts]
    d[:] = [int(x) for x in displs]
    outs = [np.full(out_len, fill, dtype=ins[0].dtype) for _ in range(p)]
    rc = lib().orc_allgather_v(algo, p, _ptrs(ins), _ptrs(outs), c, d, dt, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle allgather_v failed rc=%d" % rc)
    return outs


def broadcast(bufs, dt, root, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1, algo=RING):
    """bufs: p equal-length arrays, written in place: every array becomes bufs[root].  algo: RING, MESH or RHD."""
    fn = lib().orc_broadcast_mesh if algo == MESH else lib().orc_broadcast_rhd if algo == RHD else lib().orc_broadcast
    rc = fn(len(bufs), _ptrs(bufs), bufs[0].size, dt, root, ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle broadcast failed rc=%d" % rc)
    return bufs


def broadcast_star(bufs, dt, root, flags=0, threads=1, return_touched=False):
    """The root hands every rank the whole buffer, all at once.  bufs are written in place."""
    touched = ctypes.c_uint64(0)
    rc = lib().orc_broadcast_star(len(bufs), _ptrs(bufs), bufs[0].size, dt, root, flags, threads, ctypes.byref(touched))
    if rc != 0:
        raise RuntimeError("oracle star broadcast failed rc=%d" % rc)
    return (bufs, touched.value) if return_touched else bufs


def broadcast_hd_blocks(bufs, dt, root, ccl_bytes=DEFAULT_CCL_BYTES, flags=0, threads=1, return_touched=False):
    """Binary-block halving-doubling broadcast (bcast_halvingdoubling.cc): blocks of power-of-two sizes, a binomial tree
    inside the root's block, then block to block.  bufs are written in place."""
    touched = ctypes.c_uint64(0)
    rc = lib().orc_broadcast_hd_blocks(len(bufs), _ptrs(bufs), bufs[0].size, dt, root, ccl_bytes, flags, threads, ctypes.byref(touched))
    if rc != 0:
        raise RuntimeError("oracle binary-block broadcast failed rc=%d" % rc)
    return (bufs, touched.value) if return_touched else bufs


def broadcast_hd_blocks_route(p, root):
    """[(sender, receiver), ...] of the binary-block broadcast, rank by rank in program order."""
    cap = 4 * p + 4
    pairs = (ctypes.c_uint32 * (2 * cap))()
    n = lib().orc_broadcast_hd_blocks_route(p, root, pairs, cap)
    assert 0 <= n <= cap
    return [(pairs[2 * i], pairs[2 * i + 1]) for i in range(n)]


def broadcast_two_level_ring(bufs, dt, root, servers, rings=1, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1,
                             return_touched=False):
    """Two-level broadcast of the ring topologies (coll_broadcast_ring_executor.cc): ring scatter in the root's server over
    one ring or the four rings of the 8-device topology, halving-doubling between the servers, ring all-gather in every
    server.  bufs are written in place."""
    touched = ctypes.c_uint64(0)
    rc = lib().orc_broadcast_two_level_ring(servers, rings, len(bufs), _ptrs(bufs), bufs[0].size, dt, root, ccl_bytes, align,
                                            flags, threads, ctypes.byref(touched))
    if rc != 0:
        raise RuntimeError("oracle two-level ring broadcast failed rc=%d" % rc)
    return (bufs, touched.value) if return_touched else bufs


def broadcast_two_level(bufs, dt, root, servers, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1,
                        return_touched=False):
    """`servers` groups of consecutive ranks: scatter in the root's group, halving-doubling broadcast of slice d among
    the ranks at position d, mesh all-gather in every group.  bufs are written in place."""
    touched = ctypes.c_uint64(0)
    rc = lib().orc_broadcast_two_level(servers, len(bufs), _ptrs(bufs), bufs[0].size, dt, root, ccl_bytes, align, flags, threads,
                                       ctypes.byref(touched))
    if rc != 0:
        raise RuntimeError("oracle two-level broadcast failed rc=%d" % rc)
    return (bufs, touched.value) if return_touched else bufs


def reduce_to_root(ins, dt, op, root, ccl_bytes=DEFAULT_CCL_BYTES, flags=0, threads=1, algo=RING, align=DEFAULT_ALIGN):
    """algo: RING, MESH (piece cut), MESH_ATOMIC (uncut, streams in index order) or RHD."""
    out = np.empty_like(ins[0])
    if algo in (MESH, MESH_ATOMIC):
        rc = lib().orc_reduce_to_root_mesh(len(ins), _ptrs(ins), out.ctypes.data, ins[0].size, dt, op, root, ccl_bytes, align,
                                           1 if algo == MESH_ATOMIC else 0, flags, threads)
    elif algo == RHD:
        rc = lib().orc_reduce_to_root_rhd(len(ins), _ptrs(ins), out.ctypes.data, ins[0].size, dt, op, root, ccl_bytes, align,
                                          flags, threads)
    else:
        rc = lib().orc_reduce_to_root(len(ins), _ptrs(ins), out.ctypes.data, ins[0].size, dt, op, root, ccl_bytes, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle reduce failed rc=%d" % rc)
    return out


def reduce_to_root_two_level(ins, dt, op, root, servers, level1=RING, atomic=False, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN,
                             flags=0, threads=1, level0="mesh"):
    """`servers` groups of consecutive ranks: mesh reduce-scatter inside a group (piece cut, or uncut when `atomic`),
    `level1` (RING or RHD) reduce of every slice towards the root's group, gather to the root inside its group."""
    out = np.empty_like(ins[0])
    mode = {"mesh": 1 if atomic else 0, "ring": 2, "ring4": 3}[level0]
    rc = lib().orc_reduce_to_root_two_level(level1, mode, servers, len(ins), _ptrs(ins), out.ctypes.data, ins[0].size,
                                            dt, op, root, ccl_bytes, align, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle two-level reduce failed rc=%d" % rc)
    return out


def scatter(src, p, dt, root, flags=0, threads=1, algo=MESH):
    """algo: MESH (the root hands every rank its block directly) or RING (the blocks travel round the ring)."""
    n = src.size // p
    outs = [np.empty(n, dtype=src.dtype) for _ in range(p)]
    fn = lib().orc_scatter_ring if algo == RING else lib().orc_scatter
    rc = fn(p, src.ctypes.data, _ptrs(outs), n, dt, root, flags, threads)
    if rc != 0:
        raise RuntimeError("oracle scatter failed rc=%d" % rc)
    return outs


def scatter_two_level(src, p, dt, root, servers, ccl_bytes=DEFAULT_CCL_BYTES, align=DEFAULT_ALIGN, flags=0, threads=1,
                      return_touched=False, level0="mesh"):
    """`servers` groups of consecutive ranks: ring scatter of the groups' runs among the ranks at the root's position,
    then inside every group from that rank the mesh scatter, or the ring scatter along the ranks in their order ("ring")
    or in the order of ring 0 of the 8-device topology ("ring4"), under the staging buffer's chunk loop."""
    n = src.size // p
    outs = [np.empty(n, dtype=src.dtype) for _ in range(p)]
    touched = ctypes.c_uint64(0)
    rc = lib().orc_scatter_two_level(servers, p, src.ctypes.data, _ptrs(outs), n, dt, root, ccl_bytes, align, flags, threads,
                                     ctypes.byref(touched), {"mesh": 0, "ring": 1, "ring4": 2}[level0])
    if rc != 0:
        raise RuntimeError("oracle two-level scatter failed rc=%d" % rc)
    return (outs, touched.value) if return_touched else outs


def alltoallv(sends, send_counts, sdispls, recvs, recv_counts, rdispls, dt, scratch_bytes=0, flags=0, threads=1):
    """counts / displs: (p, p) uint64 arrays, row r = rank r's arguments.  recvs are written in place.
    Returns 0, or 1 when the send / receive tables are not symmetric."""
    p = len(sends)
    sc = np.ascontiguousarray(send_counts, dtype=np.uint64)
    sd = np.ascontiguousarray(sdispls, dtype=np.uint64)
    rc_ = np.ascontiguousarray(recv_counts, dtype=np.uint64)
    rd = np.ascontiguousarray(rdispls, dtype=np.uint64)
    pu64 = ctypes.POINTER(ctypes.c_uint64)
    rc = lib().orc_alltoallv(p, _ptrs(sends), sc.ctypes.data_as(pu64), sd.ctypes.data_as(pu64), _ptrs(recvs),
                             rc_.ctypes.data_as(pu64), rd.ctypes.data_as(pu64), dt, scratch_bytes, flags, threads)
    if rc not in (0, 1):
        raise RuntimeError("oracle alltoallv failed rc=%d" % rc)
    return rc


def alltoallv_rounds(send_counts, recv_counts, dt, scratch_bytes):
    """The BCopy form's transfer loop, per step: (rounds per step as a list, largest piece, bytes sent over all ranks)."""
    p = send_counts.shape[0]
    sc = np.ascontiguousarray(send_counts, dtype=np.uint64)
    rc = np.ascontiguousarray(recv_counts, dtype=np.uint64)
    rounds, biggest, total = _u64arr(p), ctypes.c_uint64(0), ctypes.c_uint64(0)
    pu64 = ctypes.POINTER(ctypes.c_uint64)
    rc_ = lib().orc_alltoallv_rounds(p, sc.ctypes.data_as(pu64), rc.ctypes.data_as(pu64), dt, scratch_bytes, rounds,
                                     ctypes.byref(biggest), ctypes.byref(total))
    if rc_ != 0:
        raise RuntimeError("oracle all-to-all-v rounds failed rc=%d" % rc_)
    return list(rounds), biggest.value, total.value


def alltoallv_staged_rounds(send_counts, servers, dt, scratch_bytes):
    """Second stage of the staged schedule in its buffer-copy form: (batches per step as a list of `servers` entries,
    list entries over all batches and ranks, bytes of the fullest batch)."""
    p = send_counts.shape[0]
    sc = np.ascontiguousarray(send_counts, dtype=np.uint64)
    rounds, entries, biggest = _u64arr(servers), ctypes.c_uint64(0), ctypes.c_uint64(0)
    rc_ = lib().orc_alltoallv_staged_rounds(p, servers, sc.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)), dt, scratch_bytes,
                                            rounds, ctypes.byref(entries), ctypes.byref(biggest))
    if rc_ != 0:
        raise RuntimeError("oracle staged all-to-all-v rounds failed rc=%d" % rc_)
    return list(rounds), entries.value, biggest.value


def alltoallv_staged(sends, send_counts, sdispls, recvs, recv_counts, rdispls, dt, servers, flags=0, threads=1):
    """The staged schedule over `servers` servers of equal size; arguments as alltoallv.  Returns 0, 1 (asymmetric
    tables) or 2 (servers of different sizes)."""
    p = len(sends)
    sc = np.ascontiguousarray(send_counts, dtype=np.uint64)
    sd = np.ascontiguousarray(sdispls, dtype=np.uint64)
    rc_ = np.ascontiguousarray(recv_counts, dtype=np.uint64)
    rd = np.ascontiguousarray(rdispls, dtype=np.uint64)
    pu64 = ctypes.POINTER(ctypes.c_uint64)
    rc = lib().orc_alltoallv_staged(p, servers, _ptrs(sends), sc.ctypes.data_as(pu64), sd.ctypes.data_as(pu64), _ptrs(recvs),
                                    rc_.ctypes.data_as(pu64), rd.ctypes.data_as(pu64), dt, flags, threads)
    if rc not in (0, 1, 2):
        raise RuntimeError("oracle staged alltoallv failed rc=%d" % rc)
    return rc


def fill_uniform_f32(n, seed, rank, threads=1, out=None):
    if out is None:
        out = np.empty(n, dtype=np.float32)
    lib().orc_fill_uniform_f32(out.ctypes.data, n, seed, rank, threads)
    return out
