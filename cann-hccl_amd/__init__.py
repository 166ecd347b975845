"""Host-side Python mirror of the HCCL C API served by lib/libhccl.so.

The library is the product; this module only binds it with ctypes (same function names, argument
order and return codes as include/hccl/hccl.h) so tests and the benchmark can call it.  Device
memory and streams come from the caller (raw pointers / hipStream_t values, e.g. torch's
tensor.data_ptr() and torch.cuda.current_stream().cuda_stream).

The package directory name contains a hyphen; load it with `load_package()` from
__graft_entry__.py, or via importlib from its path.
"""
import ctypes
import json
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libhccl.so")

# HcclResult (include/hccl/hccl_types.h)
HCCL_SUCCESS, HCCL_E_PARA, HCCL_E_PTR, HCCL_E_MEMORY, HCCL_E_INTERNAL, HCCL_E_NOT_SUPPORT = 0, 1, 2, 3, 4, 5
HCCL_E_NOT_FOUND, HCCL_E_UNAVAIL, HCCL_E_SYSCALL, HCCL_E_TIMEOUT = 6, 7, 8, 9
HCCL_E_RUNTIME, HCCL_E_AGAIN, HCCL_E_REMOTE, HCCL_E_SUSPENDING, HCCL_E_RESERVED = 15, 20, 21, 22, 23
# HcclReduceOp
HCCL_REDUCE_SUM, HCCL_REDUCE_PROD, HCCL_REDUCE_MAX, HCCL_REDUCE_MIN = 0, 1, 2, 3
# HcclDataType
(HCCL_DATA_TYPE_INT8, HCCL_DATA_TYPE_INT16, HCCL_DATA_TYPE_INT32, HCCL_DATA_TYPE_FP16, HCCL_DATA_TYPE_FP32,
 HCCL_DATA_TYPE_INT64, HCCL_DATA_TYPE_UINT64, HCCL_DATA_TYPE_UINT8, HCCL_DATA_TYPE_UINT16, HCCL_DATA_TYPE_UINT32,
 HCCL_DATA_TYPE_FP64, HCCL_DATA_TYPE_BFP16, HCCL_DATA_TYPE_INT128) = range(13)
DTYPE_SIZE = {0: 1, 1: 2, 2: 4, 3: 2, 4: 4, 5: 8, 6: 8, 7: 1, 8: 2, 9: 4, 10: 8, 11: 2, 12: 16}
COLL_ALLREDUCE, COLL_REDUCESCATTER, COLL_ALLGATHER, COLL_ALLTOALLV, COLL_BROADCAST, COLL_REDUCE, COLL_SCATTER = range(7)
ALGO_RING, ALGO_MESH, ALGO_RHD, ALGO_PAIRWISE = range(4)

# Every symbol include/hccl/hccl.h and include/hccl/hccl_amd_ext.h declare.
EXPORTS = [
    "HcclAllReduce", "HcclReduceScatter", "HcclAllGather", "HcclAlltoAllV", "HcclAlltoAll", "HcclAlltoAllVC", "HcclReduceScatterV",
    "HcclAllGatherV", "HcclBarrier", "HcclCommInitAll", "HcclCommDestroy", "HcclGetRankSize", "HcclGetRankId",
    "HcclGetCommName", "HcclSetConfig", "HcclGetConfig", "HcclGetCommAsyncError", "HcclGetErrorString",
    "HcclGetCommConfigCapability", "HcclCommSuspend", "HcclCommResume", "HcclCommInitClusterInfo",
    "HcclCommInitClusterInfoConfig", "HcclCreateSubCommConfig", "HcclGetRootInfo", "HcclCommInitRootInfo",
    "HcclCommInitRootInfoConfig", "HcclBroadcast", "HcclScatter", "HcclSend", "HcclRecv", "HcclReduce",
    "HcclBatchSendRecv", "HcclCommSetMemoryRange", "HcclCommUnsetMemoryRange", "HcclCommActivateCommMemory",
    "HcclCommDeactivateCommMemory", "HcclAmdSetParam", "HcclAmdGetLastOpInfo", "HcclAmdDescribePlan", "HcclAmdReduceScatterNoAlloc",
]


class HcclAmdOpInfo(ctypes.Structure):
    _fields_ = [("coll", ctypes.c_int32), ("algo", ctypes.c_int32), ("fused", ctypes.c_int32), ("graph", ctypes.c_int32),
                ("cacheHit", ctypes.c_int32), ("launches", ctypes.c_uint32), ("bytesRead", ctypes.c_uint64),
                ("bytesWritten", ctypes.c_uint64), ("schedRead", ctypes.c_uint64), ("schedWritten", ctypes.c_uint64),
                ("scratchBytes", ctypes.c_uint64), ("teamLaunches", ctypes.c_uint32), ("reserved", ctypes.c_uint32)]


class HcclCommConfig(ctypes.Structure):
    _fields_ = [("reserved", ctypes.c_char * 24), ("hcclBufferSize", ctypes.c_uint32), ("hcclDeterministic", ctypes.c_uint32),
                ("hcclCommName", ctypes.c_char * 128), ("hcclUdi", ctypes.c_char * 128), ("hcclOpExpansionMode", ctypes.c_uint32),
                ("hcclRdmaTrafficClass", ctypes.c_uint32), ("hcclRdmaServiceLevel", ctypes.c_uint32)]


def comm_config_init():
    """What the inline HcclCommConfigInit of hccl.h writes."""
    cfg = HcclCommConfig()
    hdr = ctypes.cast(ctypes.byref(cfg), ctypes.POINTER(ctypes.c_uint64))
    hdr[0] = ctypes.sizeof(HcclCommConfig)
    hdr[1] = 0xf0f0f0f0 | (5 << 32)          # magic word, version
    hdr[2] = 0
    cfg.hcclBufferSize = 0xffffffff
    cfg.hcclDeterministic = 0xffffffff
    cfg.hcclOpExpansionMode = 0
    cfg.hcclRdmaTrafficClass = 0xffffffff
    cfg.hcclRdmaServiceLevel = 0xffffffff
    return cfg


def comm_init_cluster_info(rank_table_path, n_ranks, config=None):
    """One HcclCommInitClusterInfo[Config] per rank of the rank table (a JSON file); returns the handles."""
    path = str(rank_table_path).encode()
    comms = []
    for r in range(n_ranks):
        c = ctypes.c_void_p()
        if config is None:
            _check("HcclCommInitClusterInfo", lib().HcclCommInitClusterInfo(path, r, ctypes.byref(c)))
        else:
            _check("HcclCommInitClusterInfoConfig", lib().HcclCommInitClusterInfoConfig(path, r, ctypes.byref(config),
                                                                                        ctypes.byref(c)))
        comms.append(c)
    return comms


def comm_init_root_info(n_ranks, config=None):
    """HcclGetRootInfo + one HcclCommInitRootInfo[Config] per rank; returns the handles."""
    info = ctypes.create_string_buffer(4108)
    _check("HcclGetRootInfo", lib().HcclGetRootInfo(info))
    comms = []
    for r in range(n_ranks):
        c = ctypes.c_void_p()
        if config is None:
            _check("HcclCommInitRootInfo", lib().HcclCommInitRootInfo(n_ranks, info, r, ctypes.byref(c)))
        else:
            _check("HcclCommInitRootInfoConfig", lib().HcclCommInitRootInfoConfig(n_ranks, info, r, ctypes.byref(config),
                                                                                  ctypes.byref(c)))
        comms.append(c)
    return comms


def create_sub_comm(comms, rank_ids, sub_comm_id, config=None):
    """HcclCreateSubCommConfig for every member; returns the sub-communicator handles in rank_ids order."""
    cfg = config or comm_config_init()
    ids = (ctypes.c_uint32 * len(rank_ids))(*rank_ids)
    subs = []
    for pos, r in enumerate(rank_ids):
        parent = ctypes.c_void_p(comms[r].value)
        sub = ctypes.c_void_p()
        _check("HcclCreateSubCommConfig", lib().HcclCreateSubCommConfig(ctypes.byref(parent), len(rank_ids), ids, sub_comm_id,
                                                                         pos, ctypes.byref(cfg), ctypes.byref(sub)))
        subs.append(sub)
    return subs


class HcclSendRecvItem(ctypes.Structure):
    _fields_ = [("sendRecvType", ctypes.c_int32), ("buf", ctypes.c_void_p), ("count", ctypes.c_uint64),
                ("dataType", ctypes.c_int32), ("remoteRank", ctypes.c_uint32)]


_lib = None


def lib():
    """Loads lib/libhccl.so; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        # nothing built yet (a fresh checkout): build once, in tree; a built library is never rebuilt from here
        import importlib.util
        spec = importlib.util.spec_from_file_location("cann_hccl_amd_build", os.path.join(os.path.dirname(__file__), "build.py"))
        builder = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(builder)
        try:
            builder.build()
        except Exception as e:   # noqa: BLE001
            raise RuntimeError("libhccl.so is not built and building it failed (needs hipcc): %s" % e)
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libhccl.so is not built: run `python cann-hccl_amd/build.py` (needs hipcc)")
    # Streams and device pointers handed to the library must belong to the HIP runtime the library
    # itself uses.  PyTorch ships its own libamdhip64 (same soname): when it is loaded first the
    # dynamic linker shares it with libhccl.so, the other way round the process ends up with two
    # runtimes.  So load PyTorch's first whenever PyTorch is installed.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    vp, u64, u32, i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int32
    L.HcclCommInitAll.argtypes = [u32, ctypes.POINTER(i32), ctypes.POINTER(vp)]
    L.HcclCommDestroy.argtypes = [vp]
    L.HcclGetRankSize.argtypes = [vp, ctypes.POINTER(u32)]
    L.HcclGetRankId.argtypes = [vp, ctypes.POINTER(u32)]
    L.HcclGetCommName.argtypes = [vp, ctypes.c_char_p]
    L.HcclAllReduce.argtypes = [vp, vp, u64, i32, i32, vp, vp]
    L.HcclReduceScatter.argtypes = [vp, vp, u64, i32, i32, vp, vp]
    L.HcclAmdReduceScatterNoAlloc.argtypes = [vp, vp, u64, i32, i32, vp, vp]
    L.HcclAllGather.argtypes = [vp, vp, u64, i32, vp, vp]
    L.HcclAlltoAllV.argtypes = [vp, vp, vp, i32, vp, vp, vp, i32, vp, vp]
    L.HcclAlltoAll.argtypes = [vp, u64, i32, vp, u64, i32, vp, vp]
    L.HcclAlltoAllVC.argtypes = [vp, vp, i32, vp, i32, vp, vp]
    L.HcclReduceScatterV.argtypes = [vp, vp, vp, vp, u64, i32, i32, vp, vp]
    L.HcclAllGatherV.argtypes = [vp, u64, vp, vp, vp, i32, vp, vp]
    L.HcclBarrier.argtypes = [vp, vp]
    L.HcclBroadcast.argtypes = [vp, u64, i32, u32, vp, vp]
    L.HcclReduce.argtypes = [vp, vp, u64, i32, i32, u32, vp, vp]
    L.HcclScatter.argtypes = [vp, vp, u64, i32, u32, vp, vp]
    L.HcclGetRootInfo.argtypes = [vp]
    L.HcclCommInitRootInfo.argtypes = [u32, vp, u32, ctypes.POINTER(vp)]
    L.HcclCommInitClusterInfo.argtypes = [ctypes.c_char_p, u32, ctypes.POINTER(vp)]
    L.HcclCommInitClusterInfoConfig.argtypes = [ctypes.c_char_p, u32, vp, ctypes.POINTER(vp)]
    L.HcclCommInitRootInfoConfig.argtypes = [u32, vp, u32, vp, ctypes.POINTER(vp)]
    L.HcclCreateSubCommConfig.argtypes = [ctypes.POINTER(vp), u32, ctypes.POINTER(u32), u64, u32, vp, ctypes.POINTER(vp)]
    L.HcclSend.argtypes = [vp, u64, i32, u32, vp, vp]
    L.HcclRecv.argtypes = [vp, u64, i32, u32, vp, vp]
    L.HcclBatchSendRecv.argtypes = [ctypes.POINTER(HcclSendRecvItem), u32, vp, vp]
    L.HcclGetErrorString.restype = ctypes.c_char_p
    L.HcclGetErrorString.argtypes = [i32]
    L.HcclGetCommConfigCapability.restype = u32
    L.HcclSetConfig.argtypes = [i32, i32]
    L.HcclGetConfig.argtypes = [i32, ctypes.POINTER(i32)]
    L.HcclGetCommAsyncError.argtypes = [vp, ctypes.POINTER(i32)]
    L.HcclCommSuspend.argtypes = [vp]
    L.HcclCommResume.argtypes = [vp]
    L.HcclAmdSetParam.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p]
    L.HcclAmdGetLastOpInfo.argtypes = [vp, ctypes.POINTER(HcclAmdOpInfo)]
    L.HcclAmdDescribePlan.argtypes = [i32, i32, u32, u64, i32, u64, u64, u64, ctypes.POINTER(u64), ctypes.c_char_p,
                                      ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)]
    _lib = L
    return L


class HcclError(RuntimeError):
    def __init__(self, fn, code):
        self.code = code
        super().__init__("%s returned %d (%s)" % (fn, code, lib().HcclGetErrorString(code).decode()))


def _check(fn, code):
    if code != HCCL_SUCCESS:
        raise HcclError(fn, code)


def comm_init_all(ndev):
    """HcclCommInitAll with device labels 0..ndev-1; returns the list of HcclComm handles."""
    devs = (ctypes.c_int32 * ndev)(*range(ndev))
    comms = (ctypes.c_void_p * ndev)()
    _check("HcclCommInitAll", lib().HcclCommInitAll(ndev, devs, comms))
    return [ctypes.c_void_p(c) for c in comms]


def comm_destroy(comms):
    for c in comms:
        _check("HcclCommDestroy", lib().HcclCommDestroy(c))


def set_param(comm, key, value):
    _check("HcclAmdSetParam", lib().HcclAmdSetParam(comm, key.encode(), str(value).encode()))


def last_op_info(comm):
    info = HcclAmdOpInfo()
    _check("HcclAmdGetLastOpInfo", lib().HcclAmdGetLastOpInfo(comm, ctypes.byref(info)))
    return {f[0]: getattr(info, f[0]) for f in HcclAmdOpInfo._fields_}


def all_reduce(comms, sends, recvs, count, dtype, op, stream):
    """One HcclAllReduce call per rank (pointers are ints); the last call issues the work."""
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclAllReduce", lib().HcclAllReduce(s, r, count, dtype, op, c, stream))


def reduce_scatter(comms, sends, recvs, recv_count, dtype, op, stream):
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclReduceScatter", lib().HcclReduceScatter(s, r, recv_count, dtype, op, c, stream))


def reduce_scatter_no_alloc(comms, sends, recvs, recv_count, dtype, op, stream):
    """HcclAmdReduceScatterNoAlloc on every rank: the reduce-scatter out of the fixed device workspace."""
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclAmdReduceScatterNoAlloc", lib().HcclAmdReduceScatterNoAlloc(s, r, recv_count, dtype, op, c, stream))


def all_gather(comms, sends, recvs, send_count, dtype, stream):
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclAllGather", lib().HcclAllGather(s, r, send_count, dtype, c, stream))


def all_to_all(comms, sends, recvs, count, dtype, stream):
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclAlltoAll", lib().HcclAlltoAll(s, count, dtype, r, count, dtype, c, stream))


def all_to_all_vc(comms, sends, recvs, matrix, dtype, stream):
    """matrix[i][j] = elements rank i sends to rank j (the same table goes to every rank)."""
    p = len(comms)
    flat = (ctypes.c_uint64 * (p * p))(*[int(matrix[i][j]) for i in range(p) for j in range(p)])
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclAlltoAllVC", lib().HcclAlltoAllVC(s, flat, dtype, r, dtype, c, stream))


def reduce_scatter_v(comms, sends, counts, displs, recvs, dtype, op, stream):
    p = len(comms)
    c = (ctypes.c_uint64 * p)(*[int(x) for x in counts])
    d = (ctypes.c_uint64 * p)(*[int(x) for x in displs])
    for r in range(p):
        _check("HcclReduceScatterV", lib().HcclReduceScatterV(sends[r], c, d, recvs[r], int(counts[r]), dtype, op, comms[r], stream))


def all_gather_v(comms, sends, recvs, counts, displs, dtype, stream):
    p = len(comms)
    c = (ctypes.c_uint64 * p)(*[int(x) for x in counts])
    d = (ctypes.c_uint64 * p)(*[int(x) for x in displs])
    for r in range(p):
        _check("HcclAllGatherV", lib().HcclAllGatherV(sends[r], int(counts[r]), recvs[r], c, d, dtype, comms[r], stream))


def broadcast(comms, bufs, count, dtype, root, stream):
    for c, b in zip(comms, bufs):
        _check("HcclBroadcast", lib().HcclBroadcast(b, count, dtype, root, c, stream))


def reduce(comms, sends, recvs, count, dtype, op, root, stream):
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclReduce", lib().HcclReduce(s, r, count, dtype, op, root, c, stream))


def scatter(comms, sends, recvs, recv_count, dtype, root, stream):
    """sends[r] may be None / 0 for ranks other than the root."""
    for c, s, r in zip(comms, sends, recvs):
        _check("HcclScatter", lib().HcclScatter(s, r, recv_count, dtype, root, c, stream))


def send(comm, buf, count, dtype, dest, stream):
    _check("HcclSend", lib().HcclSend(buf, count, dtype, dest, comm, stream))


def recv(comm, buf, count, dtype, src, stream):
    _check("HcclRecv", lib().HcclRecv(buf, count, dtype, src, comm, stream))


def batch_send_recv(comm, items, stream):
    """items: list of (is_send, buf, count, dtype, remote_rank)."""
    arr = (HcclSendRecvItem * len(items))()
    for i, (is_send, buf, count, dtype, remote) in enumerate(items):
        arr[i].sendRecvType = 0 if is_send else 1
        arr[i].buf = buf
        arr[i].count = count
        arr[i].dataType = dtype
        arr[i].remoteRank = remote
    _check("HcclBatchSendRecv", lib().HcclBatchSendRecv(arr, len(items), comm, stream))


def barrier(comms, stream):
    for c in comms:
        _check("HcclBarrier", lib().HcclBarrier(c, stream))


class _A2avTables(list):
    """Rows of four host uint64 tables, as addresses; keeps the arrays they point into alive."""


def a2av_tables(send_counts, sdispls, recv_counts, rdispls):
    """Per rank, the four host uint64[p] arrays HcclAlltoAllV takes (build once, reuse across calls).  Sequences of
    sequences or p x p numpy arrays (the latter cost no per-element conversion)."""
    p = len(send_counts)
    try:
        import numpy as np
    except ImportError:
        np = None
    if np is not None and all(isinstance(t, np.ndarray) for t in (send_counts, sdispls, recv_counts, rdispls)):
        keep = [np.ascontiguousarray(t, dtype=np.uint64) for t in (send_counts, sdispls, recv_counts, rdispls)]
        base = [t.ctypes.data for t in keep]
        out = _A2avTables([b + r * p * 8 for b in base] for r in range(p))
        out.keep = keep
        return out
    return [[(ctypes.c_uint64 * p)(*[int(x) for x in t[r]]) for t in (send_counts, sdispls, recv_counts, rdispls)]
            for r in range(p)]


def all_to_all_v(comms, sends, send_counts, sdispls, recvs, recv_counts, rdispls, dtype, stream, tables=None):
    """counts / displs: per rank, sequences of p integers (elements); or pass tables=a2av_tables(...)."""
    if tables is None:
        tables = a2av_tables(send_counts, sdispls, recv_counts, rdispls)
    fn = lib().HcclAlltoAllV
    for r, c in enumerate(comms):
        t = tables[r]
        _check("HcclAlltoAllV", fn(sends[r], t[0], t[1], dtype, recvs[r], t[2], t[3], dtype, c, stream))


def describe_plan(coll, algo, p, count, dtype, ccl_bytes=200 << 20, align=128, in_place_mask=0, tables=None):
    """Plan a collective without a GPU; returns the plan as a dict (see HcclAmdDescribePlan)."""
    tab = None
    if tables is not None and coll != COLL_ALLTOALLV:
        flat = [int(x) for t in tables for x in t]          # (counts, displs)
        tab = (ctypes.c_uint64 * len(flat))(*flat)
    elif tables is not None:
        flat = [int(x) for t in tables for row in t for x in row]
        tab = (ctypes.c_uint64 * len(flat))(*flat)
    cap = 1 << 20
    while True:
        buf = ctypes.create_string_buffer(cap)
        need = ctypes.c_size_t(0)
        rc = lib().HcclAmdDescribePlan(coll, algo, p, count, dtype, ccl_bytes, align, in_place_mask, tab, buf, cap,
                                       ctypes.byref(need))
        if rc == HCCL_E_MEMORY:
            cap = need.value + 16
            continue
        _check("HcclAmdDescribePlan", rc)
        return json.loads(buf.value.decode())
