"""C-ABI conformance without a GPU: every declared symbol is exported, argument checks return the
reference's codes in the reference's order (op_base.cc / param_check.cc), and the rendezvous of the
simulated ranks behaves (mismatch, suspend / resume, time-out)."""
import ctypes
import re
import os
import threading

import pytest

from hccl_loader import load, ROOT

H = load()
L = H.lib()
STREAM = ctypes.c_void_p(0x1000)     # any non-null value: never dereferenced before a launch
BUF_A, BUF_B = ctypes.c_void_p(0x10000), ctypes.c_void_p(0x20000)


@pytest.fixture
def comms():
    cs = H.comm_init_all(4)
    yield cs
    for c in cs:
        assert L.HcclCommDestroy(c) in (H.HCCL_SUCCESS, H.HCCL_E_PARA)   # a pending rendezvous is dropped


def test_library_exports_every_declared_symbol():
    declared = set()
    for header in ("hccl.h", "hccl_amd_ext.h"):
        text = open(os.path.join(ROOT, "include", "hccl", header)).read()
        declared |= set(re.findall(r"extern\s+(?:const\s+)?[\w\s\*]+?\b(Hccl\w+)\s*\(", text))
    assert declared == set(H.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name


def test_error_strings():
    assert L.HcclGetErrorString(0) == b"no error"
    assert L.HcclGetErrorString(1) == b"parameter error"
    assert L.HcclGetErrorString(2) == b"empty pointer"
    assert L.HcclGetErrorString(9) == b"timeout"
    assert L.HcclGetErrorString(21) == b"error cqe"
    assert L.HcclGetErrorString(23) == b"unknow error"
    assert L.HcclGetErrorString(-1) == b"unknow error"
    assert L.HcclGetCommConfigCapability() == 5


def test_comm_init_all_checks():
    devs = (ctypes.c_int32 * 4)(0, 1, 2, 3)
    out = (ctypes.c_void_p * 4)()
    assert L.HcclCommInitAll(0, devs, out) == H.HCCL_E_PARA
    assert L.HcclCommInitAll(4, devs, None) == H.HCCL_E_PTR
    assert L.HcclCommInitAll(4, None, out) == H.HCCL_E_PTR
    dup = (ctypes.c_int32 * 4)(0, 1, 1, 3)
    assert L.HcclCommInitAll(4, dup, out) == H.HCCL_E_PARA


def test_rank_queries(comms):
    n, r = ctypes.c_uint32(), ctypes.c_uint32()
    for i, c in enumerate(comms):
        assert L.HcclGetRankSize(c, ctypes.byref(n)) == 0 and n.value == 4
        assert L.HcclGetRankId(c, ctypes.byref(r)) == 0 and r.value == i
    assert L.HcclGetRankSize(None, ctypes.byref(n)) == H.HCCL_E_PTR
    assert L.HcclGetRankSize(comms[0], None) == H.HCCL_E_PTR
    name = ctypes.create_string_buffer(128)
    assert L.HcclGetCommName(comms[0], name) == 0 and name.value
    assert L.HcclCommDestroy(None) == H.HCCL_SUCCESS


def test_allreduce_check_order(comms):
    c = comms[0]
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    # count == 0 succeeds before any pointer check
    assert L.HcclAllReduce(None, None, 0, FP32, SUM, None, None) == H.HCCL_SUCCESS
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, None, STREAM) == H.HCCL_E_PTR
    assert L.HcclAllReduce(None, BUF_B, 8, FP32, SUM, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAllReduce(BUF_A, None, 8, FP32, SUM, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAllReduce(BUF_A, BUF_B, 0x800000000, FP32, SUM, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, 13, SUM, c, STREAM) == H.HCCL_E_NOT_SUPPORT      # hif8
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, 255, SUM, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, c, None) == H.HCCL_E_PTR             # null stream
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, 7, c, STREAM) == H.HCCL_E_NOT_SUPPORT      # bad op
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, H.HCCL_DATA_TYPE_INT128, SUM, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclAllReduce(ctypes.c_void_p(0x10001), BUF_B, 8, FP32, SUM, c, STREAM) == H.HCCL_E_PARA  # misaligned


def test_reducescatter_allgather_checks(comms):
    c = comms[0]
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    assert L.HcclReduceScatter(None, None, 0, FP32, SUM, None, None) == H.HCCL_SUCCESS
    assert L.HcclReduceScatter(BUF_A, BUF_B, 4, FP32, SUM, None, STREAM) == H.HCCL_E_PTR
    assert L.HcclReduceScatter(BUF_A, BUF_B, 4, FP32, 9, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclAllGather(None, None, 0, FP32, None, None) == H.HCCL_SUCCESS
    assert L.HcclAllGather(BUF_A, None, 4, FP32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAllGather(BUF_A, BUF_B, 4, 99, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclAllGather(BUF_A, BUF_B, 4, FP32, c, None) == H.HCCL_E_PTR


def test_alltoallv_checks(comms):
    c = comms[0]
    I32 = H.HCCL_DATA_TYPE_INT32
    ones = (ctypes.c_uint64 * 4)(1, 1, 1, 1)
    zeros = (ctypes.c_uint64 * 4)(0, 0, 0, 0)
    big = (ctypes.c_uint64 * 4)(1, 0x800000000, 1, 1)
    assert L.HcclAlltoAllV(BUF_A, None, ones, I32, BUF_B, ones, ones, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAllV(BUF_A, ones, ones, I32, BUF_B, ones, ones, I32, c, None) == H.HCCL_E_PTR
    assert L.HcclAlltoAllV(BUF_A, ones, ones, I32, BUF_B, ones, ones, I32, None, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAllV(BUF_A, ones, ones, I32, BUF_A, ones, ones, I32, c, STREAM) == H.HCCL_E_PARA   # same buffer
    assert L.HcclAlltoAllV(BUF_A, big, ones, I32, BUF_B, ones, ones, I32, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclAlltoAllV(None, ones, ones, I32, BUF_B, ones, ones, I32, c, STREAM) == H.HCCL_E_PTR     # sends something
    assert L.HcclAlltoAllV(BUF_A, ones, ones, 14, BUF_B, ones, ones, I32, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    # a rank that neither sends nor receives may pass null buffers: it only joins the rendezvous
    assert L.HcclAlltoAllV(None, zeros, zeros, I32, None, zeros, zeros, I32, c, STREAM) == H.HCCL_SUCCESS


def test_sibling_entry_checks(comms):
    c = comms[0]
    I32, SUM = H.HCCL_DATA_TYPE_INT32, H.HCCL_REDUCE_SUM
    ones = (ctypes.c_uint64 * 4)(1, 1, 1, 1)
    zeros = (ctypes.c_uint64 * 4)(0, 0, 0, 0)
    # HcclAlltoAll (op_base.cc:2422): both counts 0 -> success first; then buffers, equal counts / types, stream, comm
    assert L.HcclAlltoAll(None, 0, I32, None, 0, I32, None, None) == H.HCCL_SUCCESS
    assert L.HcclAlltoAll(None, 4, I32, BUF_B, 4, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAll(BUF_A, 4, I32, BUF_B, 8, I32, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclAlltoAll(BUF_A, 4, I32, BUF_B, 4, H.HCCL_DATA_TYPE_FP32, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclAlltoAll(BUF_A, 4, I32, BUF_B, 4, I32, c, None) == H.HCCL_E_PTR
    assert L.HcclAlltoAll(BUF_A, 4, I32, BUF_A, 4, I32, c, STREAM) == H.HCCL_E_PARA
    # HcclAlltoAllVC (op_base.cc:2633, param_check.cc:205-242): 4 x 4 matrix of element counts
    m1 = (ctypes.c_uint64 * 16)(*([1] * 16))
    mbig = (ctypes.c_uint64 * 16)(*([0x800000000] * 16))
    assert L.HcclAlltoAllVC(BUF_A, None, I32, BUF_B, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAllVC(BUF_A, m1, I32, BUF_B, I32, None, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAllVC(BUF_A, m1, I32, BUF_A, I32, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclAlltoAllVC(BUF_A, mbig, I32, BUF_B, I32, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclAlltoAllVC(None, m1, I32, BUF_B, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAllVC(BUF_A, m1, I32, None, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAlltoAllVC(BUF_A, m1, I32, BUF_B, I32, c, None) == H.HCCL_E_PTR
    assert L.HcclAlltoAllVC(BUF_A, m1, 14, BUF_B, I32, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclAlltoAllVC(BUF_A, m1, I32, BUF_B, 14, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    # HcclReduceScatterV (op_base.cc:1585)
    assert L.HcclReduceScatterV(BUF_A, None, ones, BUF_B, 1, I32, SUM, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclReduceScatterV(BUF_A, ones, ones, None, 1, I32, SUM, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclReduceScatterV(BUF_A, zeros, zeros, None, 0, I32, SUM, c, STREAM) == H.HCCL_SUCCESS   # nothing to reduce
    assert L.HcclReduceScatterV(None, ones, ones, BUF_B, 1, I32, SUM, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclReduceScatterV(BUF_A, ones, ones, BUF_B, 2, I32, SUM, c, STREAM) == H.HCCL_E_PARA       # recvCount != sendCounts[rank]
    assert L.HcclReduceScatterV(BUF_A, ones, ones, BUF_B, 1, I32, 9, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    # HcclAllGatherV (op_base.cc:1863)
    assert L.HcclAllGatherV(BUF_A, 1, BUF_B, None, ones, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAllGatherV(None, 1, BUF_B, ones, ones, I32, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclAllGatherV(None, 0, None, zeros, zeros, I32, c, STREAM) == H.HCCL_SUCCESS
    assert L.HcclAllGatherV(BUF_A, 2, BUF_B, ones, ones, I32, c, STREAM) == H.HCCL_E_PARA
    # HcclBarrier (op_base.cc:1353)
    assert L.HcclBarrier(None, STREAM) == H.HCCL_E_PTR
    assert L.HcclBarrier(c, None) == H.HCCL_E_PTR
    # ranks that pass different block tables do not form a collective
    twos = (ctypes.c_uint64 * 4)(2, 1, 1, 1)
    assert L.HcclReduceScatterV(BUF_A, ones, ones, BUF_B, 1, I32, SUM, comms[1], STREAM) == H.HCCL_SUCCESS
    assert L.HcclReduceScatterV(BUF_A, twos, ones, BUF_B, 1, I32, SUM, comms[2], STREAM) == H.HCCL_E_PARA


def test_mismatched_ranks_are_rejected(comms):
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[0], STREAM) == H.HCCL_SUCCESS
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[0], STREAM) == H.HCCL_E_AGAIN      # same rank twice
    assert L.HcclAllReduce(BUF_A, BUF_B, 16, FP32, SUM, comms[1], STREAM) == H.HCCL_E_PARA      # other count
    # the failed rendezvous was dropped: a fresh one starts cleanly
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[1], STREAM) == H.HCCL_SUCCESS
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, H.HCCL_REDUCE_MAX, comms[2], STREAM) == H.HCCL_E_PARA


def test_suspend_resume(comms):
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    assert L.HcclCommSuspend(None) == H.HCCL_E_PTR
    assert L.HcclCommSuspend(comms[0]) == H.HCCL_SUCCESS
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[1], STREAM) == H.HCCL_E_SUSPENDING
    assert L.HcclCommResume(comms[0]) == H.HCCL_SUCCESS
    assert L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[1], STREAM) == H.HCCL_SUCCESS
    err = ctypes.c_int32(-1)
    assert L.HcclGetCommAsyncError(comms[0], ctypes.byref(err)) == 0 and err.value == 0


def test_blocking_arrival_times_out(comms):
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    H.set_param(comms[0], "blocking_arrive", 1)
    H.set_param(comms[0], "arrive_timeout_ms", 50)
    results = {}

    def call(r):
        results[r] = L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[r], STREAM)

    ts = [threading.Thread(target=call, args=(r,)) for r in (0, 1)]    # ranks 2 and 3 never call
    for t in ts:
        t.start()
    for t in ts:
        t.join(10)
    # whichever rank's wait runs out first ends the rendezvous; the other one wakes up with the same verdict
    assert results == {0: H.HCCL_E_TIMEOUT, 1: H.HCCL_E_TIMEOUT}, results


def test_blocked_rank_learns_of_a_mismatch(comms):
    # rank 0 waits inside its call; rank 1 then joins with another count: both get HCCL_E_PARA
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    H.set_param(comms[0], "blocking_arrive", 1)
    H.set_param(comms[0], "arrive_timeout_ms", 5000)
    results = {}

    def first():
        results[0] = L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, comms[0], STREAM)

    t = threading.Thread(target=first)
    t.start()
    import time
    time.sleep(0.2)
    results[1] = L.HcclAllReduce(BUF_A, BUF_B, 9, FP32, SUM, comms[1], STREAM)
    t.join(10)
    assert results == {0: H.HCCL_E_PARA, 1: H.HCCL_E_PARA}, results


def test_set_config_deterministic():
    if "HCCL_DETERMINISTIC" in os.environ:
        pytest.skip("environment overrides the switch")
    v = ctypes.c_int32(-1)
    assert L.HcclSetConfig(0, 2) == H.HCCL_E_PARA
    assert L.HcclSetConfig(0, 1) == H.HCCL_SUCCESS
    assert L.HcclGetConfig(0, ctypes.byref(v)) == 0 and v.value == 1
    assert L.HcclSetConfig(0, 0) == H.HCCL_SUCCESS
    assert L.HcclGetConfig(0, ctypes.byref(v)) == 0 and v.value == 0
    assert L.HcclGetConfig(0, None) == H.HCCL_E_PTR


def test_amd_params(comms):
    assert L.HcclAmdSetParam(comms[0], b"algo", b"mesh") == 0
    assert L.HcclAmdSetParam(comms[0], b"algo", b"bogus") == H.HCCL_E_PARA
    assert L.HcclAmdSetParam(comms[0], b"nonsense", b"1") == H.HCCL_E_PARA
    assert L.HcclAmdSetParam(comms[0], b"buffsize_mib", b"0") == H.HCCL_E_PARA
    assert L.HcclAmdSetParam(None, b"algo", b"ring") == H.HCCL_E_PTR
    # every documented key takes its documented values and nothing else
    good = {b"algo": [b"ring", b"mesh", b"rhd", b"pairwise", b"auto"], b"deterministic": [b"0", b"1"], b"fuse": [b"0", b"1"],
            b"graph": [b"0", b"1"], b"buffsize_mib": [b"1", b"200"], b"buffsize_bytes": [b"4096"], b"align": [b"4", b"128"],
            b"level0": [b"mesh", b"ring", b"ring4"], b"step_stores": [b"auto", b"nt", b"ordinary"],
            b"fused_stores": [b"auto", b"nt", b"ordinary"], b"step_sweep": [b"forward", b"alternate"], b"cache_entries": [b"1", b"1024"], b"blocks_per_cu": [b"0", b"2"],
            b"blocking_arrive": [b"0", b"1"], b"arrive_timeout_ms": [b"1000"]}
    for key, values in good.items():
        for v in values:
            assert L.HcclAmdSetParam(comms[0], key, v) == 0, (key, v)
    # network ports are named for groups of 8 ranks only (this group has 4)
    assert L.HcclAmdSetParam(comms[0], b"nic_ranks", b"all") == 0
    assert L.HcclAmdSetParam(comms[0], b"nic_ranks", b"0,2") == H.HCCL_E_PARA
    eight = H.comm_init_all(8)
    for v in (b"0", b"0,4", b"7,3", b"0,2,4,6", b"0,1,2,3,4,5,6,7", b"all", b""):
        assert L.HcclAmdSetParam(eight[0], b"nic_ranks", v) == 0, v
    for v in (b"0,1,2", b"8", b"0,0", b"x", b"0,,1", b"-1", b"0,1,2,3,4"):
        assert L.HcclAmdSetParam(eight[0], b"nic_ranks", v) == H.HCCL_E_PARA, v
    H.comm_destroy(eight)
    bad = {b"level0": b"star", b"step_stores": b"maybe", b"fused_stores": b"maybe", b"cache_entries": b"0", b"align": b"0",
           b"servers": b"0"}
    for key, v in bad.items():
        assert L.HcclAmdSetParam(comms[0], key, v) == H.HCCL_E_PARA, (key, v)
    p = ctypes.c_uint32(0)
    assert L.HcclGetRankSize(comms[0], ctypes.byref(p)) == 0
    assert L.HcclAmdSetParam(comms[0], b"servers", str(p.value).encode()) == 0            # every rank its own group
    assert L.HcclAmdSetParam(comms[0], b"servers", str(p.value + 1).encode()) == H.HCCL_E_PARA   # does not divide the ranks
    for key, v in ((b"algo", b"auto"), (b"servers", b"1"), (b"level0", b"mesh"), (b"fuse", b"1"), (b"graph", b"1"),
                   (b"deterministic", b"0"), (b"step_stores", b"auto"), (b"fused_stores", b"nt"), (b"step_sweep", b"alternate"), (b"blocking_arrive", b"0"),
                   (b"buffsize_mib", b"200"), (b"align", b"128"), (b"blocks_per_cu", b"0"), (b"cache_entries", b"1024")):
        assert L.HcclAmdSetParam(comms[0], key, v) == 0                                   # back to the defaults


def test_unsupported_entry_points_link_and_refuse(comms):
    assert L.HcclCommSetMemoryRange(comms[0], BUF_A, 4096, 0, 0) == H.HCCL_E_NOT_SUPPORT


def test_send_recv_checks_and_matching(comms):
    FP32 = H.HCCL_DATA_TYPE_FP32
    assert L.HcclSend(None, 0, FP32, 1, None, None) == H.HCCL_SUCCESS                       # count 0 first
    assert L.HcclSend(BUF_A, 4, FP32, 1, None, STREAM) == H.HCCL_E_PTR
    assert L.HcclSend(None, 4, FP32, 1, comms[0], STREAM) == H.HCCL_E_PTR
    assert L.HcclSend(BUF_A, 4, FP32, 1, comms[0], None) == H.HCCL_E_PTR
    assert L.HcclSend(BUF_A, 4, 200, 1, comms[0], STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclSend(BUF_A, 4, FP32, 7, comms[0], STREAM) == H.HCCL_E_PARA                  # no such rank
    assert L.HcclRecv(None, 4, FP32, 1, comms[0], STREAM) == H.HCCL_E_PTR
    assert L.HcclBatchSendRecv(None, 1, comms[0], STREAM) == H.HCCL_E_PTR
    # a send waits for its receive; a receive that disagrees on the count is refused
    err = ctypes.c_int32(-1)
    assert L.HcclGetCommAsyncError(comms[0], ctypes.byref(err)) == 0 and err.value == H.HCCL_SUCCESS
    assert L.HcclSend(BUF_A, 4, FP32, 1, comms[0], STREAM) == H.HCCL_SUCCESS
    assert L.HcclRecv(BUF_B, 8, FP32, 0, comms[1], STREAM) == H.HCCL_E_PARA
    # the send returned success before its receive turned up: the sender learns of the failure here
    assert L.HcclGetCommAsyncError(comms[0], ctypes.byref(err)) == 0 and err.value == H.HCCL_E_PARA


def test_rooted_entry_checks(comms):
    c = comms[0]
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    assert L.HcclBroadcast(None, 0, FP32, 0, None, None) == H.HCCL_SUCCESS                  # count 0 first
    assert L.HcclBroadcast(BUF_A, 4, FP32, 0, None, STREAM) == H.HCCL_E_PTR
    assert L.HcclBroadcast(None, 4, FP32, 0, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclBroadcast(BUF_A, 4, FP32, 0, c, None) == H.HCCL_E_PTR
    assert L.HcclBroadcast(BUF_A, 4, FP32, 4, c, STREAM) == H.HCCL_E_PARA                    # root out of range
    assert L.HcclReduce(None, None, 0, FP32, SUM, 0, None, None) == H.HCCL_SUCCESS
    assert L.HcclReduce(BUF_A, None, 4, FP32, SUM, 0, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclReduce(BUF_A, BUF_B, 4, FP32, 8, 0, c, STREAM) == H.HCCL_E_NOT_SUPPORT
    assert L.HcclReduce(BUF_A, BUF_B, 4, FP32, SUM, 9, c, STREAM) == H.HCCL_E_PARA
    assert L.HcclScatter(None, BUF_B, 0, FP32, 0, c, STREAM) == H.HCCL_SUCCESS
    assert L.HcclScatter(None, None, 4, FP32, 0, c, STREAM) == H.HCCL_E_PTR
    assert L.HcclScatter(None, BUF_B, 4, FP32, 0, c, STREAM) == H.HCCL_E_PTR                 # rank 0 is the root: needs sendBuf
    assert L.HcclScatter(None, BUF_B, 4, FP32, 1, c, STREAM) == H.HCCL_SUCCESS               # not the root: joins
    assert L.HcclScatter(BUF_A, BUF_B, 4, FP32, 2, comms[1], STREAM) == H.HCCL_E_PARA        # ranks disagree on the root


def test_no_gpu_means_loud_failure(comms):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    FP32, SUM = H.HCCL_DATA_TYPE_FP32, H.HCCL_REDUCE_SUM
    codes = [L.HcclAllReduce(BUF_A, BUF_B, 8, FP32, SUM, c, STREAM) for c in comms]
    assert codes[:3] == [0, 0, 0] and codes[3] == H.HCCL_E_RUNTIME          # the issuing rank reports it
    err = ctypes.c_int32(0)
    assert L.HcclGetCommAsyncError(comms[0], ctypes.byref(err)) == 0 and err.value == H.HCCL_E_RUNTIME


def test_root_info_init_and_comm_config():
    assert L.HcclGetRootInfo(None) == H.HCCL_E_PTR
    comms = H.comm_init_root_info(3)
    n, r = ctypes.c_uint32(), ctypes.c_uint32()
    for i, c in enumerate(comms):
        assert L.HcclGetRankSize(c, ctypes.byref(n)) == 0 and n.value == 3
        assert L.HcclGetRankId(c, ctypes.byref(r)) == 0 and r.value == i
    H.comm_destroy(comms)
    # argument rules (op_base.cc:1055-1110): rank within range, one handle per rank, same size on every rank
    info = ctypes.create_string_buffer(4108)
    assert L.HcclGetRootInfo(info) == 0
    c = ctypes.c_void_p()
    assert L.HcclCommInitRootInfo(0, info, 0, ctypes.byref(c)) == H.HCCL_E_PARA
    assert L.HcclCommInitRootInfo(2, info, 2, ctypes.byref(c)) == H.HCCL_E_PARA
    assert L.HcclCommInitRootInfo(2, None, 0, ctypes.byref(c)) == H.HCCL_E_PTR
    assert L.HcclCommInitRootInfo(2, info, 0, None) == H.HCCL_E_PTR
    assert L.HcclCommInitRootInfo(2, info, 0, ctypes.byref(c)) == 0
    d = ctypes.c_void_p()
    assert L.HcclCommInitRootInfo(2, info, 0, ctypes.byref(d)) == H.HCCL_E_PARA       # rank 0 exists
    assert L.HcclCommInitRootInfo(3, info, 1, ctypes.byref(d)) == H.HCCL_E_PARA       # other group size
    assert L.HcclCommInitRootInfo(2, ctypes.create_string_buffer(4108), 1, ctypes.byref(d)) == H.HCCL_E_PARA   # foreign token
    assert L.HcclCommDestroy(c) == 0
    # configuration rules (comm_config.cc:29-178)
    cfg = H.comm_config_init()
    cfg.hcclBufferSize = 16
    cfg.hcclDeterministic = 1
    cfg.hcclCommName = b"tensor_parallel_0"
    comms = H.comm_init_root_info(2, cfg)
    name = ctypes.create_string_buffer(128)
    assert L.HcclGetCommName(comms[0], name) == 0 and name.value == b"tensor_parallel_0"
    H.comm_destroy(comms)
    for field, value in (("hcclBufferSize", 0), ("hcclDeterministic", 2)):
        bad = H.comm_config_init()
        setattr(bad, field, value)
        info = ctypes.create_string_buffer(4108)
        assert L.HcclGetRootInfo(info) == 0
        assert L.HcclCommInitRootInfoConfig(2, info, 0, ctypes.byref(bad), ctypes.byref(c)) == H.HCCL_E_PARA
    raw = H.HcclCommConfig()                                                          # never initialised: no magic word
    assert L.HcclCommInitRootInfoConfig(2, info, 0, ctypes.byref(raw), ctypes.byref(c)) == H.HCCL_E_PARA
    assert L.HcclCommInitRootInfoConfig(2, info, 0, None, ctypes.byref(c)) == H.HCCL_E_PTR


def test_sub_communicator(comms):
    subs = H.create_sub_comm(comms, [1, 3], 7)
    n, r = ctypes.c_uint32(), ctypes.c_uint32()
    for pos, sc in enumerate(subs):
        assert L.HcclGetRankSize(sc, ctypes.byref(n)) == 0 and n.value == 2
        assert L.HcclGetRankId(sc, ctypes.byref(r)) == 0 and r.value == pos
    H.comm_destroy(subs)
    cfg = H.comm_config_init()
    out = ctypes.c_void_p()
    parent = ctypes.c_void_p(comms[0].value)
    ids = (ctypes.c_uint32 * 2)(1, 3)
    # a rank outside the sub-communicator passes no list and the invalid id: nothing happens
    assert L.HcclCreateSubCommConfig(ctypes.byref(parent), 0, None, 0xFFFFFFFF, 0, ctypes.byref(cfg), ctypes.byref(out)) == 0
    assert out.value is None
    assert L.HcclCreateSubCommConfig(ctypes.byref(parent), 2, None, 5, 0, ctypes.byref(cfg), ctypes.byref(out)) == H.HCCL_E_PARA
    assert L.HcclCreateSubCommConfig(ctypes.byref(parent), 2, ids, 5, 2, ctypes.byref(cfg), ctypes.byref(out)) == H.HCCL_E_PARA
    assert L.HcclCreateSubCommConfig(ctypes.byref(parent), 2, ids, 5, 0, ctypes.byref(cfg), ctypes.byref(out)) == H.HCCL_E_PARA  # rank 0 is not rankIds[0]
    assert L.HcclCreateSubCommConfig(ctypes.byref(parent), 2, ids, 5, 0, ctypes.byref(cfg), None) == H.HCCL_E_PTR


def test_caller_compiles_against_the_reference_header_and_links(tmp_path):
    """A program written against the reference's own inc/hccl/hccl.h (only acl/acl.h comes from this
    repository) must compile and link against libhccl.so: same names, same argument lists."""
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("hccl_build", os.path.join(root, "cann-hccl_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    own = build.build_abi_caller(force=True, out=str(tmp_path / "caller_own"))
    assert os.path.exists(own)
    ref_inc = "/root/reference/inc"
    if not os.path.isdir(ref_inc):
        pytest.skip("reference tree not present on this machine")
    theirs = build.build_abi_caller(include_dirs=[ref_inc], out=str(tmp_path / "caller_ref"))
    assert os.path.exists(theirs)


def test_table_arena_keeps_blocks_of_collectives_recorded_into_a_callers_graph(tmp_path):
    """The bookkeeping behind the lifetime rule for captured collectives, on the host: a pinned block's chunk
    survives Reset() untouched, unpinned chunks are reused or freed, nothing leaks (tests/c_abi/arena_check.cc
    against cann-hccl_amd/csrc/arena.h with malloc / free as the allocator)."""
    import os
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "arena_check")
    subprocess.run([cxx, "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(root, "cann-hccl_amd", "csrc"),
                    os.path.join(root, "tests", "c_abi", "arena_check.cc"), "-o", exe], check=True)
    out = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "OK", out.stdout


def test_plans_derived_from_a_template_of_another_count_are_the_planners_own(tmp_path):
    """A caller whose sizes change from call to call gets its plans by scaling an earlier plan of the same request
    whenever the schedule scales (counts that cut into whole slices).  tests/c_abi/plan_template_check.cc holds every
    derived plan against the plan made from scratch (27 schedules x 2 element sizes x in place or not x 10 x 10
    counts), on the host, against the planner's sources (cann-hccl_amd/csrc/plan*.cc) alone.  The same program holds the plans of the
    variable-count reduce-scatter that are derived from the plan over blocks of 16, 32, 64 ... elements against the
    planner's own (ring, uncut mesh, halving-doubling; 2 to 32 ranks; tables of equal, tiny, mixed and large blocks),
    and checks that the piece-cut mesh, tables with gaps or empty blocks and in-place calls get no such template."""
    import os
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "plan_template_check")
    subprocess.run([cxx, "-O2", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(root, "cann-hccl_amd", "csrc"),
                    "-I", os.path.join(root, "include"), os.path.join(root, "tests", "c_abi", "plan_template_check.cc"),
                    *_planner_sources(root), "-o", exe], check=True)
    out = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    assert out.returncode == 0 and out.stdout.startswith("OK"), out.stdout
    derived = int(out.stdout.split()[3])
    assert derived > 1000, out.stdout
    tables = int(out.stdout.split("templates,")[1].split()[0])
    assert tables > 300, out.stdout


def _planner_sources(root):
    return [os.path.join(root, "cann-hccl_amd", "csrc", f)
            for f in ("plan.cc", "plan_schedules.cc", "plan_lower.cc", "plan_fuse.cc", "plan_template.cc")]


def test_seeded_walk_over_requests_and_counts_derives_only_the_planners_own_plans(tmp_path):
    """tests/c_abi/plan_template_walk.cc: random requests (collective, schedule, 2 .. 33 ranks, rank groups, rings inside a
    group, ranks with a network port, ranks in place, element size, CCL buffer size) and for each a sequence of counts --
    whole slices, ragged, tiny, several chunks -- or of block tables, with up to four templates kept per request as the
    library keeps them: 20 000 derived plans per run, each compared with the plan made from scratch; tables with gaps or
    empty blocks must not be derived.  HCCL_AMD_TEST_SEED_SHIFT moves the walk to other cases."""
    import os
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "plan_template_walk")
    subprocess.run([cxx, "-O2", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(root, "cann-hccl_amd", "csrc"),
                    "-I", os.path.join(root, "include"), os.path.join(root, "tests", "c_abi", "plan_template_walk.cc"),
                    *_planner_sources(root), "-o", exe], check=True)
    out = subprocess.run([exe, "20000"], stdout=subprocess.PIPE, text=True, timeout=300)
    print(out.stdout)
    assert out.returncode == 0 and out.stdout.startswith("OK"), out.stdout
    words = out.stdout.replace("(", " ").split()
    assert int(words[1]) >= 20000, out.stdout
    assert int(words[3]) > 1000 and int(words[8]) > 100, out.stdout          # ragged counts, block templates


def _rank_table(path, servers, per_server, **edits):
    import json
    table = {"server_count": str(servers), "status": "completed", "version": "1.0", "server_list": []}
    for s in range(servers):
        devices = [{"device_id": str(d), "device_ip": "192.168.%d.%d" % (s, d), "rank_id": str(s * per_server + d)}
                   for d in range(per_server)]
        table["server_list"].append({"server_id": "10.0.0.%d" % (s + 1), "device": devices})
    table.update(edits)
    with open(path, "w") as f:
        json.dump(table, f, indent=1)
    return str(path).encode()


def test_comm_from_rank_table(tmp_path):
    # HcclCommInitClusterInfo: the rank table's ranks form one group; its servers become the rank groups
    path = _rank_table(tmp_path / "ranktable.json", 2, 4)
    comms = []
    for r in range(8):
        c = ctypes.c_void_p()
        assert L.HcclCommInitClusterInfo(path, r, ctypes.byref(c)) == H.HCCL_SUCCESS
        comms.append(c)
    n, rank = ctypes.c_uint32(0), ctypes.c_uint32(99)
    assert L.HcclGetRankSize(comms[5], ctypes.byref(n)) == 0 and n.value == 8
    assert L.HcclGetRankId(comms[5], ctypes.byref(rank)) == 0 and rank.value == 5
    extra = ctypes.c_void_p()
    assert L.HcclCommInitClusterInfo(path, 8, ctypes.byref(extra)) == H.HCCL_E_PARA        # not in the table
    H.comm_destroy(comms)
    # with a configuration
    cfg = H.comm_config_init()
    cfg.hcclBufferSize = 64
    comms = []
    for r in range(8):
        c = ctypes.c_void_p()
        assert L.HcclCommInitClusterInfoConfig(path, r, ctypes.byref(cfg), ctypes.byref(c)) == H.HCCL_SUCCESS
        comms.append(c)
    H.comm_destroy(comms)
    # refusals
    c = ctypes.c_void_p()
    assert L.HcclCommInitClusterInfo(None, 0, ctypes.byref(c)) == H.HCCL_E_PTR
    assert L.HcclCommInitClusterInfo(path, 0, None) == H.HCCL_E_PTR
    assert L.HcclCommInitClusterInfo(str(tmp_path / "missing.json").encode(), 0, ctypes.byref(c)) == H.HCCL_E_PARA
    bad = tmp_path / "bad.json"
    bad.write_text("{ not json")
    assert L.HcclCommInitClusterInfo(str(bad).encode(), 0, ctypes.byref(c)) == H.HCCL_E_PARA
    wrong_count = _rank_table(tmp_path / "count.json", 2, 4, server_count="3")
    assert L.HcclCommInitClusterInfo(wrong_count, 0, ctypes.byref(c)) == H.HCCL_E_PARA
    empty = _rank_table(tmp_path / "empty.json", 2, 4, server_list=[], server_count="0")
    assert L.HcclCommInitClusterInfo(empty, 0, ctypes.byref(c)) == H.HCCL_E_PARA
    import json
    uneven = json.loads(open(tmp_path / "ranktable.json").read())
    uneven["server_list"][1]["device"].pop()
    (tmp_path / "uneven.json").write_text(json.dumps(uneven))
    assert L.HcclCommInitClusterInfo(str(tmp_path / "uneven.json").encode(), 0, ctypes.byref(c)) == H.HCCL_E_NOT_SUPPORT
    twice = json.loads(open(tmp_path / "ranktable.json").read())
    twice["server_list"][1]["device"][0]["rank_id"] = "0"
    (tmp_path / "twice.json").write_text(json.dumps(twice))
    assert L.HcclCommInitClusterInfo(str(tmp_path / "twice.json").encode(), 0, ctypes.byref(c)) == H.HCCL_E_PARA
