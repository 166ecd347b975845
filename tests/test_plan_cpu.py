"""Product planner and fuser on the CPU: the plan the library would execute (HcclAmdDescribePlan)
is interpreted with numpy and compared with the checker, step-by-step form and fused form."""
import numpy as np
import pytest

import closed_forms as cf
import plan_interp
from closed_forms import BF16, FP16, FP32, INT8, INT32, INT64, MAX, MIN, PROD, SUM
from hccl_loader import load
from test_oracle_schedules import _a2av_case

H = load()
RING, MESH, RHD, MESH_ATOMIC = 0, 1, 2, 4


def _bytes(arrs):
    return [a.view(np.uint8).copy() for a in arrs]


def _ins(dt, p, n, seed):
    rng = np.random.default_rng(seed)
    return [cf.random_input(dt, n, rng) for _ in range(p)]


def _same(dt, got_bytes, want):
    got = got_bytes.view(cf.CARRIER[dt])
    if dt in (FP16, BF16, FP32):
        nn = np.isnan(cf.widen(dt, got).astype(np.float64)) & np.isnan(cf.widen(dt, want).astype(np.float64))
        return np.array_equal(got[~nn], want[~nn])
    return np.array_equal(got, want)


@pytest.mark.parametrize("algo", [RING, MESH, RHD, MESH_ATOMIC])
@pytest.mark.parametrize("p", [1, 2, 3, 4, 5, 6, 8, 12, 16, 24])
def test_allreduce_plan_matches_checker(orc, algo, p):
    for dt, op, n, ccl in ((FP32, SUM, 1000, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, PROD, 777, 200 << 20),
                           (INT8, MAX, 333, 200 << 20), (FP16, SUM, 2049, 2048)):
        unit = H.DTYPE_SIZE[dt]
        ins = _ins(dt, p, n, p * 7 + op)
        want = orc.allreduce(ins, dt, op, algo=algo, ccl_bytes=ccl)
        for mask in (0, (1 << p) - 1):
            plan = H.describe_plan(H.COLL_ALLREDUCE, algo, p, n, dt, ccl_bytes=ccl, in_place_mask=mask)
            assert plan["scratchBytes"] == 0
            for fused in (False, True):
                if fused and not plan["fusedOk"]:
                    continue
                sends = _bytes(ins)
                recvs = _bytes(ins) if mask else [np.full(n * unit, 0xA5, np.uint8) for _ in range(p)]
                runner = plan_interp.run_fused if fused else plan_interp.run_steps
                runner(plan, sends, recvs, dt, op, in_place=bool(mask))
                for r in range(p):
                    assert _same(dt, recvs[r], want[r]), (algo, p, dt, op, ccl, mask, fused, r)
                if not mask:
                    assert all(np.array_equal(s, i.view(np.uint8)) for s, i in zip(sends, ins))   # send buffers untouched
            if p <= 32:
                assert plan["fusedOk"], (algo, p)


def test_allreduce_ring_byte_counts():
    p, n = 8, 1 << 20
    S = n * 4
    plan = H.describe_plan(H.COLL_ALLREDUCE, RING, p, n, FP32)
    assert plan["stepRead"] + plan["stepWritten"] == 5 * (p - 1) * S     # partials live in the receive buffer
    assert plan["fusedRead"] == p * S and plan["fusedWritten"] == p * S
    assert len(plan["phases"]) == 2 * (p - 1)
    plan = H.describe_plan(H.COLL_ALLREDUCE, RHD, 32, n, FP32)
    assert plan["fusedRead"] == 32 * S and plan["fusedWritten"] == 32 * S
    plan = H.describe_plan(H.COLL_ALLREDUCE, RHD, 24, n, FP32)
    assert plan["fusedOk"] and plan["fused"][0]["kind"] == 2 and plan["fused"][0]["nleaf"] == 16


@pytest.mark.parametrize("algo", [RING, MESH, RHD, MESH_ATOMIC])
@pytest.mark.parametrize("p", [1, 2, 3, 6, 8, 12])
def test_reducescatter_plan_matches_checker(orc, algo, p):
    for dt, op, n, ccl in ((FP32, SUM, 500, 200 << 20), (BF16, SUM, 301, 128 * p * 2), (INT64, MIN, 100, 200 << 20)):
        unit = H.DTYPE_SIZE[dt]
        ins = _ins(dt, p, n * p, p + op)
        want = orc.reducescatter(ins, dt, op, algo=algo, ccl_bytes=ccl)
        plan = H.describe_plan(H.COLL_REDUCESCATTER, algo, p, n, dt, ccl_bytes=ccl)
        for fused in (False, True):
            sends = _bytes(ins)
            recvs = [np.full(n * unit, 0x5A, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
            for r in range(p):
                assert _same(dt, recvs[r], want[r]), (algo, p, dt, fused, r)
            assert all(np.array_equal(s, i.view(np.uint8)) for s, i in zip(sends, ins))


@pytest.mark.parametrize("algo", [RING, MESH, RHD])
@pytest.mark.parametrize("p", [1, 2, 5, 6, 8, 12])
def test_allgather_plan_matches_checker(orc, algo, p):
    for dt, n, ccl in ((INT8, 301, 200 << 20), (INT32, 100, 128 * p * 2)):
        unit = H.DTYPE_SIZE[dt]
        ins = _ins(dt, p, n, p)
        want = orc.allgather(ins, dt, algo=algo, ccl_bytes=ccl)
        plan = H.describe_plan(H.COLL_ALLGATHER, algo, p, n, dt, ccl_bytes=ccl)
        for fused in (False, True):
            sends = _bytes(ins)
            recvs = [np.full(n * unit * p, 0x5A, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(cf.CARRIER[dt]), want[r]), (algo, p, dt, fused, r)


@pytest.mark.parametrize("p", [1, 2, 3, 8, 16])
def test_alltoallv_plan_matches_checker(orc, p):
    cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 10 + p)
    sends = [(np.arange(n, dtype=np.int32) + (r << 20)) for r, n in enumerate(sl)]
    want = [np.full(n, -1, np.int32) for n in rl]
    assert orc.alltoallv(sends, cnt, sdis, want, rcnt, rdis, INT32) == 0
    plan = H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE, p, 0, INT32, tables=(cnt, sdis, rcnt, rdis))
    assert len(plan["phases"]) <= p
    for fused in (False, True):
        recvs = [np.full(n, -1, np.int32).view(np.uint8).copy() for n in rl]
        (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, _bytes(sends), recvs, INT32, 0)
        for r in range(p):
            assert np.array_equal(recvs[r].view(np.int32), want[r]), (p, fused, r)


@pytest.mark.parametrize("p", [2, 3, 8])
def test_alltoallv_plan_moves_big_blocks_in_pieces_of_the_buffer(orc, p):
    # a block larger than the CCL buffer goes in pieces, one phase each: as many phases per step as the checker's
    # restatement of the reference's transfer loop makes calls, no piece larger than the buffer
    cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 70 + p, max_count=3000)
    cnt[cnt == 0] = 1                       # every step moves something (an empty step has no phase to count)
    sdis = np.concatenate([np.zeros((p, 1), np.uint64), np.cumsum(cnt, axis=1)[:, :-1]], axis=1).astype(np.uint64)
    rcnt = cnt.T.copy()
    rdis = np.concatenate([np.zeros((p, 1), np.uint64), np.cumsum(rcnt, axis=1)[:, :-1]], axis=1).astype(np.uint64)
    sl, rl = [int(x) for x in cnt.sum(axis=1)], [int(x) for x in rcnt.sum(axis=1)]
    sends = [(np.arange(n, dtype=np.int32) + (r << 20)) for r, n in enumerate(sl)]
    for ccl in (512, 4096, 1 << 20):
        want = [np.full(n, -1, np.int32) for n in rl]
        assert orc.alltoallv(sends, cnt, sdis, want, rcnt, rdis, INT32, scratch_bytes=ccl) == 0
        rounds, biggest, total = orc.alltoallv_rounds(cnt, rcnt, INT32, ccl)
        plan = H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE, p, 0, INT32, ccl_bytes=ccl, tables=(cnt, sdis, rcnt, rdis))
        assert len(plan["phases"]) == sum(rounds), (p, ccl, rounds)
        assert max(st["n"] for ph in plan["phases"] for st in ph) == max(biggest, 4 * int(np.diag(cnt).max()))
        assert sum(st["n"] for ph in plan["phases"][1:] for st in ph) == total
        at = 1
        for i in range(1, p):                                        # step i: ranks r -> r + i, piece t in phase t of the step
            for t in range(rounds[i]):
                for st in plan["phases"][at + t]:
                    assert st["dst"][0] == (st["a"][0] + i) % p and st["n"] <= ccl
            at += rounds[i]
        for fused in (False, True):
            recvs = [np.full(n, -1, np.int32).view(np.uint8).copy() for n in rl]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, _bytes(sends), recvs, INT32, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.int32), want[r]), (p, ccl, fused, r)


@pytest.mark.parametrize("p,servers", [(4, 2), (8, 2), (8, 4), (6, 3), (16, 4), (12, 12), (9, 3)])
def test_staged_alltoallv_plan_matches_checker(orc, p, servers):
    cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 40 + p + servers)
    sends = [(np.arange(n, dtype=np.int32) + (r << 20)) for r, n in enumerate(sl)]
    want = [np.full(n, -1, np.int32) for n in rl]
    assert orc.alltoallv_staged(sends, cnt, sdis, want, rcnt, rdis, INT32, servers) == 0
    plan = H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE | (servers << 8), p, 0, INT32, tables=(cnt, sdis, rcnt, rdis))
    flat = H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE, p, 0, INT32, tables=(cnt, sdis, rcnt, rdis))
    m = p // servers
    # stage one: own blocks, then the neighbours' (none when a server holds one rank); stage two: one phase per server
    assert len(plan["phases"]) <= 2 + servers
    # the workspace holds, per rank, what its server addresses to the ranks with its local index
    work = max(sum(int(cnt[r // m * m + k, j]) for j in range(r % m, p, m) for k in range(m)) for r in range(p)) * 4
    assert work <= plan["scratchBytes"] <= work + max(sl) * 4 + 256
    moved = 4 * int(cnt.sum())
    assert sum(s["n"] for ph in plan["phases"] for s in ph) == 2 * moved      # every block moves twice step by step ...
    assert sum(it["n"] for it in plan["fused"]) == moved                      # ... and once when fused
    assert sum(it["n"] for it in flat["fused"]) == moved
    for fused in (False, True):
        recvs = [np.full(n, -1, np.int32).view(np.uint8).copy() for n in rl]
        (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, _bytes(sends), recvs, INT32, 0)
        for r in range(p):
            assert np.array_equal(recvs[r].view(np.int32), want[r]), (p, servers, fused, r)
    uneven = next(s for s in range(2, p + 2) if p % s)         # a server count that does not divide the ranks
    with pytest.raises(H.HcclError):
        H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE | (uneven << 8), p, 0, INT32, tables=(cnt, sdis, rcnt, rdis))


@pytest.mark.parametrize("p,servers", [(8, 2), (12, 3), (8, 4)])
def test_staged_alltoallv_plan_batches_runs_larger_than_the_buffer(orc, p, servers):
    # between the servers a run larger than the CCL buffer goes in batches, one phase each, a block cut where a batch
    # is full: as many phases and as many transfers as the checker's restatement of the reference's packing counts
    m = p // servers
    cnt = _a2av_case(p, 75 + p + servers, max_count=900)[0]
    cnt[cnt == 0] = 3
    rcnt = cnt.T.copy()
    sdis = np.concatenate([np.zeros((p, 1), np.uint64), np.cumsum(cnt, axis=1)[:, :-1]], axis=1).astype(np.uint64)
    rdis = np.concatenate([np.zeros((p, 1), np.uint64), np.cumsum(rcnt, axis=1)[:, :-1]], axis=1).astype(np.uint64)
    sl, rl = [int(x) for x in cnt.sum(axis=1)], [int(x) for x in rcnt.sum(axis=1)]
    sends = [(np.arange(n, dtype=np.int32) + (r << 20)) for r, n in enumerate(sl)]
    want = [np.full(n, -1, np.int32) for n in rl]
    assert orc.alltoallv_staged(sends, cnt, sdis, want, rcnt, rdis, INT32, servers) == 0
    for ccl in (1024, 4096, 1 << 20):
        rounds, entries, biggest = orc.alltoallv_staged_rounds(cnt, servers, INT32, ccl)
        plan = H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE | (servers << 8), p, 0, INT32, ccl_bytes=ccl,
                               tables=(cnt, sdis, rcnt, rdis))
        assert len(plan["phases"]) == 2 + sum(rounds), (p, servers, ccl, rounds)
        between = [st for ph in plan["phases"][3:] for st in ph]              # after stage one and the local runs
        assert len(between) == entries, (p, servers, ccl)
        at = 3
        for i in range(1, servers):
            for t in range(rounds[i]):
                per_pair = {}
                for st in plan["phases"][at + t]:
                    a, d = st["a"][0], st["dst"][0]
                    assert d % m == a % m and d // m == (a // m + i) % servers
                    per_pair[(a, d)] = per_pair.get((a, d), 0) + st["n"]
                assert max(per_pair.values()) <= ccl                         # a batch fits the buffer
            at += rounds[i]
        for fused in (False, True):
            recvs = [np.full(n, -1, np.int32).view(np.uint8).copy() for n in rl]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, _bytes(sends), recvs, INT32, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.int32), want[r]), (p, servers, ccl, fused, r)


def _copy_items(plan):
    """The fused copy items of a plan as (destination rank, offset, source rank, offset, bytes), neighbours joined."""
    rows = sorted((d[0], d[2], it["src"][0][0], it["src"][0][2], it["n"]) for it in plan["fused"] for d in it["dst"])
    out = []
    for row in rows:
        if out and out[-1][0] == row[0] and out[-1][2] == row[2] and out[-1][1] + out[-1][4] == row[1] and \
                out[-1][3] + out[-1][4] == row[3]:
            out[-1] = out[-1][:4] + (out[-1][4] + row[4],)
        else:
            out.append(row)
    return out


def test_block_moving_plans_take_the_short_cut_and_agree_with_the_general_path(orc):
    # all-to-all-v, scatter and send / receive are planned by a direct pass over their blocks; with
    # HCCL_AMD_PLAN_VERIFY=1 (read once per process, hence the child process) every request goes through the general
    # planner with its symbolic verification: same phases, same bytes, the same blocks in the fused form
    import json
    import os
    import subprocess
    import sys
    p = 6
    cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 77, max_count=2000)
    requests = [
        dict(coll=H.COLL_ALLTOALLV, algo=H.ALGO_PAIRWISE, p=p, count=0, ccl_bytes=200 << 20, tables=True),
        dict(coll=H.COLL_ALLTOALLV, algo=H.ALGO_PAIRWISE, p=p, count=0, ccl_bytes=1024, tables=True),
        dict(coll=H.COLL_ALLTOALLV, algo=H.ALGO_PAIRWISE | (2 << 8), p=p, count=0, ccl_bytes=200 << 20, tables=True),   # staged, 2 x 3
        dict(coll=H.COLL_ALLTOALLV, algo=H.ALGO_PAIRWISE | (3 << 8), p=p, count=0, ccl_bytes=2048, tables=True),       # staged in batches
        dict(coll=H.COLL_SCATTER, algo=2, p=p, count=1003, ccl_bytes=200 << 20, tables=False),
        dict(coll=H.COLL_SCATTER, algo=2 | (3 << 21), p=p, count=1003, ccl_bytes=200 << 20, tables=False),
    ]

    vcounts = [5, 0, 301, 77, 1024, 3]
    vdispls = [400, 0, 0, 2000, 410, 395]                      # not in rank order, with gaps
    for algo in (RING, MESH, RHD):
        requests.append(dict(coll=H.COLL_ALLGATHER, algo=algo, p=p, count=0, ccl_bytes=200 << 20, tables="v"))

    def plans():
        out = []
        for rq in requests:
            tables = (vcounts, vdispls) if rq["tables"] == "v" else ((cnt, sdis, rcnt, rdis) if rq["tables"] else None)
            plan = H.describe_plan(rq["coll"], rq["algo"], rq["p"], rq["count"], INT32, ccl_bytes=rq["ccl_bytes"], tables=tables)
            steps = [sorted((st["dst"][0], st["dst"][2], st["a"][0], st["a"][2], st["n"]) for st in ph) for ph in plan["phases"]]
            out.append(dict(steps=steps, items=_copy_items(plan), bytes=[plan[k] for k in ("stepRead", "stepWritten", "fusedRead",
                                                                                         "fusedWritten", "scratchBytes")],
                            fusedOk=plan["fusedOk"]))
        return out

    if os.environ.get("HCCL_AMD_PLAN_CHILD") == "1":
        return plans()
    here = plans()
    code = ("import json, sys; sys.path.insert(0, %r); import test_plan_cpu as t; from oracle import oracle; "
            "print('PLANS' + json.dumps(t.test_block_moving_plans_take_the_short_cut_and_agree_with_the_general_path(oracle)))"
            % os.path.dirname(__file__))
    env = dict(os.environ, HCCL_AMD_PLAN_VERIFY="1", HCCL_AMD_PLAN_CHILD="1")
    env["PYTHONPATH"] = os.pathsep.join([os.path.dirname(os.path.dirname(__file__)), env.get("PYTHONPATH", "")])
    res = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert res.returncode == 0, res.stderr[-2000:]
    there = json.loads(res.stdout[res.stdout.index("PLANS") + 5:])
    for i, (a, b) in enumerate(zip(here, there)):
        assert a["fusedOk"] and b["fusedOk"]
        assert a["bytes"] == b["bytes"], (i, a["bytes"], b["bytes"])
        assert [[list(x) for x in ph] for ph in a["steps"]] == b["steps"], i
        assert [list(x) for x in a["items"]] == b["items"], i


def test_plan_rejects_bad_requests():
    with pytest.raises(H.HcclError):
        H.describe_plan(H.COLL_ALLREDUCE, RING, 0, 10, FP32)
    with pytest.raises(H.HcclError):
        H.describe_plan(H.COLL_REDUCESCATTER, H.ALGO_PAIRWISE, 4, 10, FP32)   # pairwise is an all-to-all schedule
    with pytest.raises(H.HcclError):
        H.describe_plan(H.COLL_ALLGATHER, RING, 8, 10, FP32, ccl_bytes=64)   # buffer below one aligned slice per rank
    # a slice alignment that the element size does not divide would cut slices inside elements
    for dt, align in ((FP32, 1), (FP32, 2), (FP32, 6), (H.HCCL_DATA_TYPE_FP64, 4), (H.HCCL_DATA_TYPE_FP64, 12)):
        for coll in (H.COLL_ALLREDUCE, H.COLL_REDUCESCATTER, H.COLL_ALLGATHER):
            with pytest.raises(H.HcclError) as e:
                H.describe_plan(coll, RING, 3, 1000, dt, align=align)
            assert e.value.code == H.HCCL_E_PARA
    H.describe_plan(H.COLL_ALLREDUCE, RING, 3, 1000, FP32, align=4)
    H.describe_plan(H.COLL_ALLREDUCE, RING, 3, 1000, H.HCCL_DATA_TYPE_INT8, align=1)


def _v_case(p, seed):
    rng = np.random.default_rng(seed)
    counts = rng.integers(0, 400, p)
    counts[rng.random(p) < 0.2] = 0
    displs, pos = np.zeros(p, np.int64), 0
    for i in rng.permutation(p):                 # blocks in shuffled order with gaps
        pos += int(rng.integers(0, 9))
        displs[i] = pos
        pos += int(counts[i])
    return counts, displs, pos + 3


@pytest.mark.parametrize("algo", [RING, MESH, RHD])
@pytest.mark.parametrize("p", [1, 2, 3, 6, 8])
def test_reducescatter_v_plan_matches_checker(orc, algo, p):
    for dt, op in ((FP32, SUM), (INT32, MAX)):
        unit = H.DTYPE_SIZE[dt]
        counts, displs, extent = _v_case(p, 5 * p + op)
        ins = _ins(dt, p, extent, p)
        plan = H.describe_plan(H.COLL_REDUCESCATTER, algo, p, 0, dt, tables=(counts, displs))
        want = orc.reducescatter_v(ins, counts, displs, dt, op, algo=algo)
        if algo == RHD:
            # halving-doubling over a table of blocks is this library's own (the reference has the mesh only): the tree
            # closed form pins planner and checker alike
            block, part1 = cf.rhd_params(p)
            for r in range(p):
                xs = [x[displs[r]:displs[r] + counts[r]] for x in ins]
                q = r // 2 if r < part1 else r - part1 // 2
                assert _same(dt, _bytes([want[r]])[0], xs[0] if p == 1 else cf.rhd_tree(dt, op, xs, q, block, part1)), (p, dt, r)
        for fused in (False, True):
            sends = _bytes(ins)
            recvs = [np.full(int(counts[r]) * unit, 0x5A, np.uint8) for r in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
            for r in range(p):
                assert _same(dt, recvs[r], want[r]), (algo, p, dt, fused, r)


@pytest.mark.parametrize("algo", [RING, MESH, RHD])
@pytest.mark.parametrize("p", [1, 2, 5, 6, 8])
def test_allgather_v_plan_matches_checker(orc, algo, p):
    counts, displs, extent = _v_case(p, 9 * p)
    ins = [np.arange(int(counts[r]), dtype=np.int32) + (r << 16) for r in range(p)]
    want = np.full(extent, 0x5A5A5A5A, np.int32)
    for r in range(p):
        want[displs[r]:displs[r] + counts[r]] = ins[r]
    if algo != RHD:
        got = orc.allgather_v(ins, counts, displs, extent, INT32, algo=algo, fill=0x5A5A5A5A)
        assert all(np.array_equal(g, want) for g in got)
    plan = H.describe_plan(H.COLL_ALLGATHER, algo, p, 0, INT32, tables=(counts, displs))
    for fused in (False, True):
        recvs = [np.full(extent * 4, 0x5A, np.uint8) for _ in range(p)]
        (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, _bytes(ins), recvs, INT32, 0)
        for r in range(p):
            assert np.array_equal(recvs[r].view(np.int32), want), (algo, p, fused, r)


@pytest.mark.parametrize("p", [1, 2, 3, 5, 8])
def test_rooted_plans_match_checker(orc, p):
    rng = np.random.default_rng(p)
    for root in sorted({0, p - 1, p // 2}):
        # broadcast (in place on every rank), two chunk settings
        n = 1003
        for ccl in (200 << 20, 1024):
            bufs = _ins(INT32, p, n, 50 + p)
            want = orc.broadcast([b.copy() for b in bufs], INT32, root, ccl_bytes=ccl)
            plan = H.describe_plan(H.COLL_BROADCAST, root, p, n, INT32, ccl_bytes=ccl, in_place_mask=(1 << p) - 1)
            for fused in (False, True):
                mem = _bytes(bufs)
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, mem, mem, INT32, 0, in_place=True)
                for r in range(p):
                    assert np.array_equal(mem[r].view(np.int32), want[r]), ("bcast", p, root, ccl, fused, r)
        # reduce to the root: ring chain x_root (+) (x_{root-1} (+) ( ... (x_{root+2} (+) x_{root+1})))
        for dt, op in ((FP32, SUM), (BF16, PROD), (INT8, MIN)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 60 + p + dt)
            want = orc.reduce_to_root(ins, dt, op, root, ccl_bytes=2048)
            chain = cf.ring_chain(dt, op, ins, root) if p > 1 else ins[0]
            assert _same(dt, want.view(np.uint8), chain)
            plan = H.describe_plan(H.COLL_REDUCE, root, p, n, dt, ccl_bytes=2048)
            for fused in (False, True):
                sends = _bytes(ins)
                recvs = [np.full(n * unit, 0x77, np.uint8) for _ in range(p)]
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                assert _same(dt, recvs[root], want), ("reduce", p, root, dt, fused)
                for r in range(p):
                    assert np.array_equal(sends[r], ins[r].view(np.uint8))
                    if r != root:
                        assert np.all(recvs[r] == 0x77)              # only the root's output is written
        # scatter
        src = rng.integers(0, 1 << 30, n * p).astype(np.int32)
        want = orc.scatter(src, p, INT32, root)
        plan = H.describe_plan(H.COLL_SCATTER, root, p, n, INT32)
        for fused in (False, True):
            sends = [src.view(np.uint8).copy() if r == root else np.zeros(0, np.uint8) for r in range(p)]
            recvs = [np.zeros(n * 4, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, INT32, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.int32), want[r]) and np.array_equal(want[r], src[r * n:(r + 1) * n])


@pytest.mark.parametrize("p", [1, 2, 3, 5, 8])
def test_rooted_mesh_plans_match_checker(orc, p):
    # mesh broadcast (scatter + all-gather) and mesh reduce (mesh reduce-scatter + gather to the root)
    n = 1003
    for root in sorted({0, p - 1, p // 2}):
        for ccl, align in ((200 << 20, 128), (1024, 128), (200 << 20, 4)):
            bufs = _ins(INT32, p, n, 150 + p)
            want = orc.broadcast([b.copy() for b in bufs], INT32, root, ccl_bytes=ccl, align=align, algo=MESH)
            assert all(np.array_equal(w, bufs[root]) for w in want)
            plan = H.describe_plan(H.COLL_BROADCAST, root | (MESH << 16), p, n, INT32, ccl_bytes=ccl, align=align,
                                   in_place_mask=(1 << p) - 1)
            if p > 1:
                assert len(plan["phases"]) == 2
            for fused in (False, True):
                mem = _bytes(bufs)
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, mem, mem, INT32, 0, in_place=True)
                for r in range(p):
                    assert np.array_equal(mem[r].view(np.int32), want[r]), ("bcast mesh", p, root, ccl, fused, r)
        for algo in (MESH, MESH_ATOMIC):
            for dt, op in ((FP32, SUM), (BF16, SUM), (INT8, MIN)):
                unit = H.DTYPE_SIZE[dt]
                ins = _ins(dt, p, n, 160 + p + dt)
                want = orc.reduce_to_root(ins, dt, op, root, ccl_bytes=2048, algo=algo)
                closed = (cf.mesh_allreduce if algo == MESH else cf.mesh_atomic_allreduce)(dt, op, ins, unit, 2048, 128)[0]
                assert _same(dt, want.view(np.uint8), closed), ("reduce mesh closed form", p, root, algo, dt)
                plan = H.describe_plan(H.COLL_REDUCE, root | (algo << 16), p, n, dt, ccl_bytes=2048)
                for fused in (False, True):
                    if fused and not plan["fusedOk"]:
                        continue
                    sends = _bytes(ins)
                    recvs = [np.full(n * unit, 0x77, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                    assert _same(dt, recvs[root], want), ("reduce mesh", p, root, algo, dt, fused)
                    for r in range(p):
                        assert np.array_equal(sends[r], ins[r].view(np.uint8))
                        if r != root:
                            assert np.all(recvs[r] == 0x77)
                assert plan["fusedOk"]


def test_order_sensitive_known_answers_through_the_planner():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_fp32.json")) as f:
        kat = json.load(f)
    xs = [np.array(v, np.float32) for v in kat["inputs"]]
    p = kat["ranks"]
    for name, algo in (("ring", RING), ("mesh", MESH), ("mesh_uncut", MESH_ATOMIC), ("rhd", RHD)):
        plan = H.describe_plan(H.COLL_ALLREDUCE, algo, p, 4, FP32, align=kat["align"])
        for fused in (False, True):
            sends = _bytes(xs)
            recvs = [np.full(16, 0xA5, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, FP32, SUM)
            for r in range(p):
                assert float(recvs[r].view(np.float32)[0]) == kat["expected_element0"][name], (name, fused, r)


def test_four_ring_known_answers_through_the_planner():
    # hand-derived sums of tests/golden/order_sensitive_four_rings_fp32.json: each of the first four elements takes
    # its own ring of the 8-device topology, and a single ring gives different bits
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_four_rings_fp32.json")) as f:
        kat = json.load(f)
    p, n = kat["ranks"], kat["elements"]
    xs = []
    for row in kat["inputs_first4"]:
        x = np.zeros(n, np.float32)
        x[:4] = row
        xs.append(x)
    for name, rings in (("ring4", 4), ("ring", 1)):
        want = np.zeros(n, np.float32)
        want[:4] = kat["expected_first4"][name]
        for level1 in (RING, RHD):
            plan = H.describe_plan(H.COLL_ALLREDUCE, level1 | (1 << 8) | (rings << 17), p, n, FP32, align=kat["align"])
            for fused in (False, True):
                sends = _bytes(xs)
                recvs = [np.full(n * 4, 0xA5, np.uint8) for _ in range(p)]
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, FP32, SUM)
                for r in range(p):
                    assert np.array_equal(recvs[r].view(np.float32), want), (name, level1, fused, r)


@pytest.mark.parametrize("p", [2, 3, 4, 5, 6, 7, 8, 12, 13, 24])
def test_reduce_rhd_plan_matches_checker_and_tree(orc, p):
    n = 1003
    for root in sorted({0, 1, p - 1, p // 2}):
        for dt, op, ccl in ((FP32, SUM, 200 << 20), (FP32, SUM, 2048), (BF16, SUM, 200 << 20), (INT8, MIN, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 260 + p + dt)
            want = orc.reduce_to_root(ins, dt, op, root, ccl_bytes=ccl, algo=RHD)
            closed = cf.rhd_reduce_to_root(dt, op, ins, unit, ccl, 128, root)
            assert _same(dt, want.view(np.uint8), closed), ("reduce rhd closed form", p, root, dt, ccl)
            plan = H.describe_plan(H.COLL_REDUCE, root | (RHD << 16), p, n, dt, ccl_bytes=ccl)
            for fused in (False, True):
                if fused and not plan["fusedOk"]:
                    continue
                sends = _bytes(ins)
                recvs = [np.full(n * unit, 0x77, np.uint8) for _ in range(p)]
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                assert _same(dt, recvs[root], want), ("reduce rhd", p, root, dt, ccl, fused)
                for r in range(p):
                    assert np.array_equal(sends[r], ins[r].view(np.uint8))
                    if r != root:
                        assert np.all(recvs[r] == 0x77)
            assert plan["fusedOk"], (p, root)


@pytest.mark.parametrize("p", [2, 3, 4, 5, 6, 7, 8, 12, 13, 24])
def test_broadcast_rhd_plan_matches_checker(orc, p):
    n = 1003
    for root in sorted({0, 1, p - 1, p // 2}):
        for ccl in (200 << 20, 1024):
            bufs = _ins(INT32, p, n, 350 + p)
            want = orc.broadcast([b.copy() for b in bufs], INT32, root, ccl_bytes=ccl, algo=RHD)
            assert all(np.array_equal(w, bufs[root]) for w in want), (p, root)
            plan = H.describe_plan(H.COLL_BROADCAST, root | (RHD << 16), p, n, INT32, ccl_bytes=ccl, in_place_mask=(1 << p) - 1)
            block = 1 << (p.bit_length() - 1)
            assert len(plan["phases"]) == (block.bit_length() - 1) + (1 if p > block else 0)   # tree depth, plus the pair hand-over
            for fused in (False, True):
                mem = _bytes(bufs)
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, mem, mem, INT32, 0, in_place=True)
                for r in range(p):
                    assert np.array_equal(mem[r].view(np.int32), want[r]), ("bcast rhd", p, root, ccl, fused, r)


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("shape", [(2, 4), (4, 2), (3, 4), (2, 8), (8, 1), (5, 3)])
def test_two_level_allreduce_plan_matches_checker(orc, level1, shape):
    servers, D = shape
    p = servers * D
    for atomic in (False, True):
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, PROD, 777, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 400 + p + n)
            want = orc.allreduce_two_level(ins, dt, op, servers, level1=level1, atomic=atomic, ccl_bytes=ccl)
            for mask in (0, (1 << p) - 1):
                plan = H.describe_plan(H.COLL_ALLREDUCE, level1 | (servers << 8) | (int(atomic) << 16), p, n, dt, ccl_bytes=ccl,
                                       in_place_mask=mask)
                assert plan["scratchBytes"] == 0
                for fused in (False, True):
                    if fused and not plan["fusedOk"]:
                        continue
                    sends = _bytes(ins)
                    recvs = _bytes(ins) if mask else [np.full(n * unit, 0xA5, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op, in_place=bool(mask))
                    for r in range(p):
                        assert _same(dt, recvs[r], want[r]), (shape, level1, atomic, dt, ccl, mask, fused, r)


@pytest.mark.parametrize("level1", [RING, RHD])
def test_two_level_fused_stack_form_keeps_operand_order(orc, level1):
    # every two-level expression has a fused form (a stack program); NaN payloads and signed zeros under
    # max / min show which operand stood left in each of its combines
    pool = np.concatenate([np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0], np.float32),
                           np.array([0x7fc00001, 0xffc00002, 0x7fa00003], np.uint32).view(np.float32)])
    for servers, D in ((2, 4), (3, 4), (4, 4), (8, 2), (5, 3)):
        p = servers * D
        rng = np.random.default_rng(31 * p + level1)
        ins = [rng.choice(pool, 1501).astype(np.float32) for _ in range(p)]
        for op in (H.HCCL_REDUCE_MAX, H.HCCL_REDUCE_MIN):
            want = orc.allreduce_two_level(ins, FP32, op, servers, level1=level1, atomic=False, align=4)
            plan = H.describe_plan(H.COLL_ALLREDUCE, level1 | (servers << 8), p, 1501, FP32, align=4)
            assert plan["fusedOk"]
            kinds = {it["kind"] for it in plan["fused"]}
            assert kinds <= {2, 3} and (3 in kinds or (level1 == RHD and D == 2))
            for it in plan["fused"]:
                if it["kind"] == 3:
                    assert len(it["src"]) == p and sum(o & 7 for o in it["ops"]) == p - 1
            sends = _bytes(ins)
            recvs = [np.full(1501 * 4, 0xA5, np.uint8) for _ in range(p)]
            plan_interp.run_fused(plan, sends, recvs, FP32, op)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.uint32), want[r].view(np.uint32)), (servers, D, level1, op, r)


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["ring", "ring4"])
def test_two_level_allreduce_with_rings_inside_a_group_matches_checker(orc, level1, level0):
    rings = 4 if level0 == "ring4" else 1
    shapes = ((1, 8), (2, 8), (3, 8)) if rings == 4 else ((2, 4), (4, 2), (3, 4), (5, 3))
    for servers, D in shapes:
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, PROD, 777, 200 << 20), (FP32, SUM, 60, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 500 + p + n)
            want = orc.allreduce_two_level(ins, dt, op, servers, level1=level1, level0=level0, ccl_bytes=ccl)
            for mask in (0, (1 << p) - 1):
                plan = H.describe_plan(H.COLL_ALLREDUCE, level1 | (servers << 8) | (rings << 17), p, n, dt, ccl_bytes=ccl,
                                       in_place_mask=mask)
                assert plan["scratchBytes"] == 0 and plan["fusedOk"]
                for fused in (False, True):
                    sends = _bytes(ins)
                    recvs = _bytes(ins) if mask else [np.full(n * unit, 0xA5, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op, in_place=bool(mask))
                    for r in range(p):
                        assert _same(dt, recvs[r], want[r]), (servers, D, level1, level0, dt, ccl, mask, fused, r)
    # groups of another size have no four-ring form
    with pytest.raises(Exception):
        H.describe_plan(H.COLL_ALLREDUCE, level1 | (2 << 8) | (4 << 17), 8, 1000, FP32)


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("shape", [(2, 4), (4, 2), (3, 4), (2, 8), (8, 1), (5, 3)])
def test_two_level_reducescatter_plan_matches_checker(orc, level1, shape):
    servers, D = shape
    p = servers * D
    for atomic in (False, True):
        for dt, op, n, ccl in ((FP32, SUM, 211, 200 << 20), (FP32, SUM, 500, 4 * p * 128), (BF16, PROD, 77, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n * p, 600 + p + n)
            want = orc.reducescatter_two_level(ins, dt, op, servers, level1=level1, atomic=atomic, ccl_bytes=ccl)
            plan = H.describe_plan(H.COLL_REDUCESCATTER, level1 | (servers << 8) | (int(atomic) << 16), p, n, dt, ccl_bytes=ccl)
            assert plan["fusedOk"]
            for fused in (False, True):
                sends = _bytes(ins)
                recvs = [np.full(n * unit, 0x5A, np.uint8) for _ in range(p)]
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                for r in range(p):
                    assert _same(dt, recvs[r], want[r]), (shape, level1, atomic, dt, ccl, fused, r)
                assert all(np.array_equal(s_, i.view(np.uint8)) for s_, i in zip(sends, ins))   # inputs stay as they were


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("shape", [(2, 4), (4, 2), (3, 4), (2, 8), (8, 1), (5, 3)])
def test_two_level_reduce_plan_matches_checker(orc, level1, shape):
    servers, D = shape
    p = servers * D
    for atomic in (False, True):
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, PROD, 777, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 700 + p + n)
            for root in sorted({0, p - 1, (D + 1) % p}):
                want = orc.reduce_to_root_two_level(ins, dt, op, root, servers, level1=level1, atomic=atomic, ccl_bytes=ccl)
                plan = H.describe_plan(H.COLL_REDUCE, root | (level1 << 16) | (servers << 20) | (int(atomic) << 28), p, n, dt,
                                       ccl_bytes=ccl)
                assert plan["fusedOk"]
                for fused in (False, True):
                    sends = _bytes(ins)
                    recvs = [np.full(n * unit, 0x77, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                    assert _same(dt, recvs[root], want), (shape, level1, atomic, dt, ccl, root, fused)
                    for r in range(p):
                        assert np.array_equal(sends[r], ins[r].view(np.uint8))
                        if r != root:
                            assert np.all(recvs[r] == 0x77)              # only the root's output is written


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["ring", "ring4"])
def test_two_level_reducescatter_with_rings_inside_a_group_matches_checker(orc, level1, level0):
    rings = 4 if level0 == "ring4" else 1
    shapes = ((2, 8), (3, 8)) if rings == 4 else ((2, 4), (4, 2), (3, 4), (5, 3))
    for servers, D in shapes:
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 211, 200 << 20), (FP32, SUM, 500, 4 * p * 128), (BF16, PROD, 77, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n * p, 800 + p + n)
            want = orc.reducescatter_two_level(ins, dt, op, servers, level1=level1, level0=level0, ccl_bytes=ccl)
            plan = H.describe_plan(H.COLL_REDUCESCATTER, level1 | (servers << 8) | (rings << 17), p, n, dt, ccl_bytes=ccl)
            assert plan["fusedOk"]
            for fused in (False, True):
                sends = _bytes(ins)
                recvs = [np.full(n * unit, 0x5A, np.uint8) for _ in range(p)]
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                for r in range(p):
                    assert _same(dt, recvs[r], want[r]), (servers, D, level1, level0, dt, ccl, fused, r)


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["ring", "ring4"])
def test_two_level_reduce_with_rings_inside_a_group_matches_checker(orc, level1, level0):
    rings = 4 if level0 == "ring4" else 1
    shapes = ((2, 8), (3, 8)) if rings == 4 else ((2, 4), (4, 2), (3, 4), (5, 3))
    for servers, D in shapes:
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, PROD, 777, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 900 + p + n)
            for root in sorted({0, p - 1, (D + 1) % p}):
                want = orc.reduce_to_root_two_level(ins, dt, op, root, servers, level1=level1, level0=level0, ccl_bytes=ccl)
                word = root | (level1 << 16) | (servers << 20) | ((1 << 29) if rings == 1 else (1 << 30))
                plan = H.describe_plan(H.COLL_REDUCE, word, p, n, dt, ccl_bytes=ccl)
                assert plan["fusedOk"]
                for fused in (False, True):
                    sends = _bytes(ins)
                    recvs = [np.full(n * unit, 0x77, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                    assert _same(dt, recvs[root], want), (servers, D, level1, level0, dt, ccl, root, fused)
                    for r in range(p):
                        if r != root:
                            assert np.all(recvs[r] == 0x77)


def _gold():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "slice_plans.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _gold()["ring"])
def test_planner_ring_slices_match_the_hand_derived_vectors(case):
    # the product's own slice plan, read off its ring all-reduce: the all-gather's first phase copies each rank's
    # reduced slice to its neighbour, so its steps name every non-empty slice once, by offset and size
    total, p, align = case["total"], case["p"], case["align"]
    if p == 1:
        return
    plan = H.describe_plan(H.COLL_ALLREDUCE, RING, p, total, H.HCCL_DATA_TYPE_INT8, align=align)
    want = sorted((o, s) for o, s in zip(case["off"], case["size"]) if s)
    seen = set()
    for ph in plan["phases"]:
        for s in ph:
            seen.add((s["dst"][2], s["n"]))
    assert set(want) <= seen, (want, sorted(seen))
    # every step is one slice, whole: nothing in the plan cuts a slice differently
    assert all(x in set(want) for x in seen), (want, sorted(seen))


@pytest.mark.parametrize("case", [c for c in _gold()["chunks"] if c["kind"] == 0])
def test_planner_chunk_plan_matches_the_hand_derived_vectors(case):
    # all-reduce chunk loop: a chunk's steps stay inside [chunk start, chunk end) of the buffers, and the chunk
    # boundaries are the hand-derived ones
    p, unit = case["p"], case["unit"]
    dt = {4: FP32, 8: INT64}[unit]
    if case["count"] > (1 << 22):
        return                                        # the big vector is covered by the checker's test; keep this one quick
    plan = H.describe_plan(H.COLL_ALLREDUCE, RING, p, case["count"], dt, ccl_bytes=case["ccl"], align=case["align"])
    bounds = [0]
    for c in case["counts"]:
        bounds.append(bounds[-1] + c * unit)
    for ph in plan["phases"]:
        for s in ph:
            lo, hi = s["dst"][2], s["dst"][2] + s["n"]
            assert any(b0 <= lo and hi <= b1 for b0, b1 in zip(bounds, bounds[1:])), (lo, hi, bounds)
    starts = {s["dst"][2] for ph in plan["phases"] for s in ph}
    assert set(bounds[:-1]) <= starts


@pytest.mark.parametrize("case", [c for c in _gold()["rhd_slices"] if c["total"] <= (1 << 22)])
def test_planner_halving_doubling_slices_match_the_hand_derived_vectors(case):
    # a halving-doubling all-reduce over a power-of-two block moves runs of 1, 2, 4, ... neighbouring slices:
    # every step of the product's plan must be such a run of the hand-derived slices, and every slice moves alone once
    block, total = case["block"], case["total"]
    plan = H.describe_plan(H.COLL_ALLREDUCE, RHD, block, total, H.HCCL_DATA_TYPE_INT8, align=case["align"])
    off, size = case["off"], case["size"]
    runs = set()
    w = 1
    while w <= block:
        for i in range(0, block, w):
            n = sum(size[i:i + w])
            if n:
                runs.add((off[i], n))
        w *= 2
    seen = {(s["dst"][2], s["n"]) for ph in plan["phases"] for s in ph}
    assert seen <= runs, (sorted(seen - runs), sorted(runs))
    assert {(o, s) for o, s in zip(off, size) if s} <= seen


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["mesh", "ring", "ring4"])
def test_two_level_allgather_plan_matches_checker(orc, level1, level0):
    rings = {"mesh": 0, "ring": 1, "ring4": 4}[level0]
    shapes = ((2, 8), (3, 8)) if rings == 4 else ((2, 4), (4, 2), (3, 4), (5, 3), (6, 1))
    for servers, D in shapes:
        p = servers * D
        for dt, n, ccl in ((INT32, 1003, 200 << 20), (INT32, 777, 4096), (BF16, 301, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, 410 + p + n)
            want = orc.allgather_two_level(ins, dt, servers, level1=level1, level0=level0, ccl_bytes=ccl)
            plan = H.describe_plan(H.COLL_ALLGATHER, level1 | (servers << 8) | (rings << 17), p, n, dt, ccl_bytes=ccl)
            if ccl >= n * unit * p:
                # one chunk: the own copy, the group's phase(s), then the schedule between the groups
                inside = 0 if D == 1 else (1 if rings == 0 else D - 1)
                between = servers - 1 if level1 == RING else len(H.describe_plan(H.COLL_ALLGATHER, RHD, servers, 8, dt)["phases"]) - 1
                # (an upper bound: the planner moves a step to the earliest phase its operands allow)
                assert len(plan["phases"]) <= 1 + inside + between, (servers, D, level1, level0, len(plan["phases"]))
            # the route, which the result cannot show: a block only moves inside a group or between two ranks
            # at the same position of their groups, and every rank takes (servers - 1) * D blocks from other groups
            crossing = [0] * p
            for ph in plan["phases"]:
                for st in ph:
                    a, d = st["a"][0], st["dst"][0]
                    assert a // D == d // D or a % D == d % D, (servers, D, level1, level0, a, d)
                    if a // D != d // D:
                        crossing[d] += st["n"]
            if level1 == RING or servers & (servers - 1) == 0:
                assert crossing == [(servers - 1) * D * n * unit] * p, (servers, D, level1, level0)
            else:
                # halving-doubling over a server count that is no power of two: the odd rank of a folded pair is
                # handed the whole result, its own group's blocks included (all_gather_recursive_hd.cc:215-236)
                assert all((servers - 1) * D * n * unit <= c <= p * n * unit for c in crossing), (servers, D, level0)
            for fused in (False, True):
                sends = _bytes(ins)
                recvs = [np.full(n * unit * p, 0x5A, np.uint8) for _ in range(p)]
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, 0)
                for r in range(p):
                    assert np.array_equal(recvs[r].view(cf.CARRIER[dt]), want[r]), (servers, D, level1, level0, dt, ccl, fused, r)
                    assert np.array_equal(sends[r], ins[r].view(np.uint8))
            # fused, every rank's output is written once and every input read p times or less
            assert sum(it["n"] * len(it["dst"]) for it in plan["fused"]) == p * p * n * unit


@pytest.mark.parametrize("p", [1, 2, 3, 5, 8, 13])
def test_ring_scatter_plan_matches_checker(orc, p):
    # the blocks travel round the ring, the farthest first; step by step they rest in the ranks' workspace on the way
    n = 257
    rng = np.random.default_rng(90 + p)
    for root in sorted({0, p - 1, p // 2}):
        src = rng.integers(0, 1 << 30, n * p).astype(np.int32)
        want = orc.scatter(src, p, INT32, root, algo=RING)
        for r in range(p):
            assert np.array_equal(want[r], src[r * n:(r + 1) * n]), (p, root, r)          # the definition
        plan = H.describe_plan(H.COLL_SCATTER, root | (1 << 20), p, n, INT32)
        if p > 1:
            assert len(plan["phases"]) == p - 1                                          # one block leaves the root per step
            hops = sum(1 for ph in plan["phases"] for s in ph) - 1                       # minus the root's own copy
            assert hops == p * (p - 1) // 2                                              # block of distance j takes j hops
            for ph in plan["phases"]:
                for s in ph:
                    a, d = s["a"][0], s["dst"][0]
                    assert d == a or d == (a + 1) % p, (p, root, a, d)                    # only to the right neighbour
        assert sum(it["n"] for it in plan["fused"]) == n * 4 * p                         # fused: every block moves once
        for fused in (False, True):
            sends = [src.view(np.uint8).copy() if r == root else np.zeros(0, np.uint8) for r in range(p)]
            recvs = [np.zeros(n * 4, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, INT32, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.int32), want[r]), (p, root, fused, r)


@pytest.mark.parametrize("p", [1, 2, 5, 8])
def test_star_broadcast_plan(orc, p):
    # one phase, every transfer from the root, the whole buffer each; same bytes as the checker's star
    n = 1003
    for root in sorted({0, p - 1, p // 2}):
        bufs = _ins(INT32, p, n, 170 + p)
        want, touched = orc.broadcast_star([b.copy() for b in bufs], INT32, root, return_touched=True)
        plan = H.describe_plan(H.COLL_BROADCAST, root | (5 << 16), p, n, INT32, ccl_bytes=1024, in_place_mask=(1 << p) - 1)
        if p > 1:
            assert len(plan["phases"]) == 1 and len(plan["phases"][0]) == p - 1
            assert all(st["a"][0] == root and st["n"] == n * 4 for st in plan["phases"][0])
        assert plan["stepWritten"] == touched // 2
        for fused in (False, True):
            mem = _bytes(bufs)
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, mem, mem, INT32, 0, in_place=True)
            for r in range(p):
                assert np.array_equal(mem[r].view(np.int32), want[r]), (p, root, fused, r)


def test_binary_block_broadcast_plan(orc):
    # the plan's transfers are the hand-derived routes, a rank's transfers in consecutive phases from the one after it
    # received; results and bytes as the checker's, step by step and fused, also under a chunk loop
    from test_oracle_schedules import HD_BLOCK_ROUTES
    n = 1003
    for (p, root), want in HD_BLOCK_ROUTES.items():
        plan = H.describe_plan(H.COLL_BROADCAST, root | (6 << 16), p, n, INT32, in_place_mask=(1 << p) - 1)
        got = sorted((st["a"][0], k, st["dst"][0]) for k, ph in enumerate(plan["phases"]) for st in ph)
        assert [(a, d) for a, _, d in got] == want, (p, root, got)
        got_at = {d: k for _, k, d in got}
        for a in range(p):
            mine = [k for s, k, _ in got if s == a]
            first = 0 if a == root else got_at[a] + 1
            assert mine == list(range(first, first + len(mine))), (p, root, a, mine)
        assert all(st["n"] == n * 4 for ph in plan["phases"] for st in ph)
    phases = {(7, 4): 4, (7, 6): 4, (6, 5): 3, (12, 3): 4, (8, 5): 3}      # the longest chain of each worked example
    for (p, root), k in phases.items():
        assert len(H.describe_plan(H.COLL_BROADCAST, root | (6 << 16), p, n, INT32)["phases"]) == k, (p, root)
    for p in (1, 2, 3, 5, 6, 7, 8, 11, 12, 13, 24, 33):
        for root in sorted({0, p - 1, p // 2}):
            for ccl in (200 << 20, 1024):
                bufs = _ins(INT32, p, n, 180 + p)
                want, touched = orc.broadcast_hd_blocks([b.copy() for b in bufs], INT32, root, ccl_bytes=ccl, return_touched=True)
                plan = H.describe_plan(H.COLL_BROADCAST, root | (6 << 16), p, n, INT32, ccl_bytes=ccl, in_place_mask=(1 << p) - 1)
                assert plan["stepWritten"] == touched // 2
                for fused in (False, True):
                    mem = _bytes(bufs)
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, mem, mem, INT32, 0, in_place=True)
                    for r in range(p):
                        assert np.array_equal(mem[r].view(np.int32), want[r]), (p, root, ccl, fused, r)


@pytest.mark.parametrize("servers,D,rings", [(2, 4, 1), (3, 3, 1), (4, 2, 1), (2, 8, 4), (1, 8, 4), (3, 8, 4)])
def test_two_level_ring_broadcast_plan(orc, servers, D, rings):
    # ring scatter in the root's group, halving-doubling between the groups, ring all-gather in every group: results and
    # bytes as the checker's (less what the all-gather would hand back to the root), and the route -- inside a group a
    # part only moves to the next device of its ring, between groups only between equal positions
    p = servers * D
    n = 1003
    rng = np.random.default_rng(650 + p)
    orders = [list(o) for o in cf.EIGHT_DEVICE_RINGS] if rings == 4 else [list(range(D))]
    nexts = {(o[i], o[(i + 1) % D]) for o in orders for i in range(D)}
    for root in sorted({0, p - 1, (D + 1) % p}):
        for ccl in (200 << 20, 1024):
            bufs = [rng.integers(0, 1 << 30, n).astype(np.int32) for _ in range(p)]
            want, touched = orc.broadcast_two_level_ring([b.copy() for b in bufs], INT32, root, servers, rings=rings, ccl_bytes=ccl,
                                                         return_touched=True)
            word = root | (RHD << 16) | (servers << 20) | ((1 << 29) if rings == 1 else (1 << 30))
            plan = H.describe_plan(H.COLL_BROADCAST, word, p, n, INT32, ccl_bytes=ccl, in_place_mask=(1 << p) - 1)
            assert plan["fusedOk"]
            back = 0
            for cur in ([n] if ccl >= n * 4 else [256] * (n // 256) + [n % 256]):
                back += cur * 4 - cf.slice_plan(cur * 4, D, 128)[root % D][1]
            assert plan["stepWritten"] == touched // 2 - back
            for ph in plan["phases"]:
                for st in ph:
                    a, d = st["a"][0], st["dst"][0]
                    assert d != root
                    if a // D == d // D:
                        assert (a % D, d % D) in nexts, (servers, D, rings, root, a, d)
                    else:
                        assert a % D == d % D, (servers, D, rings, root, a, d)
            for fused in (False, True):
                mem = _bytes(bufs)
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, mem, mem, INT32, 0, in_place=True)
                for r in range(p):
                    assert np.array_equal(mem[r].view(np.int32), want[r]), (servers, D, rings, root, ccl, fused, r)
    # four rings need groups of 8
    with pytest.raises(H.HcclError):
        H.describe_plan(H.COLL_BROADCAST, 0 | (RHD << 16) | (2 << 20) | (1 << 30), 8, n, INT32)


@pytest.mark.parametrize("servers,D", [(2, 4), (4, 2), (3, 4), (5, 3), (6, 1), (2, 8)])
def test_two_level_broadcast_plan(orc, servers, D):
    # scatter inside the root's group, halving-doubling between the groups, all-gather inside every group:
    # every rank ends with the root's data, and a block only moves inside a group or between equal positions
    p = servers * D
    n = 1003
    rng = np.random.default_rng(600 + p)
    for root in sorted({0, p - 1, (D + 1) % p}):
        for ccl in (200 << 20, 1024):
            bufs = [rng.integers(0, 1 << 30, n).astype(np.int32) for _ in range(p)]
            plan = H.describe_plan(H.COLL_BROADCAST, root | (MESH << 16) | (servers << 20), p, n, INT32, ccl_bytes=ccl,
                                   in_place_mask=(1 << p) - 1)
            for ph in plan["phases"]:
                for st in ph:
                    a, d = st["a"][0], st["dst"][0]
                    assert a // D == d // D or a % D == d % D, (servers, D, root, a, d)
                    assert d != root                                             # the root's data stays where it is
            if ccl >= n * 4 and D > 1 and servers > 1:
                flat = H.describe_plan(H.COLL_BROADCAST, root | (MESH << 16), p, n, INT32, in_place_mask=(1 << p) - 1)
                assert len(plan["phases"]) > len(flat["phases"])                 # two more stages than scatter + gather
            # The checker's executor for the same schedule receives the same bytes, plus the slices that the all-gather
            # of the root's group hands back to the root, which holds them already: the plan leaves the root alone.
            out, touched = orc.broadcast_two_level([b.copy() for b in bufs], INT32, root, servers, ccl_bytes=ccl,
                                                   return_touched=True)
            assert all(np.array_equal(b, bufs[root]) for b in out)
            back_to_root, left = 0, n
            while left > 0 and D > 1:
                cur = min(left, ccl // 4)
                back_to_root += cur * 4 - cf.broadcast_slices(cur, 4, D, 128)[root % D][1]
                left -= cur
            assert plan["stepWritten"] == touched // 2 - back_to_root, (servers, D, root, ccl)
            assert plan["stepRead"] == plan["stepWritten"]
            for fused in (False, True):
                sends = _bytes(bufs)
                recvs = [s for s in sends]                                       # one buffer per rank
                (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, INT32, 0, in_place=True)
                for r in range(p):
                    assert np.array_equal(recvs[r].view(np.int32), bufs[root]), (servers, D, root, ccl, fused, r)


@pytest.mark.parametrize("servers,D", [(2, 4), (4, 2), (3, 4), (5, 3), (6, 1), (2, 8), (1, 4)])
def test_two_level_scatter_plan(orc, servers, D):
    # a group's run of blocks travels round the ring of the ranks at the root's position, then every such rank hands
    # the ranks of its group their blocks
    p = servers * D
    n = 1003
    rng = np.random.default_rng(640 + p)
    for root in sorted({0, p - 1, (D + 1) % p}):
        src = rng.integers(0, 1 << 30, n * p).astype(np.int32)
        plan = H.describe_plan(H.COLL_SCATTER, root | (servers << 21), p, n, INT32)
        if servers > 1:
            assert len(plan["phases"]) == servers                        # servers - 1 ring steps, one hand-over
            for ph in plan["phases"][:-1]:
                for st in ph:
                    a, d = st["a"][0], st["dst"][0]
                    assert a % D == d % D == root % D and d // D == (a // D + 1) % servers, (servers, D, root, a, d)
                    assert st["n"] == n * 4 * D
            hops = sum(1 for ph in plan["phases"][:-1] for st in ph)
            assert hops == servers * (servers - 1) // 2                   # the run of the group j away makes j hops
        for st in plan["phases"][-1]:
            a, d = st["a"][0], st["dst"][0]
            assert a == d // D * D + root % D and st["n"] == n * 4, (servers, D, root, a, d)
        # The checker's executor for the same schedule moves the same bytes, plus what the reference's staging costs
        # and the plan leaves out: the root packing its p blocks, and the p - servers blocks that land in a
        # receiver's staging buffer before they are copied out (the plan's hand-over writes the receive buffer).
        for ccl in (200 << 20, 4096 * p):
            want, touched = orc.scatter_two_level(src, p, INT32, root, servers, ccl_bytes=ccl, return_touched=True)
            for r in range(p):
                assert np.array_equal(want[r], src[r * n:(r + 1) * n])
            assert plan["stepWritten"] == touched // 2 - (2 * p - servers) * n * 4, (servers, D, root, ccl)
        assert plan["stepRead"] == plan["stepWritten"]
        for fused in (False, True):
            sends = [src.view(np.uint8).copy() if r == root else np.zeros(0, np.uint8) for r in range(p)]
            recvs = [np.zeros(n * 4, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, INT32, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.int32), src[r * n:(r + 1) * n]), (servers, D, root, fused, r)
        assert sum(it["n"] for it in plan["fused"]) == n * 4 * p          # fused: every block moves once


@pytest.mark.parametrize("servers,D,level0", [(2, 4, "ring"), (3, 3, "ring"), (4, 2, "ring"), (2, 8, "ring4"), (3, 8, "ring4")])
def test_two_level_scatter_with_rings_inside_plan(orc, servers, D, level0):
    # level 1 as the mesh variant; inside a group a block only moves from a rank to the next one of the ring (rank order,
    # or ring 0 of the 8-device topology), starting at the rank at the root's position
    p = servers * D
    n = 1003
    rng = np.random.default_rng(660 + p)
    order = list(cf.EIGHT_DEVICE_RINGS[0]) if level0 == "ring4" else list(range(D))
    nexts = {(order[i], order[(i + 1) % D]) for i in range(D)}
    bit = (1 << 29) if level0 == "ring" else (1 << 30)
    for root in sorted({0, p - 1, (D + 1) % p}):
        src = rng.integers(0, 1 << 30, n * p).astype(np.int32)
        plan = H.describe_plan(H.COLL_SCATTER, root | (servers << 21) | bit, p, n, INT32)
        assert len(plan["phases"]) == (servers - 1) + (D - 1)
        inside = 0
        for k, ph in enumerate(plan["phases"]):
            for st in ph:
                a, d = st["a"][0], st["dst"][0]
                if k < servers - 1 and a // D != d // D:
                    assert a % D == d % D == root % D and d // D == (a // D + 1) % servers
                elif a != d:
                    assert a // D == d // D and (a % D, d % D) in nexts, (servers, D, level0, root, a, d)
                    inside += 1
        assert inside == servers * D * (D - 1) // 2
        want, touched = orc.scatter_two_level(src, p, INT32, root, servers, return_touched=True, level0=level0)
        assert plan["stepWritten"] == touched // 2 - (2 * p - servers) * n * 4, (servers, D, level0, root)
        for fused in (False, True):
            sends = [src.view(np.uint8).copy() if r == root else np.zeros(0, np.uint8) for r in range(p)]
            recvs = [np.zeros(n * 4, np.uint8) for _ in range(p)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, INT32, 0)
            for r in range(p):
                assert np.array_equal(recvs[r].view(np.int32), want[r]), (servers, D, level0, root, fused, r)
        assert sum(it["n"] for it in plan["fused"]) == n * 4 * p          # fused: every block moves once


PRUNED_PORTS = ([0], [5], [0, 4], [2, 3], [1, 6], [0, 2, 4, 6], [1, 2, 3, 7], [4, 5, 6, 7])


def _nic_bits(nic):
    return sum(1 << (20 + r) for r in nic)


def test_ring_pruned_allreduce_plan_matches_checker(orc):
    # 8-rank ring with fewer network ports than ranks (reduce_scatter_ring.cc:160-168, 299-477): the plan, step by
    # step and fused, against the checker's restatement of the template, out of place and in place
    p = 8
    for nic in PRUNED_PORTS:
        for dt, op, n, ccl in ((FP32, SUM, 1000, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, PROD, 777, 200 << 20), (INT8, MAX, 333, 200 << 20)):
            unit = H.DTYPE_SIZE[dt]
            ins = _ins(dt, p, n, len(nic) * 11 + op)
            want = orc.allreduce_ring_pruned([x.copy() for x in ins], dt, op, nic, ccl_bytes=ccl)
            for mask in (0, (1 << p) - 1):
                plan = H.describe_plan(H.COLL_ALLREDUCE, RING | _nic_bits(nic), p, n, dt, ccl_bytes=ccl, in_place_mask=mask)
                assert plan["scratchBytes"] == 0 and plan["fusedOk"]
                assert len(plan["phases"]) == 14 or ccl < n * unit           # 7 reduce hops, 7 copy hops, as the plain ring
                for fused in (False, True):
                    sends = _bytes(ins)
                    recvs = _bytes(ins) if mask else [np.full(n * unit, 0xA5, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op, in_place=bool(mask))
                    for r in range(p):
                        assert _same(dt, recvs[r], want[r]), (nic, dt, op, ccl, mask, fused, r)
    # all eight ports, or none named: the plain ring
    plain = H.describe_plan(H.COLL_ALLREDUCE, RING, p, 1000, FP32)
    assert H.describe_plan(H.COLL_ALLREDUCE, RING | _nic_bits(range(8)), p, 1000, FP32) == plain
    # 3 ports do not divide 8 slices; ports on a ring that is not 8 ranks make no sense
    for bad_p, nic in ((8, [0, 1, 2]), (8, [0, 1, 2, 3, 4]), (6, [0, 3]), (16, [0, 4])):
        with pytest.raises(H.HcclError):
            H.describe_plan(H.COLL_ALLREDUCE, RING | _nic_bits(nic), bad_p, 1000, FP32)


def test_two_level_reducescatter_with_fewer_ports_than_devices_plan(orc):
    # servers of 8 devices of which only some have a network port: the plan, step by step and fused if it fuses, against
    # the checker's restatement of the executor's branch and against the hand-derived answers
    from test_oracle_schedules import _two_level_pruned_kat
    for servers in (2, 3):
        p = 8 * servers
        for nic in ([0], [5], [0, 4], [2, 3], [1, 6], [0, 2, 4, 6], [1, 2, 3, 7]):
            for dt, op, n, ccl in ((FP32, SUM, 211, 200 << 20), (FP32, SUM, 500, 4 * p * 128), (BF16, PROD, 77, 200 << 20)):
                unit = H.DTYPE_SIZE[dt]
                ins = _ins(dt, p, n * p, 850 + p + n)
                want = orc.reducescatter_two_level_pruned(ins, dt, op, servers, nic, ccl_bytes=ccl)
                plan = H.describe_plan(H.COLL_REDUCESCATTER, RING | (servers << 8) | (4 << 17) | _nic_bits(nic), p, n, dt, ccl_bytes=ccl)
                for fused in ((False, True) if plan["fusedOk"] else (False,)):
                    sends = _bytes(ins)
                    recvs = [np.full(n * unit, 0x5A, np.uint8) for _ in range(p)]
                    (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, dt, op)
                    for r in range(p):
                        assert _same(dt, recvs[r], want[r]), (servers, nic, dt, ccl, fused, r)
                        assert np.array_equal(sends[r], ins[r].view(np.uint8))
    kat = _two_level_pruned_kat()
    n = kat["elements_per_block"]
    for case in kat["cases"]:
        xs = [np.full(16 * n, v, np.float32) for v in case["inputs_per_rank"]]
        plan = H.describe_plan(H.COLL_REDUCESCATTER, RING | (2 << 8) | (4 << 17) | _nic_bits(kat["nic_devices"]), 16, n, FP32)
        for fused in ((False, True) if plan["fusedOk"] else (False,)):
            sends = _bytes(xs)
            recvs = [np.full(n * 4, 0x5A, np.uint8) for _ in range(16)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, FP32, SUM)
            for b in range(16):
                want = (np.full(n, case["pruned_every_element"], np.float32) if "pruned_every_element" in case
                        else np.repeat(np.array(case["block_halves"][b], np.float32), n // 2))
                assert np.array_equal(recvs[b].view(np.float32), want), (case["name"], fused, b)
    # all ports: the ordinary branch; the halving-doubling schedule between the servers, one ring inside, or a variable-count
    # table do not go with a port list
    plain = H.describe_plan(H.COLL_REDUCESCATTER, RING | (2 << 8) | (4 << 17), 16, 100, FP32)
    assert H.describe_plan(H.COLL_REDUCESCATTER, RING | (2 << 8) | (4 << 17) | _nic_bits(range(8)), 16, 100, FP32) == plain
    for word in (RHD | (2 << 8) | (4 << 17), RING | (2 << 8) | (1 << 17), RING | (2 << 8)):
        with pytest.raises(H.HcclError):
            H.describe_plan(H.COLL_REDUCESCATTER, word | _nic_bits([0, 4]), 16, 100, FP32)


def test_ring_pruned_known_answers_through_the_planner():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_ring_pruned_fp32.json")) as f:
        kat = json.load(f)
    n = kat["elements"]
    xs = [np.full(n, v, np.float32) for v in kat["inputs_per_rank"]]
    per = n // 8
    for case in kat["cases"] + [dict(kat["plain_ring"], nic_ranks=[])]:
        want = np.repeat(np.array(case["slice_values"], np.float32), per)
        plan = H.describe_plan(H.COLL_ALLREDUCE, RING | _nic_bits(case["nic_ranks"]), 8, n, FP32)
        for fused in (False, True):
            sends = _bytes(xs)
            recvs = [np.full(n * 4, 0xA5, np.uint8) for _ in range(8)]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, FP32, SUM)
            for r in range(8):
                assert np.array_equal(recvs[r].view(np.float32), want), (case["nic_ranks"], fused, r)
