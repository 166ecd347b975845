"""Seeded random walk over the planner's parameter space on the CPU: collective, schedule, rank count, size,
buffer size, alignment, which ranks run in place, rank groups.  Integer sums, so the expected result needs no
schedule: it is the plain numpy sum / concatenation / copy.  Both forms of every plan are interpreted."""
import os

import numpy as np
import pytest

import plan_interp
from closed_forms import INT32, SUM
from hccl_loader import load

# other random cases without touching the file: HCCL_AMD_TEST_SEED_SHIFT=1000 python -m pytest ...
SEED_SHIFT = int(os.environ.get("HCCL_AMD_TEST_SEED_SHIFT", "0"))
H = load()
RING, MESH, RHD, MESH_ATOMIC = 0, 1, 2, 4


def _case(rng):
    coll = int(rng.choice([H.COLL_ALLREDUCE, H.COLL_REDUCESCATTER, H.COLL_ALLGATHER, H.COLL_BROADCAST, H.COLL_REDUCE]))
    p = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 24]))
    n = int(rng.choice([1, 2, 31, 32, 33, 255, 1000, 2049, int(rng.integers(1, 3000))]))
    align = int(rng.choice([128, 128, 4, 64, 512]))
    ccl = int(rng.choice([200 << 20, 200 << 20, 4 * p * align, 4096, 4 * int(rng.integers(p, 40 * p))]))
    algo = int(rng.choice([RING, MESH, RHD, MESH_ATOMIC]))
    servers, rings = 1, 0
    if coll in (H.COLL_ALLREDUCE, H.COLL_REDUCESCATTER, H.COLL_REDUCE, H.COLL_ALLGATHER) and rng.random() < 0.4:
        servers = int(rng.choice([s for s in range(1, p + 1) if p % s == 0]))
        algo = int(rng.choice([RING, RHD]))
        if coll in (H.COLL_ALLREDUCE, H.COLL_REDUCESCATTER, H.COLL_ALLGATHER) and rng.random() < 0.4 and (coll == H.COLL_ALLREDUCE or servers > 1):
            rings = 4 if p // servers == 8 and rng.random() < 0.6 else 1
    mask = 0
    if coll == H.COLL_ALLREDUCE and rng.random() < 0.5:
        mask = int(rng.integers(0, 1 << p))
    return coll, p, n, align, ccl, algo, servers, rings, mask, int(rng.integers(0, p))


@pytest.mark.parametrize("seed", range(8))
def test_random_plans_compute_the_plain_result(seed):
    rng = np.random.default_rng(7000 + SEED_SHIFT + seed)
    done = 0
    while done < 40:
        coll, p, n, align, ccl, algo, servers, rings, mask, root = _case(rng)
        if coll in (H.COLL_ALLGATHER, H.COLL_BROADCAST) and algo == MESH_ATOMIC:
            algo = MESH
        if coll == H.COLL_ALLREDUCE:
            word = algo | (servers << 8) | (rings << 17) if (servers > 1 or rings) else algo
        elif coll == H.COLL_REDUCESCATTER:
            word = algo | (servers << 8) | (rings << 17) if servers > 1 else algo
        elif coll == H.COLL_ALLGATHER:
            word = algo | (servers << 8) | (rings << 17) if servers > 1 else algo
        elif coll == H.COLL_REDUCE and servers > 1:
            word = root | (algo << 16) | (servers << 20)
        else:
            word = root | (algo << 16)
        in_n = n * p if coll == H.COLL_REDUCESCATTER else n
        out_n = n * p if coll == H.COLL_ALLGATHER else n
        ins = [rng.integers(-1000, 1000, in_n).astype(np.int32) for _ in range(p)]
        label = (seed, done, coll, p, n, align, ccl, algo, servers, rings, mask, root)
        try:
            plan = H.describe_plan(coll, word, p, n, INT32, ccl_bytes=ccl, align=align,
                                   in_place_mask=(1 << p) - 1 if coll == H.COLL_BROADCAST else mask)
        except Exception as e:   # noqa: BLE001
            # the only request the planner may turn down here: a buffer that holds no element per rank
            # under the executor's chunk rule (rounded down to the alignment, except in the two-level reduce-scatter)
            if (coll == H.COLL_REDUCESCATTER and servers > 1) or (coll == H.COLL_ALLGATHER and servers > 1 and rings):
                per = ccl // (p * 4)
            elif coll in (H.COLL_REDUCESCATTER, H.COLL_ALLGATHER):
                per = ccl // p // align * align // 4
            else:
                per = ccl // 4
            assert per == 0, (label, repr(e))
            continue
        total = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)
        if coll == H.COLL_ALLREDUCE:
            want = [total] * p
        elif coll == H.COLL_REDUCESCATTER:
            want = [total[r * n:(r + 1) * n] for r in range(p)]
        elif coll == H.COLL_ALLGATHER:
            want = [np.concatenate(ins)] * p
        elif coll == H.COLL_BROADCAST:
            want = [ins[root]] * p
        else:
            want = [total if r == root else None for r in range(p)]
        for fused in (False, True):
            if fused and not plan["fusedOk"]:
                continue
            sends = [x.view(np.uint8).copy() for x in ins]
            if coll == H.COLL_BROADCAST:
                recvs = [x.view(np.uint8).copy() if r == root else np.full(out_n * 4, 0x5A, np.uint8) for r, x in enumerate(ins)]
                place = True
            else:
                recvs = [sends[r].copy() if (mask >> r) & 1 else np.full(out_n * 4, 0x5A, np.uint8) for r in range(p)]
                place = mask
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, sends, recvs, INT32, SUM, in_place=place)
            for r in range(p):
                if want[r] is not None:
                    assert np.array_equal(recvs[r].view(np.int32), want[r]), (label, fused, r)
            for r in range(p):
                if coll != H.COLL_BROADCAST and not (mask >> r) & 1:
                    assert np.array_equal(sends[r], ins[r].view(np.uint8)), (label, fused, r, "send buffer changed")
        done += 1


@pytest.mark.parametrize("seed", range(4))
def test_random_alltoallv_plans_deliver_every_block(seed):
    """All-to-all-v with random counts (many of them zero), displacements in shuffled order with gaps, element
    sizes 1 to 8, flat and staged over every server count that divides the ranks: each block arrives where the
    receiver's table says, nothing else in the receive buffers changes, the send buffers stay as they were."""
    rng = np.random.default_rng(9100 + SEED_SHIFT + seed)
    from closed_forms import INT8, INT16, INT64
    unit_of = {INT8: 1, INT16: 2, INT32: 4, INT64: 8}
    for case in range(25):
        p = int(rng.choice([1, 2, 3, 4, 6, 8, 9, 12, 16]))
        servers = int(rng.choice([s for s in range(1, p + 1) if p % s == 0]))
        dt = int(rng.choice(list(unit_of)))
        u = unit_of[dt]
        cnt = rng.integers(0, int(rng.choice([3, 40, 700])), (p, p)).astype(np.uint64)
        cnt[rng.random((p, p)) < rng.choice([0.0, 0.2, 0.7])] = 0
        sdis, rdis = np.zeros((p, p), np.uint64), np.zeros((p, p), np.uint64)
        sl, rl = [], []
        for r in range(p):
            pos = 0
            for j in rng.permutation(p):
                pos += int(rng.integers(0, 9))
                sdis[r, j] = pos
                pos += int(cnt[r, j])
            sl.append(pos + 3)
            pos = 0
            for i in rng.permutation(p):
                pos += int(rng.integers(0, 9))
                rdis[r, i] = pos
                pos += int(cnt[i, r])
            rl.append(pos + 3)
        sends = [rng.integers(0, 256, n * u).astype(np.uint8) for n in sl]
        want = [np.full(n * u, 0x5A, np.uint8) for n in rl]
        for i in range(p):
            for j in range(p):
                c = int(cnt[i, j]) * u
                want[j][int(rdis[j, i]) * u:int(rdis[j, i]) * u + c] = sends[i][int(sdis[i, j]) * u:int(sdis[i, j]) * u + c]
        label = (seed, case, p, servers, dt)
        plan = H.describe_plan(H.COLL_ALLTOALLV, H.ALGO_PAIRWISE | (servers << 8), p, 0, dt, tables=(cnt, sdis, cnt.T.copy(), rdis))
        assert plan["fusedOk"], label
        for fused in (False, True):
            src = [x.copy() for x in sends]
            recvs = [np.full(n * u, 0x5A, np.uint8) for n in rl]
            (plan_interp.run_fused if fused else plan_interp.run_steps)(plan, src, recvs, dt, SUM)
            for r in range(p):
                assert np.array_equal(recvs[r], want[r]), (label, fused, r)
                assert np.array_equal(src[r], sends[r]), (label, fused, r, "send buffer changed")
