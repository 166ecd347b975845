"""Seeded random walk over the planner's parameter space on the CPU: collective, schedule, rank count, size,
buffer size, alignment, which ranks run in place, rank groups.  Integer sums, so the expected result needs no
schedule: it is the plain numpy sum / concatenation / copy.  Both forms of every plan are interpreted."""
import numpy as np
import pytest

import plan_interp
from closed_forms import INT32, SUM
from hccl_loader import load

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
    if coll in (H.COLL_ALLREDUCE, H.COLL_REDUCESCATTER, H.COLL_REDUCE) and rng.random() < 0.4:
        servers = int(rng.choice([s for s in range(1, p + 1) if p % s == 0]))
        algo = int(rng.choice([RING, RHD]))
        if coll in (H.COLL_ALLREDUCE, H.COLL_REDUCESCATTER) and rng.random() < 0.4 and (coll == H.COLL_ALLREDUCE or servers > 1):
            rings = 4 if p // servers == 8 and rng.random() < 0.6 else 1
    mask = 0
    if coll == H.COLL_ALLREDUCE and rng.random() < 0.5:
        mask = int(rng.integers(0, 1 << p))
    return coll, p, n, align, ccl, algo, servers, rings, mask, int(rng.integers(0, p))


@pytest.mark.parametrize("seed", range(8))
def test_random_plans_compute_the_plain_result(seed):
    rng = np.random.default_rng(7000 + seed)
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
            word = algo
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
            if coll == H.COLL_REDUCESCATTER and servers > 1:
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
