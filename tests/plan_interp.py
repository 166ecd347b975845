"""Test-side interpreter of a plan (the JSON of HcclAmdDescribePlan) over numpy byte buffers.

Used on the CPU to check the product's planner and fuser against the checker before any kernel
runs; element arithmetic comes from closed_forms.combine (numpy / torch), not from the product and
not from the checker.
"""
import numpy as np

import closed_forms as cf


def _view(buf, off, n, dt):
    return buf[off:off + n].view(cf.CARRIER[dt])


def _send_side(sends, recvs, in_place):
    """in_place: True (every rank), False, or a bit mask of the ranks whose two buffers are one."""
    if in_place is True:
        return recvs
    if not in_place:
        return sends
    return [recvs[r] if (in_place >> r) & 1 else sends[r] for r in range(len(sends))]


def run_steps(plan, sends, recvs, dt, op, in_place=False):
    """sends / recvs: lists of uint8 arrays (recvs are written).  Scratch is made on demand."""
    p = plan["p"]
    scratch = [np.zeros(plan["scratchBytes"], np.uint8) for _ in range(p)]
    bufs = {0: _send_side(sends, recvs, in_place), 1: recvs, 2: scratch}
    for phase in plan["phases"]:
        writes = []
        for s in phase:
            n = s["n"]
            a = _view(bufs[s["a"][1]][s["a"][0]], s["a"][2], n, dt).copy()
            if s["r"]:
                b = _view(bufs[s["b"][1]][s["b"][0]], s["b"][2], n, dt)
                a = cf.combine(dt, op, a, b)
            writes.append((s["dst"], a))
        for dst, val in writes:
            _view(bufs[dst[1]][dst[0]], dst[2], val.nbytes, dt)[:] = val


def run_fused(plan, sends, recvs, dt, op, in_place=False):
    assert plan["fusedOk"]
    src_bufs = _send_side(sends, recvs, in_place)
    results = []
    for it in plan["fused"]:
        n = it["n"]
        def load(ref):
            return _view(src_bufs[ref[0]] if ref[1] == 0 else recvs[ref[0]], ref[2], n, dt).copy()
        if it["kind"] in (0, 1):
            acc = load(it["src"][0])
            for j in range(1, len(it["src"])):
                v = load(it["src"][j])
                acc = cf.combine(dt, op, acc, v) if it["accLeft"][j] else cf.combine(dt, op, v, acc)
        elif it["kind"] == 3:
            # stack form: push each source, then fold the two topmost values ops[j] & 7 times
            stack = []
            for j, ref in enumerate(it["src"]):
                stack.append(load(ref))
                for f in range(it["ops"][j] & 7):
                    top = stack.pop()
                    under = stack.pop()
                    lower_is_left = (it["ops"][j] >> (8 + f)) & 1
                    stack.append(cf.combine(dt, op, under, top) if lower_is_left else cf.combine(dt, op, top, under))
            assert len(stack) == 1
            acc = stack[0]
        else:
            leaves = []
            for i in range(it["nleaf"]):
                v = load(it["src"][2 * i])
                if it["src"][2 * i + 1] is not None:
                    v = cf.combine(dt, op, v, load(it["src"][2 * i + 1]))
                leaves.append(v)
            w = 1
            while w < it["nleaf"]:
                for i in range(0, it["nleaf"], 2 * w):
                    leaves[i] = cf.combine(dt, op, leaves[i], leaves[i + w])
                w *= 2
            acc = leaves[0]
        results.append((it["dst"], acc))
    for dsts, val in results:           # all reads happen before any write, as in one fused pass
        for d in dsts:
            _view(recvs[d[0]], d[2], val.nbytes, dt)[:] = val
