"""Independent closed forms used to pin the CPU checker and the HIP library.

Nothing here shares code with oracle/hccl_oracle.cc or with the product: element arithmetic comes
from numpy / torch, schedules are written as the reduction chains and trees the templates imply.
"""
import numpy as np
import torch

INT8, INT16, INT32, FP16, FP32, INT64, UINT64, UINT8, UINT16, UINT32, FP64, BF16 = range(12)
SUM, PROD, MAX, MIN = range(4)

CARRIER = {
    INT8: np.int8, INT16: np.int16, INT32: np.int32, FP16: np.uint16, FP32: np.float32, INT64: np.int64,
    UINT64: np.uint64, UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32, FP64: np.float64, BF16: np.uint16,
}
UNSIGNED_VIEW = {INT8: np.uint8, INT16: np.uint16, INT32: np.uint32, INT64: np.uint64,
                 UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32, UINT64: np.uint64}
INT_TYPES = tuple(UNSIGNED_VIEW)
ALL_TYPES = tuple(CARRIER)


def bf16_bits_to_f32(bits):
    return torch.from_numpy(bits.astype(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()


def f32_to_bf16_bits(x):
    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().astype(np.uint16)


def widen(dt, x):
    if dt == FP16:
        return x.view(np.float16).astype(np.float32)
    if dt == BF16:
        return bf16_bits_to_f32(x)
    return x


def narrow(dt, x):
    if dt == FP16:
        with np.errstate(over="ignore"):
            return x.astype(np.float16).view(np.uint16)
    if dt == BF16:
        return f32_to_bf16_bits(x)
    return x


def combine(dt, op, a, b):
    """a (+) b with a the local operand, b the received one; carrier arrays in, carrier array out."""
    with np.errstate(over="ignore", invalid="ignore"):
        if dt in INT_TYPES:
            if op in (SUM, PROD):
                ua, ub = a.view(UNSIGNED_VIEW[dt]), b.view(UNSIGNED_VIEW[dt])
                r = (ua + ub) if op == SUM else (ua * ub)
                return r.astype(UNSIGNED_VIEW[dt]).view(CARRIER[dt])
            return np.where(b > a, b, a) if op == MAX else np.where(b < a, b, a)
        fa, fb = widen(dt, a), widen(dt, b)
        if op == SUM:
            return narrow(dt, fa + fb)
        if op == PROD:
            return narrow(dt, fa * fb)
        pick = (fb > fa) if op == MAX else (fb < fa)
        return np.where(pick, b, a)


def slice_plan(total, n, align):
    per = -(-total // n)
    per = -(-per // align) * align
    out, residue = [], total
    for _ in range(n):
        size = min(per, residue)
        out.append((total - residue, size))
        residue -= size
    return out


def broadcast_slices(count, unit, n, align):
    """Slices of the mesh broadcast's scatter / all-gather (CollBroadcastExecutor::GetRankSliceSize,
    coll_broadcast_executor.cc:275-306): ceil-ish share of the bytes rounded up to `align`, the rest to the last."""
    share = (count * unit) // n + (1 if count % n else 0)
    per = -(-share // align) * align
    out, residue = [], count * unit
    for i in range(n):
        size = min(per, residue)
        out.append((i * per if size else 0, size))
        residue -= size
    return out


def ring_chain(dt, op, xs, s):
    """Ring reduce-scatter result for slice s: x[s] (+) (x[s-1] (+) (... (x[s+2] (+) x[s+1])))."""
    p = len(xs)
    acc = xs[(s + 1) % p]
    for j in range(2, p + 1):
        acc = combine(dt, op, xs[(s + j) % p], acc)
    return acc


def ring_allreduce(dt, op, ins, unit, ccl_bytes, align):
    p = len(ins)
    n = ins[0].size
    if p == 1:
        return [ins[0].copy()]
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for s, (off, size) in enumerate(slice_plan(cur * unit, p, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi > lo:
                out[lo:hi] = ring_chain(dt, op, [x[lo:hi] for x in ins], s)
        base += cur
    return [out.copy() for _ in range(p)]


def ring_pruned_allreduce(dt, op, ins, unit, ccl_bytes, align, nic):
    """Ring all-reduce over 8 ranks of which only `nic` (ascending) own a network port: the 8 slices of a chunk of
    the loop form len(nic) runs of 8 / len(nic) slices, and every slice of run j is the ring chain that ends at rank
    nic[j] (reduce_scatter_ring.cc:299-477) instead of at the rank with the slice's own number."""
    p = len(ins)
    assert p == 8 and len(nic) in (1, 2, 4)
    run = 8 // len(nic)
    n = ins[0].size
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for s, (off, size) in enumerate(slice_plan(cur * unit, p, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi > lo:
                out[lo:hi] = ring_chain(dt, op, [x[lo:hi] for x in ins], nic[s // run])
        base += cur
    return [out.copy() for _ in range(p)]


def mesh_chain(dt, op, xs, r, t):
    """Deterministic mesh reduce-scatter, piece t of slice r: x[r] (+) x[r-1-((0+t)%(p-1))] (+) ... left to right."""
    p = len(xs)
    acc = xs[r]
    for rnd in range(1, p):
        order = (rnd + t - 1) % (p - 1)
        acc = combine(dt, op, acc, xs[(r - (order + 1)) % p])
    return acc


def mesh_allreduce(dt, op, ins, unit, ccl_bytes, align):
    p = len(ins)
    n = ins[0].size
    if p == 1:
        return [ins[0].copy()]
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    nstream = p - 1 if p > 2 else 1
    while base < n:
        cur = min(n - base, max_per)
        for r, (off, size) in enumerate(slice_plan(cur * unit, p, align)):
            if size == 0:
                continue
            for t, (poff, psize) in enumerate(slice_plan(size, nstream, align)):
                lo, hi = base + (off + poff) // unit, base + (off + poff + psize) // unit
                if hi > lo:
                    out[lo:hi] = mesh_chain(dt, op, [x[lo:hi] for x in ins], r, t)
        base += cur
    return [out.copy() for _ in range(p)]


def mesh_atomic_chain(dt, op, xs, r):
    """Mesh reduce-scatter without the piece cut, streams taken in index order:
    ((x[r] (+) x[r+1]) (+) x[r+2]) ... (+) x[r+p-1]."""
    p = len(xs)
    acc = xs[r]
    for j in range(p - 1):
        acc = combine(dt, op, acc, xs[(r + 1 + j) % p])
    return acc


def mesh_atomic_allreduce(dt, op, ins, unit, ccl_bytes, align):
    p = len(ins)
    n = ins[0].size
    if p == 1:
        return [ins[0].copy()]
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for r, (off, size) in enumerate(slice_plan(cur * unit, p, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi > lo:
                out[lo:hi] = mesh_atomic_chain(dt, op, [x[lo:hi] for x in ins], r)
        base += cur
    return [out.copy() for _ in range(p)]


def rhd_params(p):
    block = 1
    while block * 2 <= p:
        block *= 2
    return block, 2 * (p - block)


def rhd_tree(dt, op, xs, q, block, part1, par=0):
    """Value held by block rank q for its own slice after the halving phase.  par: parity of the rank
    that stands for a folded pair (0 in the all-reduce; the root's parity in the rooted reduce)."""
    def leaf(b):
        if 2 * b < part1:
            return combine(dt, op, xs[2 * b + par], xs[(2 * b + par) ^ 1])
        return xs[b + part1 // 2]

    steps = block.bit_length() - 1

    def v(b, s):
        if s == 0:
            return leaf(b)
        mask = block >> s
        return combine(dt, op, v(b, s - 1), v(b ^ mask, s - 1))

    return v(q, steps)


def rhd_allreduce(dt, op, ins, unit, ccl_bytes, align):
    p = len(ins)
    n = ins[0].size
    if p == 1:
        return [ins[0].copy()]
    block, part1 = rhd_params(p)
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for q, (off, size) in enumerate(slice_plan(cur * unit, block, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi > lo:
                out[lo:hi] = rhd_tree(dt, op, [x[lo:hi] for x in ins], q, block, part1)
        base += cur
    return [out.copy() for _ in range(p)]


def rhd_reduce_to_root(dt, op, ins, unit, ccl_bytes, align, root):
    """Recursive halving-doubling reduce: the all-reduce tree, with the folded pairs represented by the
    rank that has the root's parity (rank 0's parity when the root is outside part one)."""
    p = len(ins)
    n = ins[0].size
    if p == 1:
        return ins[0].copy()
    block, part1 = rhd_params(p)
    par = (0 if root >= part1 else root) % 2
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for q, (off, size) in enumerate(slice_plan(cur * unit, block, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi > lo:
                out[lo:hi] = rhd_tree(dt, op, [x[lo:hi] for x in ins], q, block, part1, par)
        base += cur
    return out


def two_level_allreduce(dt, op, ins, unit, ccl_bytes, align, servers, level1, atomic):
    """Groups of D = p / servers consecutive ranks: mesh chain inside a group for slice d (per piece when the
    slice is cut), then the level-1 closed form (ring_allreduce or rhd_allreduce) over the groups' partial
    results of that slice."""
    p = len(ins)
    D = p // servers
    n = ins[0].size
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for d, (off, size) in enumerate(slice_plan(cur * unit, D, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi <= lo:
                continue
            partial = []
            for s in range(servers):
                xs = [x[lo:hi] for x in ins[s * D:(s + 1) * D]]
                if D == 1:
                    partial.append(xs[0].copy())
                elif atomic:
                    partial.append(mesh_atomic_chain(dt, op, xs, d))
                else:
                    acc = np.empty_like(xs[0])
                    nstream = D - 1 if D > 2 else 1
                    for t, (poff, psize) in enumerate(slice_plan(size, nstream, align)):
                        a, b = poff // unit, (poff + psize) // unit
                        if b > a:
                            acc[a:b] = mesh_chain(dt, op, [x[a:b] for x in xs], d, t)
                    partial.append(acc)
            out[lo:hi] = level1(dt, op, partial, unit, 1 << 62, align)[0]
        base += cur
    return [out.copy() for _ in range(p)]


EIGHT_DEVICE_RINGS = ((0, 1, 2, 6, 5, 4, 7, 3), (0, 3, 7, 4, 5, 6, 2, 1), (0, 2, 3, 1, 5, 7, 6, 4), (0, 4, 6, 7, 5, 1, 3, 2))


def two_level_ring_allreduce(dt, op, ins, unit, ccl_bytes, align, servers, level1, rings):
    """Groups of D = p / servers consecutive ranks with ring(s) inside: the slice of device `dev` is cut into one
    part per ring; part k is the ring chain over the group's ranks taken in ring k's order, at the position
    of `dev` in that order.  Then the level-1 closed form over the groups' partial results of the slice."""
    p = len(ins)
    D = p // servers
    n = ins[0].size
    orders = EIGHT_DEVICE_RINGS if rings == 4 else (tuple(range(D)),)
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for dev, (off, size) in enumerate(slice_plan(cur * unit, D, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi <= lo:
                continue
            partial = []
            for s in range(servers):
                xs = [x[lo:hi] for x in ins[s * D:(s + 1) * D]]
                if D == 1:
                    partial.append(xs[0].copy())
                    continue
                acc = np.empty_like(xs[0])
                for k, (poff, psize) in enumerate(slice_plan(size, len(orders), align)):
                    a, b = poff // unit, (poff + psize) // unit
                    if b > a:
                        order = orders[k]
                        acc[a:b] = ring_chain(dt, op, [xs[order[i]][a:b] for i in range(D)], order.index(dev))
                partial.append(acc)
            out[lo:hi] = level1(dt, op, partial, unit, 1 << 62, align)[0]
        base += cur
    return [out.copy() for _ in range(p)]


def two_level_reducescatter(dt, op, ins, unit, ccl_bytes, align, servers, level1, atomic, rings=0):
    """Groups of D = p / servers consecutive ranks.  Block j = s * D + d of every input is first reduced over the
    ranks at one position d' of all groups (level1 "ring": the ring chain for ring slice s; "rhd": the halving
    tree of the block rank that owns slice s), giving one partial per position; the partials are then reduced
    by the mesh chain of rank d inside group s (per piece when the block is cut)."""
    p = len(ins)
    D = p // servers
    n = ins[0].size // p
    max_per = ccl_bytes // (p * unit)
    block, part1 = rhd_params(servers)
    outs = []
    for r in range(p):
        s, d = divmod(r, D)
        out = np.empty(n, dtype=ins[0].dtype)
        base = 0
        while base < n:
            cur = min(n - base, max_per)
            lo = r * n + base
            partial = []
            for dd in range(D):
                xs = [ins[ss * D + dd][lo:lo + cur] for ss in range(servers)]
                if servers == 1:
                    partial.append(xs[0])
                elif level1 == "ring":
                    partial.append(ring_chain(dt, op, xs, s))
                else:
                    q = s // 2 if s < part1 else s - part1 // 2
                    partial.append(rhd_tree(dt, op, xs, q, block, part1))
            if D == 1:
                out[base:base + cur] = partial[0]
            elif rings:
                # ring(s) inside the group: part k of the block goes round ring k, whose order decides the chain
                orders = EIGHT_DEVICE_RINGS if rings == 4 else (tuple(range(D)),)
                for k, (poff, psize) in enumerate(slice_plan(cur * unit, len(orders), align)):
                    a, b = poff // unit, (poff + psize) // unit
                    if b > a:
                        order = orders[k]
                        out[base + a:base + b] = ring_chain(dt, op, [partial[order[i]][a:b] for i in range(D)], order.index(d))
            elif atomic:
                out[base:base + cur] = mesh_atomic_chain(dt, op, partial, d)
            else:
                nstream = D - 1 if D > 2 else 1
                for t, (poff, psize) in enumerate(slice_plan(cur * unit, nstream, align)):
                    a, b = poff // unit, (poff + psize) // unit
                    if b > a:
                        out[base + a:base + b] = mesh_chain(dt, op, [x[a:b] for x in partial], d, t)
            base += cur
        outs.append(out)
    return outs


def two_level_reduce_to_root(dt, op, ins, unit, ccl_bytes, align, servers, level1, atomic, root, rings=0):
    """Groups of D = p / servers consecutive ranks: the mesh chain inside every group for slice d (per piece when the
    slice is cut), then the groups' partial results of that slice reduced towards the root's group: level1 "ring" is
    the ring chain ending at that group, "rhd" the halving-doubling reduce tree."""
    p = len(ins)
    D = p // servers
    n = ins[0].size
    root_server = root // D
    out = np.empty_like(ins[0])
    max_per = ccl_bytes // unit
    base = 0
    while base < n:
        cur = min(n - base, max_per)
        for d, (off, size) in enumerate(slice_plan(cur * unit, D, align)):
            lo, hi = base + off // unit, base + (off + size) // unit
            if hi <= lo:
                continue
            partial = []
            for s in range(servers):
                xs = [x[lo:hi] for x in ins[s * D:(s + 1) * D]]
                if D == 1:
                    partial.append(xs[0].copy())
                elif rings:
                    orders = EIGHT_DEVICE_RINGS if rings == 4 else (tuple(range(D)),)
                    acc = np.empty_like(xs[0])
                    for k, (poff, psize) in enumerate(slice_plan(size, len(orders), align)):
                        a, b = poff // unit, (poff + psize) // unit
                        if b > a:
                            order = orders[k]
                            acc[a:b] = ring_chain(dt, op, [xs[order[i]][a:b] for i in range(D)], order.index(d))
                    partial.append(acc)
                elif atomic:
                    partial.append(mesh_atomic_chain(dt, op, xs, d))
                else:
                    acc = np.empty_like(xs[0])
                    nstream = D - 1 if D > 2 else 1
                    for t, (poff, psize) in enumerate(slice_plan(size, nstream, align)):
                        a, b = poff // unit, (poff + psize) // unit
                        if b > a:
                            acc[a:b] = mesh_chain(dt, op, [x[a:b] for x in xs], d, t)
                    partial.append(acc)
            if servers == 1:
                out[lo:hi] = partial[0]
            elif level1 == "ring":
                out[lo:hi] = ring_chain(dt, op, partial, root_server)
            else:
                out[lo:hi] = rhd_reduce_to_root(dt, op, partial, unit, 1 << 62, align, root_server)
        base += cur
    return out


def naive_reduce(dt, op, xs):
    acc = xs[0]
    for x in xs[1:]:
        acc = combine(dt, op, acc, x)
    return acc


def random_input(dt, n, rng, small=False):
    """Carrier array of n random elements; `small` keeps floats integer-valued so sums are exact."""
    if dt in (FP32, FP64):
        if small:
            return rng.integers(-64, 65, n).astype(CARRIER[dt])
        return rng.uniform(-1.0, 1.0, n).astype(CARRIER[dt])
    if dt == FP16:
        v = rng.integers(-8, 9, n).astype(np.float32) if small else rng.standard_normal(n).astype(np.float32)
        return v.astype(np.float16).view(np.uint16)
    if dt == BF16:
        v = rng.integers(-8, 9, n).astype(np.float32) if small else rng.standard_normal(n).astype(np.float32)
        return f32_to_bf16_bits(v)
    if dt == INT64:
        return rng.integers(-(1 << 40), (1 << 40), n, dtype=np.int64)
    if dt == UINT64:
        return rng.integers(0, 1 << 63, n, dtype=np.uint64)
    info = np.iinfo(CARRIER[dt])
    return rng.integers(info.min, int(info.max) + 1, n, dtype=np.int64).astype(CARRIER[dt])
