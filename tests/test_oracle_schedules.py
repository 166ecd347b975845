"""Pins the checker's schedules (message-passing restatement) against closed forms that do not share
code with it: reduction chains / trees evaluated with numpy + torch arithmetic, order-independent
integer results, and permutation closed forms."""
import numpy as np
import pytest

import closed_forms as cf
from closed_forms import (ALL_TYPES, BF16, FP16, FP32, FP64, INT8, INT32, INT64, INT_TYPES, MAX, MIN, PROD, SUM)

RING, MESH, RHD, MESH_ATOMIC = 0, 1, 2, 4
OPS = (SUM, PROD, MAX, MIN)


def test_element_ops_match_numpy_and_torch(orc):
    rng = np.random.default_rng(1)
    for dt in ALL_TYPES:
        a = cf.random_input(dt, 4099, rng)
        b = cf.random_input(dt, 4099, rng)
        for op in OPS:
            got = orc.reduce(dt, op, a, b)
            want = cf.combine(dt, op, a, b)
            if dt in (FP16, BF16, FP32, FP64):
                both_nan = np.isnan(cf.widen(dt, got).astype(np.float64)) & np.isnan(cf.widen(dt, want).astype(np.float64))
                assert np.array_equal(got[~both_nan], want[~both_nan]), (dt, op)
            else:
                assert np.array_equal(got, want), (dt, op)


def test_half_conversions_exhaustive(orc):
    # every fp16 bit pattern widens exactly as numpy does, and narrows back to itself
    bits = np.arange(65536, dtype=np.uint16)
    f = orc.fp16_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(f[ok].view(np.uint32), ref[ok].view(np.uint32))
    assert np.array_equal(orc.f32_to_fp16(f)[ok], bits[ok])
    # every bf16 bit pattern likewise (torch is the independent converter)
    fb = orc.bf16_to_f32(bits)
    refb = cf.bf16_bits_to_f32(bits)
    okb = ~np.isnan(refb)
    assert np.array_equal(fb[okb].view(np.uint32), refb[okb].view(np.uint32))
    assert np.array_equal(orc.f32_to_bf16(fb)[okb], bits[okb])


def test_narrowing_rounds_to_nearest_even(orc):
    rng = np.random.default_rng(2)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000).astype(np.float32),
        np.array([65504.0, 65519.9, 65520.0, 70000.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -14,
                  6.1e-5, 5.96e-8, 2.98e-8, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)])
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.f32_to_fp16(x), x.astype(np.float16).view(np.uint16))
    assert np.array_equal(orc.f32_to_bf16(x), cf.f32_to_bf16_bits(x))
    # halfway cases for bf16: 1 + 2^-8 ties to even (1.0), 1 + 3*2^-8 ties to 1 + 2^-6
    t = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], dtype=np.float32)
    assert list(orc.f32_to_bf16(t)) == [0x3f80, 0x3f82]


def _inputs(dt, p, n, seed, small=False):
    rng = np.random.default_rng(seed)
    return [cf.random_input(dt, n, rng, small) for _ in range(p)]


def _eq(dt, got, want):
    if dt in (FP16, BF16, FP32, FP64):
        g, w = cf.widen(dt, got).astype(np.float64), cf.widen(dt, want).astype(np.float64)
        nn = np.isnan(g) & np.isnan(w)
        return np.array_equal(got[~nn], want[~nn])
    return np.array_equal(got, want)


CLOSED = {RING: cf.ring_allreduce, MESH: cf.mesh_allreduce, RHD: cf.rhd_allreduce, MESH_ATOMIC: cf.mesh_atomic_allreduce}


@pytest.mark.parametrize("algo", [RING, MESH, RHD, MESH_ATOMIC])
def test_allreduce_fp32_sum_matches_closed_form_all_p(orc, algo):
    # fp32 sum is order-sensitive: only the right chain / tree reproduces these bits
    for p in range(1, 34):
        n = 257 + 3 * p
        ins = _inputs(FP32, p, n, 100 + p)
        for align in (4, 128):
            got = orc.allreduce(ins, FP32, SUM, algo=algo, align=align)
            want = CLOSED[algo](FP32, SUM, ins, 4, 200 << 20, align)
            for r in range(p):
                assert np.array_equal(got[r], want[r]), (algo, p, align, r)


@pytest.mark.parametrize("algo", [RING, MESH, RHD, MESH_ATOMIC])
@pytest.mark.parametrize("dt", ALL_TYPES)
def test_allreduce_all_types_ops_match_closed_form(orc, algo, dt):
    unit = orc.dtype_size(dt)
    for p in (2, 3, 5, 8, 12):
        for op in OPS:
            ins = _inputs(dt, p, 1000, 7 * p + op)
            got = orc.allreduce(ins, dt, op, algo=algo)
            want = CLOSED[algo](dt, op, ins, unit, 200 << 20, 128)
            for r in range(p):
                assert _eq(dt, got[r], want[r]), (algo, dt, p, op, r)


@pytest.mark.parametrize("algo", [RING, MESH, RHD, MESH_ATOMIC])
def test_allreduce_chunked_matches_closed_form(orc, algo):
    # CCL buffer smaller than the payload: the chunk loop restarts the slice plan per chunk
    p, n = 8, 5000
    ins = _inputs(FP32, p, n, 5)
    for ccl in (4096, 4100, 1 << 14):
        got = orc.allreduce(ins, FP32, SUM, algo=algo, ccl_bytes=ccl)
        want = CLOSED[algo](FP32, SUM, ins, 4, ccl, 128)
        for r in range(p):
            assert np.array_equal(got[r], want[r]), (algo, ccl, r)


def test_ring_order_sensitive_known_answer(orc):
    # p = 4, one element per slice (align 4): slice 0 must be x0 + (x3 + (x2 + x1)).
    # With x1 = 2^24, x2 = 1, x3 = -2^24, x0 = 1: (2^24 + 1) = 2^24 in fp32, then -2^24 -> 0, then +1 -> 1.
    # A left-to-right sum x0+x1+x2+x3 gives 0 + ... = (1+2^24)=2^24, +1 = 2^24, -2^24 = 0.
    big = np.float32(2.0 ** 24)
    xs = [np.array([1, 0, 0, 0], np.float32), np.array([big, 0, 0, 0], np.float32),
          np.array([1, 0, 0, 0], np.float32), np.array([-big, 0, 0, 0], np.float32)]
    got = orc.allreduce(xs, FP32, SUM, algo=RING, align=4)
    assert got[0][0] == np.float32(1.0)
    assert all(np.array_equal(got[0], g) for g in got)


@pytest.mark.parametrize("algo", [RING, MESH, RHD, MESH_ATOMIC])
@pytest.mark.parametrize("dt", INT_TYPES)
def test_integer_results_are_schedule_independent(orc, algo, dt):
    for p in (2, 3, 7, 8, 16, 24):
        for op in OPS:
            ins = _inputs(dt, p, 777, p + 31 * op)
            got = orc.allreduce(ins, dt, op, algo=algo)
            want = cf.naive_reduce(dt, op, ins)
            for r in range(p):
                assert np.array_equal(got[r], want), (algo, dt, p, op)


@pytest.mark.parametrize("algo", [RING, MESH, RHD])
def test_exact_float_sums_equal_integer_sums(orc, algo):
    for dt in (FP32, FP16, BF16, FP64):
        for p in (3, 8, 24):
            ins = _inputs(dt, p, 513, p, small=True)
            got = orc.allreduce(ins, dt, SUM, algo=algo)
            exact = sum(cf.widen(dt, x).astype(np.float64) for x in ins)
            assert np.array_equal(cf.widen(dt, got[0]).astype(np.float64), exact), (algo, dt, p)


@pytest.mark.parametrize("algo", [RING, MESH, RHD])
def test_modes_agree(orc, algo):
    # snapshot vs pointer messages, staged vs zero-staging, 1 vs 4 threads, in-place vs out-of-place
    p, n = 6, 70001
    ins = _inputs(FP32, p, n, 9)
    base = orc.allreduce(ins, FP32, SUM, algo=algo)
    for flags in (orc.DIRECT, orc.ZERO_STAGING, orc.DIRECT | orc.ZERO_STAGING):
        for threads in (1, 4):
            work = [x.copy() for x in ins]
            got = orc.allreduce(work, FP32, SUM, algo=algo, flags=flags, threads=threads)
            for r in range(p):
                assert np.array_equal(got[r], base[r]), (algo, flags, threads)
            if not flags & orc.ZERO_STAGING:
                assert all(np.array_equal(w, x) for w, x in zip(work, ins))   # staged mode leaves inputs alone
    work = [x.copy() for x in ins]
    got = orc.allreduce(work, FP32, SUM, algo=algo, outs=work)                 # in place
    for r in range(p):
        assert np.array_equal(got[r], base[r])


def test_zero_staging_byte_count_matches_formula(orc):
    # ring all-reduce out-of-place touches (5p - 3) * S bytes when slices are equal
    p, n = 8, 1 << 16
    ins = _inputs(FP32, p, n, 3)
    _, touched = orc.allreduce([x.copy() for x in ins], FP32, SUM, flags=orc.DIRECT | orc.ZERO_STAGING, return_touched=True)
    assert touched == (5 * p - 3) * n * 4


def test_reducescatter_rhd_matches_tree(orc):
    # standalone recursive halving-doubling reduce-scatter: rank r's block is the halving tree of the
    # block rank that owns it (a pair of ranks shares one block rank in the fold part)
    for dt in (FP32, BF16, INT32):
        for p in (1, 2, 3, 5, 6, 8, 12, 24):
            n = 211
            for op in (SUM, MAX):
                ins = _inputs(dt, p, n * p, 3 * p + op)
                for ccl in (200 << 20, 128 * p * 2):
                    got = orc.reducescatter(ins, dt, op, algo=RHD, ccl_bytes=ccl)
                    block, part1 = cf.rhd_params(p)
                    for r in range(p):
                        xs = [x[r * n:(r + 1) * n] for x in ins]
                        q = r // 2 if r < part1 else r - part1 // 2
                        want = xs[0] if p == 1 else cf.rhd_tree(dt, op, xs, q, block, part1)
                        assert _eq(dt, got[r], want), (dt, p, op, ccl, r)


def test_allgather_rhd_is_the_permutation(orc):
    for p in (1, 2, 3, 5, 6, 8, 12, 24):
        ins = _inputs(INT32, p, 97, p)
        for ccl in (200 << 20, 128 * p * 2):
            got = orc.allgather(ins, INT32, algo=RHD, ccl_bytes=ccl)
            want = np.concatenate(ins)
            assert all(np.array_equal(g, want) for g in got), (p, ccl)


@pytest.mark.parametrize("algo", [RING, MESH, MESH_ATOMIC])
def test_reducescatter_matches_chain(orc, algo):
    for dt in (FP32, BF16, INT8, INT64):
        unit = orc.dtype_size(dt)
        for p in (1, 2, 3, 8):
            n = 333
            for op in OPS:
                ins = _inputs(dt, p, n * p, p + op)
                for ccl in (200 << 20, 128 * p * 2):
                    got = orc.reducescatter(ins, dt, op, algo=algo, ccl_bytes=ccl)
                    for r in range(p):
                        xs = [x[r * n:(r + 1) * n] for x in ins]
                        if p == 1:
                            want = xs[0]
                        elif algo == RING:
                            want = cf.ring_chain(dt, op, xs, r)
                        elif algo == MESH_ATOMIC:
                            want = cf.mesh_atomic_chain(dt, op, xs, r)
                        else:
                            want = np.empty_like(xs[0])
                            # the piece cut restarts in every chunk of the loop
                            max_per = ccl // p // 128 * 128 // unit
                            nstream = p - 1 if p > 2 else 1
                            base = 0
                            while base < n:
                                cur = min(max_per, n - base)
                                for t, (po, ps) in enumerate(cf.slice_plan(cur * unit, nstream, 128)):
                                    lo, hi = base + po // unit, base + (po + ps) // unit
                                    if hi > lo:
                                        want[lo:hi] = cf.mesh_chain(dt, op, [x[lo:hi] for x in xs], r, t)
                                base += cur
                        assert _eq(dt, got[r], want), (algo, dt, p, op, ccl, r)


@pytest.mark.parametrize("algo", [RING, MESH])
def test_allgather_is_the_permutation(orc, algo):
    for dt in (INT8, FP16, INT32, INT64):
        for p in (1, 2, 5, 8, 16):
            n = 301
            ins = _inputs(dt, p, n, p)
            for ccl in (200 << 20, 128 * p * 2):
                got = orc.allgather(ins, dt, algo=algo, ccl_bytes=ccl)
                want = np.concatenate(ins)
                for r in range(p):
                    assert np.array_equal(got[r], want), (algo, dt, p, ccl)


def _a2av_case(p, seed, max_count=300):
    rng = np.random.default_rng(seed)
    cnt = rng.integers(0, max_count, (p, p)).astype(np.uint64)
    cnt[rng.random((p, p)) < 0.15] = 0
    sdis = np.zeros((p, p), np.uint64)
    rdis = np.zeros((p, p), np.uint64)
    send_len, recv_len = [], []
    for r in range(p):
        pos = 0
        for j in rng.permutation(p):               # destinations laid out in a shuffled order, with gaps
            pos += int(rng.integers(0, 17))
            sdis[r, j] = pos
            pos += int(cnt[r, j])
        send_len.append(pos + 5)
        pos = 0
        for i in rng.permutation(p):
            pos += int(rng.integers(0, 17))
            rdis[r, i] = pos
            pos += int(cnt[i, r])
        recv_len.append(pos + 5)
    return cnt, sdis, cnt.T.copy(), rdis, send_len, recv_len


def test_alltoallv_is_the_permutation(orc):
    for p in (1, 2, 3, 8, 16):
        cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, p)
        sends = [(np.arange(n, dtype=np.int32) + (r << 20)) for r, n in enumerate(sl)]
        for scratch in (0, 64, 1000):
            recvs = [np.full(n, -1, np.int32) for n in rl]
            assert orc.alltoallv(sends, cnt, sdis, recvs, rcnt, rdis, INT32, scratch_bytes=scratch) == 0
            for j in range(p):
                want = np.full(rl[j], -1, np.int32)
                for i in range(p):
                    c = int(cnt[i, j])
                    want[int(rdis[j, i]):int(rdis[j, i]) + c] = sends[i][int(sdis[i, j]):int(sdis[i, j]) + c]
                assert np.array_equal(recvs[j], want), (p, scratch, j)


def test_alltoallv_rounds_of_the_piecewise_form(orc):
    # Hand-worked: 3 ranks, int32, a 400-byte buffer.  Step 1: rank 0 sends 1000 B (3 pieces: 400, 400, 200), rank 1
    # 800 B (2 pieces of 400), rank 2 nothing -> the slowest rank makes 3 calls (rank 1 receives 1000 B in 3 and sends
    # in 2).  Step 2: 0 -> 2 400 B (1 piece), 1 -> 0 4 B, 2 -> 1 1204 B (4 pieces: 3 x 400 + 4) -> 4 calls.
    cnt = np.array([[5, 250, 100], [1, 7, 200], [0, 301, 9]], np.uint64)
    rounds, biggest, total = orc.alltoallv_rounds(cnt, cnt.T.copy(), INT32, 400)
    assert rounds == [1, 3, 4] and biggest == 400 and total == 4 * (250 + 200 + 0 + 100 + 1 + 301)
    # with a buffer that holds every block each step is one call; an empty step makes none
    assert orc.alltoallv_rounds(cnt, cnt.T.copy(), INT32, 1 << 20)[0] == [1, 1, 1]
    only_diag = np.diag([3, 4, 5]).astype(np.uint64)
    assert orc.alltoallv_rounds(only_diag, only_diag.T.copy(), INT32, 400)[0] == [1, 0, 0]
    # any table: the slowest rank of step i needs ceil(largest block of the step / buffer) calls
    for p in (2, 5, 8):
        cnt, _, rcnt, _, _, _ = _a2av_case(p, 900 + p, max_count=3000)
        for scratch in (64, 1000, 4096):
            rounds, biggest, total = orc.alltoallv_rounds(cnt, rcnt, INT32, scratch)
            for i in range(1, p):
                big = max(int(cnt[r, (r + i) % p]) * 4 for r in range(p))
                assert rounds[i] == -(-big // scratch), (p, scratch, i)
            assert total == 4 * (int(cnt.sum()) - int(np.trace(cnt))) and biggest <= scratch


def test_staged_alltoallv_batches_of_the_buffer_copy_form(orc):
    # Hand-worked: 2 servers of 2 ranks, int8, a 10-byte buffer.  Rank 0 hands rank 2 the blocks of its server's two
    # ranks, 7 and 8 bytes: batches [7, 3] and [5] (the second block is cut where the first batch is full) = 2 batches,
    # 3 list entries.  Rank 1 hands rank 3 one block of 25 bytes and an empty one: [10] [10] [5] = 3 batches, 3 entries.
    cnt = np.zeros((4, 4), np.uint64)
    cnt[0, 2], cnt[1, 2], cnt[0, 3] = 7, 8, 25
    assert orc.alltoallv_staged_rounds(cnt, 2, INT8, 10) == ([1, 3], 6, 10)
    assert orc.alltoallv_staged_rounds(cnt, 2, INT8, 100) == ([1, 1], 3, 25)      # everything fits: one batch per run
    # any table: a pair's batches = ceil(run / buffer), and every full batch adds one cut unless it ends on a block's end
    for p, servers in ((8, 2), (12, 3), (8, 4)):
        m = p // servers
        cnt = _a2av_case(p, 950 + p, max_count=900)[0]
        for scratch in (256, 4096):
            rounds, entries, biggest = orc.alltoallv_staged_rounds(cnt, servers, INT32, scratch)
            want_entries = 0
            for i in range(1, servers):
                most = 0
                for r in range(p):
                    c, l = divmod(r, m)
                    dest = (c + i) % servers * m + l
                    blocks = [int(cnt[c * m + k, dest]) * 4 for k in range(m)]
                    most = max(most, -(-sum(blocks) // scratch))
                    ends = set(np.cumsum(blocks).tolist())
                    cuts = [x for x in range(scratch, sum(blocks), scratch) if x not in ends]
                    want_entries += sum(1 for b in blocks if b) + len(cuts)
                assert rounds[i] == most, (p, servers, scratch, i)
            assert entries == want_entries and biggest <= scratch


def _a2av_definition(p, cnt, sdis, rdis, sends, rl):
    """What an all-to-all-v is: rank j's receive buffer holds, at rdispls[j][i], the block rank i addressed to j."""
    out = []
    for j in range(p):
        want = np.full(rl[j], -1, np.int32)
        for i in range(p):
            c = int(cnt[i, j])
            want[int(rdis[j, i]):int(rdis[j, i]) + c] = sends[i][int(sdis[i, j]):int(sdis[i, j]) + c]
        out.append(want)
    return out


def test_staged_alltoallv_is_the_permutation(orc):
    # the staged route (gather inside a server, pairwise between servers) delivers exactly the definition
    for p, servers in ((4, 2), (8, 2), (8, 4), (6, 3), (6, 2), (16, 2), (16, 4), (12, 12), (5, 1), (9, 3)):
        cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 7 * p + servers)
        sends = [(np.arange(n, dtype=np.int32) + (r << 20)) for r, n in enumerate(sl)]
        keep = [x.copy() for x in sends]
        for flags in (0, orc.DIRECT):
            recvs = [np.full(n, -1, np.int32) for n in rl]
            assert orc.alltoallv_staged(sends, cnt, sdis, recvs, rcnt, rdis, INT32, servers, flags=flags) == 0
            want = _a2av_definition(p, cnt, sdis, rdis, sends, rl)
            for j in range(p):
                assert np.array_equal(recvs[j], want[j]), (p, servers, flags, j)
        assert all(np.array_equal(a, b) for a, b in zip(sends, keep))


def test_staged_alltoallv_rejects_bad_requests(orc):
    p = 6
    cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 3)
    sends = [np.zeros(n + 8, np.int32) for n in sl]
    recvs = [np.zeros(n + 8, np.int32) for n in rl]
    assert orc.alltoallv_staged(sends, cnt, sdis, recvs, rcnt, rdis, INT32, 4) == 2       # 6 ranks do not fill 4 servers
    bad = rcnt.copy()
    bad[2, 1] += 1
    assert orc.alltoallv_staged(sends, cnt, sdis, recvs, bad, rdis, INT32, 2) == 1


def test_alltoallv_rejects_asymmetric_tables(orc):
    p = 4
    cnt, sdis, rcnt, rdis, sl, rl = _a2av_case(p, 1)
    rcnt = rcnt.copy()
    rcnt[2, 1] += 1
    sends = [np.zeros(n + 8, np.int32) for n in sl]
    recvs = [np.zeros(n + 8, np.int32) for n in rl]
    assert orc.alltoallv(sends, cnt, sdis, recvs, rcnt, rdis, INT32) == 1


def test_uniform_fill_is_counter_based(orc):
    a = orc.fill_uniform_f32(100000, 42, 3, threads=1)
    b = orc.fill_uniform_f32(100000, 42, 3, threads=4)
    c = orc.fill_uniform_f32(100000, 42, 4)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(float(a.mean())) < 0.01


def _order_kat():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_fp32.json")) as f:
        return json.load(f)


def test_order_sensitive_known_answers_all_schedules(orc):
    # one hand-derived input on which ring, both mesh variants and halving-doubling give four different sums
    kat = _order_kat()
    xs = [np.array(v, np.float32) for v in kat["inputs"]]
    for name, algo in (("ring", RING), ("mesh", MESH), ("mesh_uncut", MESH_ATOMIC), ("rhd", RHD)):
        got = orc.allreduce([x.copy() for x in xs], FP32, SUM, algo=algo, align=kat["align"])
        assert all(float(g[0]) == kat["expected_element0"][name] for g in got), (name, [float(g[0]) for g in got])
        assert all(np.array_equal(g[1:], np.zeros(3, np.float32)) for g in got)
        # and the closed forms agree with the hand derivation
        want = CLOSED[algo](FP32, SUM, xs, 4, 200 << 20, kat["align"])
        assert float(want[0][0]) == kat["expected_element0"][name], name


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("atomic", [False, True])
def test_two_level_allreduce_matches_closed_form(orc, level1, atomic):
    # (servers, ranks per server): mesh inside a server, ring or halving-doubling between servers
    closed1 = cf.ring_allreduce if level1 == RING else cf.rhd_allreduce
    for servers, D in ((2, 4), (4, 2), (3, 4), (2, 8), (8, 1), (1, 8), (5, 3), (6, 2)):
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, SUM, 1501, 200 << 20),
                               (INT32, MAX, 700, 200 << 20)):
            ins = _inputs(dt, p, n, 31 * p + n)
            got = orc.allreduce_two_level(ins, dt, op, servers, level1=level1, atomic=atomic, ccl_bytes=ccl)
            want = cf.two_level_allreduce(dt, op, ins, orc.dtype_size(dt), ccl, 128, servers, closed1, atomic)
            for r in range(p):
                assert _eq(dt, got[r], want[r]), (servers, D, level1, atomic, dt, ccl, r)
    # one server is the plain mesh all-reduce
    ins = _inputs(FP32, 8, 4099, 5)
    a = orc.allreduce_two_level(ins, FP32, SUM, 1, level1=level1, atomic=atomic)
    b = orc.allreduce(ins, FP32, SUM, algo=MESH_ATOMIC if atomic else MESH)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["ring", "ring4"])
def test_two_level_allreduce_with_rings_inside_a_server_matches_closed_form(orc, level1, level0):
    # ring(s) inside a server (one ring in rank order, or the four rings of the 8-device topology, each on its
    # part of every slice), ring or halving-doubling between servers
    closed1 = cf.ring_allreduce if level1 == RING else cf.rhd_allreduce
    shapes = ((1, 8), (2, 8), (3, 8)) if level0 == "ring4" else ((2, 4), (4, 2), (3, 4), (1, 8), (5, 3), (8, 1))
    rings = 4 if level0 == "ring4" else 1
    for servers, D in shapes:
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, SUM, 1501, 200 << 20),
                               (INT32, MAX, 700, 200 << 20), (FP32, SUM, 100, 200 << 20)):
            ins = _inputs(dt, p, n, 37 * p + n)
            got = orc.allreduce_two_level(ins, dt, op, servers, level1=level1, level0=level0, ccl_bytes=ccl)
            want = cf.two_level_ring_allreduce(dt, op, ins, orc.dtype_size(dt), ccl, 128, servers, closed1, rings)
            for r in range(p):
                assert _eq(dt, got[r], want[r]), (servers, D, level1, level0, dt, ccl, r)
    # one server with one ring is the plain ring all-reduce
    ins = _inputs(FP32, 8, 4099, 5)
    a = orc.allreduce_two_level(ins, FP32, SUM, 1, level1=level1, level0="ring")
    b = orc.allreduce(ins, FP32, SUM, algo=RING)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    # four rings: a different association than one ring, visible in fp32 sums of generic data
    if level0 == "ring4":
        c = orc.allreduce_two_level(ins, FP32, SUM, 1, level1=level1, level0="ring4")
        assert not all(np.array_equal(x, y) for x, y in zip(b, c))
        # every rank holds the same result whatever ring a part went through
        assert all(np.array_equal(c[0], x) for x in c)


def test_multi_ring_parts_of_a_slice():
    # the cut of one rank slice into one part per ring: RoundUp(ceil(size / rings), 128) each, the last shorter,
    # left-over rings empty (hand-computed: 1000 B over 4 rings -> 256, 256, 256, 232; 300 B -> 128, 128, 44, 0)
    assert [s for _, s in cf.slice_plan(1000, 4, 128)] == [256, 256, 256, 232]
    assert [s for _, s in cf.slice_plan(300, 4, 128)] == [128, 128, 44, 0]


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("atomic", [False, True])
def test_two_level_reducescatter_matches_closed_form(orc, level1, atomic):
    # between the servers first (ring or halving-doubling over the whole input), then the mesh inside a server
    for servers, D in ((2, 4), (4, 2), (3, 4), (2, 8), (8, 1), (5, 3), (6, 2)):
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 211, 200 << 20), (FP32, SUM, 500, 4 * p * 128), (BF16, SUM, 301, 200 << 20),
                               (INT32, MAX, 70, 200 << 20)):
            ins = _inputs(dt, p, n * p, 41 * p + n)
            got = orc.reducescatter_two_level(ins, dt, op, servers, level1=level1, atomic=atomic, ccl_bytes=ccl)
            want = cf.two_level_reducescatter(dt, op, ins, orc.dtype_size(dt), ccl, 128, servers,
                                              "ring" if level1 == RING else "rhd", atomic)
            for r in range(p):
                assert _eq(dt, got[r], want[r]), (servers, D, level1, atomic, dt, ccl, r)
    # one server is the plain mesh reduce-scatter
    ins = _inputs(FP32, 8, 8 * 409, 5)
    a = orc.reducescatter_two_level(ins, FP32, SUM, 1, level1=level1, atomic=atomic)
    b = orc.reducescatter(ins, FP32, SUM, algo=MESH_ATOMIC if atomic else MESH)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("atomic", [False, True])
def test_two_level_reduce_to_root_matches_closed_form(orc, level1, atomic):
    # mesh inside a server, then every slice reduced towards the root's server, then gathered to the root
    for servers, D in ((2, 4), (4, 2), (3, 4), (2, 8), (8, 1), (5, 3), (6, 2), (1, 4)):
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, SUM, 1501, 200 << 20),
                               (INT32, MAX, 700, 200 << 20)):
            ins = _inputs(dt, p, n, 43 * p + n)
            for root in sorted({0, p - 1, p // 2, (D + 1) % p}):
                got = orc.reduce_to_root_two_level(ins, dt, op, root, servers, level1=level1, atomic=atomic, ccl_bytes=ccl)
                want = cf.two_level_reduce_to_root(dt, op, ins, orc.dtype_size(dt), ccl, 128, servers,
                                                   "ring" if level1 == RING else "rhd", atomic, root)
                assert _eq(dt, got, want), (servers, D, level1, atomic, dt, ccl, root)
    # one server is the plain mesh reduce
    ins = _inputs(FP32, 8, 4099, 5)
    a = orc.reduce_to_root_two_level(ins, FP32, SUM, 3, 1, level1=level1, atomic=atomic)
    b = orc.reduce_to_root(ins, FP32, SUM, 3, algo=MESH_ATOMIC if atomic else MESH)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["ring", "ring4"])
def test_two_level_reducescatter_with_rings_inside_a_server_matches_closed_form(orc, level1, level0):
    rings = 4 if level0 == "ring4" else 1
    shapes = ((2, 8), (3, 8), (1, 8)) if rings == 4 else ((2, 4), (4, 2), (3, 4), (5, 3), (1, 6))
    for servers, D in shapes:
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 211, 200 << 20), (FP32, SUM, 500, 4 * p * 128), (BF16, SUM, 301, 200 << 20),
                               (INT32, MAX, 70, 200 << 20)):
            ins = _inputs(dt, p, n * p, 47 * p + n)
            got = orc.reducescatter_two_level(ins, dt, op, servers, level1=level1, level0=level0, ccl_bytes=ccl)
            want = cf.two_level_reducescatter(dt, op, ins, orc.dtype_size(dt), ccl, 128, servers,
                                              "ring" if level1 == RING else "rhd", False, rings=rings)
            for r in range(p):
                assert _eq(dt, got[r], want[r]), (servers, D, level1, level0, dt, ccl, r)


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["ring", "ring4"])
def test_two_level_reduce_to_root_with_rings_inside_a_server_matches_closed_form(orc, level1, level0):
    rings = 4 if level0 == "ring4" else 1
    shapes = ((2, 8), (3, 8), (1, 8)) if rings == 4 else ((2, 4), (4, 2), (3, 4), (5, 3))
    for servers, D in shapes:
        p = servers * D
        for dt, op, n, ccl in ((FP32, SUM, 2003, 200 << 20), (FP32, SUM, 5000, 4096), (BF16, SUM, 1501, 200 << 20)):
            ins = _inputs(dt, p, n, 53 * p + n)
            for root in sorted({0, p - 1, (D + 1) % p}):
                got = orc.reduce_to_root_two_level(ins, dt, op, root, servers, level1=level1, level0=level0, ccl_bytes=ccl)
                want = cf.two_level_reduce_to_root(dt, op, ins, orc.dtype_size(dt), ccl, 128, servers,
                                                   "ring" if level1 == RING else "rhd", False, root, rings=rings)
                assert _eq(dt, got, want), (servers, D, level1, level0, dt, ccl, root)


def test_order_sensitive_known_answers_two_level(orc):
    # the same hand-derived input on two groups of two ranks: a fifth sum for the all-reduce, and the reduce-scatter's
    # groups-first order
    kat = _order_kat()
    xs = [np.array(v, np.float32) for v in kat["inputs"]]
    want = kat["expected_two_level_2x2"]
    for level1 in (RING, RHD):
        for level0, atomic in (("mesh", False), ("mesh", True), ("ring", False)):
            got = orc.allreduce_two_level([x.copy() for x in xs], FP32, SUM, 2, level1=level1, atomic=atomic, align=kat["align"],
                                          level0=level0)
            assert all(float(g[0]) == want["allreduce_element0"] for g in got), (level1, level0, atomic)
            rs = orc.reducescatter_two_level([x.copy() for x in xs], FP32, SUM, 2, level1=level1, atomic=atomic, align=kat["align"],
                                             level0=level0)
            assert float(rs[0][0]) == want["reducescatter_rank0"], (level1, level0, atomic)
    closed = cf.two_level_allreduce(FP32, SUM, xs, 4, 200 << 20, kat["align"], 2, cf.ring_allreduce, False)
    assert float(closed[0][0]) == want["allreduce_element0"]


def _four_ring_kat():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_four_rings_fp32.json")) as f:
        kat = json.load(f)
    xs = []
    for row in kat["inputs_first4"]:
        x = np.zeros(kat["elements"], np.float32)
        x[:4] = row
        xs.append(x)
    return kat, xs


def test_order_sensitive_known_answers_four_rings(orc):
    # hand-derived: each of the first four elements travels its own ring, and only that ring's order loses the 1
    kat, xs = _four_ring_kat()
    assert [list(o) for o in cf.EIGHT_DEVICE_RINGS] == kat["ring_orders"]
    for level0 in ("ring4", "ring"):
        want = np.zeros(kat["elements"], np.float32)
        want[:4] = kat["expected_first4"][level0]
        for level1 in (RING, RHD):
            got = orc.allreduce_two_level([x.copy() for x in xs], FP32, SUM, 1, level1=level1, align=kat["align"], level0=level0)
            assert all(np.array_equal(g, want) for g in got), (level0, level1, got[0][:4])
    closed = cf.two_level_ring_allreduce(FP32, SUM, xs, 4, 200 << 20, kat["align"], 1, cf.ring_allreduce, 4)
    assert np.array_equal(closed[0][:4], np.array(kat["expected_first4"]["ring4"], np.float32))


def _two_level_pruned_kat():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_two_level_pruned_fp32.json")) as f:
        return json.load(f)


def test_two_level_reducescatter_with_fewer_ports_than_devices(orc):
    # Definition on integers for every choice of 1 and 2 port devices and some of 4, several servers, ragged counts
    # and a chunk loop; then the hand-derived order-sensitive answers, which the ordinary two-level branch misses.
    import itertools
    rng = np.random.default_rng(4100)
    ports = [list(c) for k in (1, 2) for c in itertools.combinations(range(8), k)] + [[0, 1, 2, 3], [1, 3, 4, 6], [0, 2, 5, 7]]
    for servers, n, ccl in ((2, 37, 200 << 20), (3, 200, 1 << 16), (1, 64, 200 << 20)):
        p = 8 * servers
        for nic in ports:
            ins = [rng.integers(-1000, 1000, n * p).astype(np.int32) for _ in range(p)]
            outs = orc.reducescatter_two_level_pruned(ins, INT32, SUM, servers, nic, ccl_bytes=ccl)
            total = np.sum(ins, axis=0, dtype=np.int64).astype(np.int32)
            for r in range(p):
                assert np.array_equal(outs[r], total[r * n:(r + 1) * n]), (servers, nic, r)
    kat = _two_level_pruned_kat()
    n, nic = kat["elements_per_block"], kat["nic_devices"]
    for case in kat["cases"]:
        xs = [np.full(16 * n, v, np.float32) for v in case["inputs_per_rank"]]
        got = orc.reducescatter_two_level_pruned([x.copy() for x in xs], FP32, SUM, 2, nic)
        plain = orc.reducescatter_two_level([x.copy() for x in xs], FP32, SUM, 2, level1=RING, level0="ring4")
        if "pruned_every_element" in case:
            assert all(np.all(g == np.float32(case["pruned_every_element"])) for g in got)
            assert all(np.all(g == np.float32(case["ordinary_two_level_every_element"])) for g in plain)
        else:
            for b in range(16):
                want = np.repeat(np.array(case["block_halves"][b], np.float32), n // 2)
                assert np.array_equal(got[b], want), (b, got[b][0], got[b][-1])
            assert any(not np.array_equal(g, q) for g, q in zip(got, plain))          # the ordinary branch slices block by block


@pytest.mark.parametrize("level1", [RING, RHD])
@pytest.mark.parametrize("level0", ["mesh", "ring", "ring4"])
def test_two_level_allgather_is_the_concatenation(orc, level1, level0):
    shapes = ((1, 8), (2, 8), (3, 8)) if level0 == "ring4" else ((2, 4), (4, 2), (3, 4), (5, 3), (6, 1), (1, 5))
    for servers, D in shapes:
        p = servers * D
        for dt, n, ccl in ((INT32, 1003, 200 << 20), (INT32, 777, 4096), (BF16, 301, 200 << 20), (INT8, 5000, 8192)):
            ins = _inputs(dt, p, n, 31 * p + n)
            got = orc.allgather_two_level(ins, dt, servers, level1=level1, level0=level0, ccl_bytes=ccl)
            want = np.concatenate(ins)
            for r in range(p):
                assert np.array_equal(got[r], want), (servers, D, level1, level0, dt, ccl, r)


def _v_blocks(p, seed, scale=400):
    """Block table of a variable-count collective: some empty blocks, shuffled order, gaps between the blocks."""
    rng = np.random.default_rng(seed)
    counts = rng.integers(0, scale, p)
    counts[rng.random(p) < 0.2] = 0
    displs, pos = np.zeros(p, np.int64), 0
    for i in rng.permutation(p):
        pos += int(rng.integers(0, 9))
        displs[i] = pos
        pos += int(counts[i])
    return counts, displs, pos + 3


@pytest.mark.parametrize("algo", [RING, MESH, MESH_ATOMIC, RHD])
def test_reducescatter_v_matches_chain(orc, algo):
    # the variable-count reduce-scatter runs the same templates over the caller's block table: block r comes out as
    # the ring chain / the mesh chains of its pieces, evaluated here with numpy on the block's elements alone
    for dt in (FP32, BF16, INT8, INT64):
        unit = orc.dtype_size(dt)
        for p in (1, 2, 3, 6, 8):
            for op in (SUM, MAX) if dt != FP32 else OPS:
                counts, displs, extent = _v_blocks(p, 31 * p + dt + op)
                ins = _inputs(dt, p, extent, 7 * p + op)
                got = orc.reducescatter_v(ins, counts, displs, dt, op, algo=algo)
                for r in range(p):
                    lo, n = int(displs[r]), int(counts[r])
                    xs = [x[lo:lo + n] for x in ins]
                    if p == 1:
                        want = xs[0]
                    elif algo == RING:
                        want = cf.ring_chain(dt, op, xs, r)
                    elif algo == MESH_ATOMIC:
                        want = cf.mesh_atomic_chain(dt, op, xs, r)
                    elif algo == RHD:
                        # the halving tree of the block rank that ends up with block r (a folded pair's block rank has
                        # both blocks of the pair)
                        block, part1 = cf.rhd_params(p)
                        want = cf.rhd_tree(dt, op, xs, r // 2 if r < part1 else r - part1 // 2, block, part1)
                    else:
                        want = np.empty_like(xs[0])
                        nstream = p - 1 if p > 2 else 1
                        for t, (po, ps) in enumerate(cf.slice_plan(n * unit, nstream, 128) if n else []):
                            a, b = po // unit, (po + ps) // unit
                            if b > a:
                                want[a:b] = cf.mesh_chain(dt, op, [x[a:b] for x in xs], r, t)
                    assert got[r].size == n and _eq(dt, got[r], want), (algo, dt, p, op, r)


def test_reducescatter_v_order_sensitive_known_answer(orc):
    # fp32 sums where the association decides the bits: 2^24 absorbs a 1 added to it directly.  Three ranks, the
    # three blocks in shuffled places; block r of rank j holds v[(j - r) % 3] with v = (2^24, 1, 1), so that the
    # ring (x_r + (x_{r-1} + x_{r+1})) gives 2^24 + 2 and the uncut mesh ((x_r + x_{r+1}) + x_{r+2}) gives 2^24
    big = np.float32(16777216.0)
    counts, displs = [5, 5, 5], [11, 0, 22]
    v = [big, np.float32(1.0), np.float32(1.0)]
    ins = []
    for j in range(3):
        x = np.zeros(30, np.float32)
        for r in range(3):
            x[displs[r]:displs[r] + 5] = v[(j - r) % 3]
        ins.append(x)
    ring = orc.reducescatter_v(ins, counts, displs, FP32, SUM, algo=RING)
    atomic = orc.reducescatter_v(ins, counts, displs, FP32, SUM, algo=MESH_ATOMIC)
    for r in range(3):
        assert np.all(ring[r] == np.float32(16777218.0)), r
        assert np.all(atomic[r] == big), r


@pytest.mark.parametrize("algo", [RING, MESH])
def test_allgather_v_is_the_permutation(orc, algo):
    for dt in (INT8, FP16, INT32, INT64):
        for p in (1, 2, 3, 6, 8, 13):
            counts, displs, extent = _v_blocks(p, 5 * p + dt)
            ins = [_inputs(dt, 1, int(counts[r]), 100 * p + r)[0] for r in range(p)]
            fill = 0x5A
            got = orc.allgather_v(ins, counts, displs, extent, dt, algo=algo, fill=fill)
            want = np.full(extent, fill, dtype=ins[0].dtype)
            for r in range(p):
                want[int(displs[r]):int(displs[r]) + int(counts[r])] = ins[r]
            for r in range(p):
                assert np.array_equal(got[r], want), (algo, dt, p, r)       # blocks in place, gaps untouched


def test_star_broadcast_delivers_and_every_byte_comes_from_the_root(orc):
    # Definition: every rank ends with the root's bytes.  Structure: p - 1 transfers of the whole buffer and nothing
    # else (a ring or a tree would move the same bytes; what tells the star apart is checked on the plan: every
    # transfer starts at the root).
    for p in (1, 2, 5, 8):
        for dt, n in ((INT32, 1), (INT8, 100003), (INT64, 5000)):
            for root in sorted({0, p - 1, p // 2}):
                bufs = _inputs(dt, p, n, root + n)
                src = bufs[root].copy()
                bufs, touched = orc.broadcast_star(bufs, dt, root, return_touched=True)
                assert all(np.array_equal(b, src) for b in bufs), (p, dt, n, root)
                assert touched == 2 * (p - 1) * n * orc.dtype_size(dt)


# Routes of the binary-block broadcast worked out by hand from bcast_halvingdoubling.cc (block parameters :26-62, the
# binomial tree of the root's block :165-228, block to block :231-396), as (sender, receiver), senders in rank order,
# each sender's transfers in the order it issues them.
HD_BLOCK_ROUTES = {
    (6, 5): [(4, 0), (4, 1), (5, 4), (5, 2), (5, 3)],                                         # blocks 4 + 2, root in the small one
    (7, 0): [(0, 2), (0, 1), (0, 4), (2, 3), (2, 5), (4, 6)],                                 # blocks 4 + 2 + 1, downwards twice
    (7, 4): [(4, 5), (4, 6), (4, 0), (4, 1), (5, 2), (5, 3)],                                 # the root's block serves both sides
    (7, 6): [(4, 0), (4, 1), (5, 2), (5, 3), (6, 4), (6, 5)],                                 # upwards twice
    (12, 3): [(0, 8), (1, 0), (2, 9), (3, 7), (3, 1), (3, 2), (4, 10), (5, 4), (6, 11), (7, 5), (7, 6)],
    (8, 5): [(1, 3), (1, 0), (3, 2), (5, 1), (5, 7), (5, 4), (7, 6)],                         # a power of two: one block, a tree
    (2, 1): [(1, 0)],
    (3, 1): [(0, 2), (1, 0)],
}


def test_binary_block_broadcast_routes_and_bytes(orc):
    # the hand-derived routes; the definition; every rank but the root receives exactly once (p - 1 transfers of the
    # whole buffer, so 2 (p - 1) n bytes touched), also under a chunk loop
    for (p, root), want in HD_BLOCK_ROUTES.items():
        assert orc.broadcast_hd_blocks_route(p, root) == want, (p, root)
    for p in list(range(1, 18)) + [24, 31, 33]:
        for root in sorted({0, p - 1, p // 2, p // 3}):
            route = orc.broadcast_hd_blocks_route(p, root)
            assert sorted(d for _, d in route) == [r for r in range(p) if r != root], (p, root)
            for dt, n, ccl in ((INT32, 1, 200 << 20), (INT8, 100003, 200 << 20), (INT64, 5000, 4096)):
                bufs = _inputs(dt, p, n, root + n)
                src = bufs[root].copy()
                bufs, touched = orc.broadcast_hd_blocks(bufs, dt, root, ccl_bytes=ccl, return_touched=True)
                assert all(np.array_equal(b, src) for b in bufs), (p, dt, n, root)
                assert touched == 2 * (p - 1) * n * orc.dtype_size(dt), (p, dt, n, root)
    # for a power of two it is the binomial tree of the recursive halving-doubling broadcast: same transfers
    for p in (2, 4, 8, 16):
        for root in range(p):
            route = orc.broadcast_hd_blocks_route(p, root)
            have = {root}
            mask = p >> 1
            tree = set()
            while mask:
                for q in sorted(have):
                    tree.add((q, q ^ mask))
                have |= {q ^ mask for q in have}
                mask >>= 1
            assert set(route) == tree, (p, root)


@pytest.mark.parametrize("shape", [(2, 4, 1), (3, 3, 1), (4, 2, 1), (1, 5, 1), (5, 1, 1), (2, 8, 4), (1, 8, 4), (3, 8, 4)])
def test_two_level_ring_broadcast_delivers_and_moves_the_closed_form_bytes(orc, shape):
    # Definition: every rank ends with the root's bytes.  Structure: the bytes received over all ranks are those of the
    # ring scatter in the root's group (a part that ends j positions behind the root is received j times), one
    # halving-doubling broadcast per slice between the groups, and one ring all-gather per group and ring -- a mesh
    # scatter, a flat broadcast or a scatter that started at another position would count differently.
    servers, D, rings = shape
    p = servers * D
    for dt, n in ((INT32, 1), (INT32, 1000), (INT8, 100003), (INT64, 5000)):
        unit = orc.dtype_size(dt)
        for root in sorted({0, p - 1, p // 2, D - 1, min(D, p - 1)}):
            for ccl in (200 << 20, 8192):
                bufs = _inputs(dt, p, n, root + n)
                src = bufs[root].copy()
                bufs, touched = orc.broadcast_two_level_ring(bufs, dt, root, servers, rings=rings, ccl_bytes=ccl, return_touched=True)
                assert all(np.array_equal(b, src) for b in bufs), (shape, dt, n, root, ccl)
                received, left = 0, n
                max_per = ccl // unit
                while left > 0 and p > 1:
                    cur = min(left, max_per)
                    sl = cf.slice_plan(cur * unit, D, 128)
                    for k in range(rings):
                        order = list(cf.EIGHT_DEVICE_RINGS[k]) if rings == 4 else list(range(D))
                        root_pos = order.index(root % D)
                        for j in range(1, D):
                            size = sl[order[(root_pos + j) % D]][1]
                            parts = cf.slice_plan(size, rings, 128)
                            received += j * parts[k][1]
                    received += (servers - 1) * cur * unit + servers * (D - 1) * cur * unit
                    left -= cur
                assert touched == 2 * received, (shape, dt, n, root, ccl, touched, received)


@pytest.mark.parametrize("shape", [(2, 4), (4, 2), (3, 2), (3, 4), (1, 4), (8, 1), (5, 3)])
def test_two_level_broadcast_delivers_and_moves_the_closed_form_bytes(orc, shape):
    # Definition: every rank ends with the root's bytes.  Structure: the bytes received over all ranks are those of
    # scatter (root's group) + one halving-doubling broadcast per slice between the groups + one mesh all-gather per
    # group -- a flat broadcast, or a level 1 that moved the whole buffer, would count differently.
    servers, D = shape
    p = servers * D
    for dt, n in ((INT32, 1), (INT32, 1000), (INT8, 100003), (INT64, 5000)):
        unit = orc.dtype_size(dt)
        for root in sorted({0, p - 1, p // 2, D - 1, min(D, p - 1)}):
            for ccl in (200 << 20, 8192):
                bufs = _inputs(dt, p, n, root + n)
                src = bufs[root].copy()
                bufs, touched = orc.broadcast_two_level(bufs, dt, root, servers, ccl_bytes=ccl, return_touched=True)
                assert all(np.array_equal(b, src) for b in bufs), (shape, dt, n, root, ccl)
                received, left = 0, n
                max_per = ccl // unit
                while left > 0 and p > 1:
                    cur = min(left, max_per)
                    sl = cf.broadcast_slices(cur, unit, D, 128)
                    total = cur * unit
                    if D > 1:
                        received += total - sl[root % D][1]                   # scatter in the root's group
                        received += servers * (D - 1) * total                 # all-gather in every group
                    received += (servers - 1) * total                        # slice d reaches position d of every other group
                    left -= cur
                assert touched == 2 * received, (shape, dt, n, root, ccl)


@pytest.mark.parametrize("shape", [(2, 4), (4, 2), (3, 2), (3, 4), (1, 4), (8, 1), (5, 3)])
def test_two_level_scatter_delivers_and_moves_the_closed_form_bytes(orc, shape):
    # Definition: rank r ends with block r of the root.  Structure: the root packs every block, a group's run of D
    # blocks makes as many hops round the ring of sub-roots as its group is away from the root's, every group's
    # sub-root hands out D - 1 blocks, every rank copies its block out -- a flat scatter, or a level 1 that went
    # point to point, would count differently.
    servers, D = shape
    p = servers * D
    for dt, n in ((INT32, 1), (INT32, 1000), (INT8, 10003), (INT64, 500)):
        unit = orc.dtype_size(dt)
        for root in sorted({0, p - 1, p // 2, D - 1, min(D, p - 1)}):
            for ccl in (200 << 20, 8192):
                src = _inputs(dt, 1, n * p, root + n)[0]
                outs, touched = orc.scatter_two_level(src, p, dt, root, servers, ccl_bytes=ccl, return_touched=True)
                for r in range(p):
                    assert np.array_equal(outs[r], src[r * n:(r + 1) * n]), (shape, dt, n, root, ccl, r)
                max_per = ccl // p // 128 * 128 // unit
                moved, left = 0, n
                while left > 0:
                    cur = max_per if left * unit * p > ccl else left
                    block = cur * unit
                    moved += p * block                                                  # packed by the root
                    moved += (servers * (servers - 1) // 2) * D * block                 # hops round the ring of sub-roots
                    moved += servers * (D - 1) * block                                  # handed out inside the groups
                    moved += p * block                                                  # copied out
                    left -= cur
                assert touched == 2 * moved, (shape, dt, n, root, ccl)


@pytest.mark.parametrize("shape", [(2, 4, "ring"), (3, 3, "ring"), (4, 2, "ring"), (1, 5, "ring"), (2, 8, "ring4"), (3, 8, "ring4")])
def test_two_level_scatter_with_rings_inside_delivers_and_moves_the_closed_form_bytes(orc, shape):
    # As above, but inside a group the blocks go round the ring from the sub-root: the block of the rank j positions
    # behind it makes j hops, D (D - 1) / 2 block hops per group where the mesh hands out D - 1.
    servers, D, level0 = shape
    p = servers * D
    for dt, n in ((INT32, 1), (INT32, 1000), (INT8, 10003)):
        unit = orc.dtype_size(dt)
        for root in sorted({0, p - 1, p // 2, D - 1, min(D, p - 1)}):
            for ccl in (200 << 20, 8192):
                src = _inputs(dt, 1, n * p, root + n)[0]
                outs, touched = orc.scatter_two_level(src, p, dt, root, servers, ccl_bytes=ccl, return_touched=True, level0=level0)
                for r in range(p):
                    assert np.array_equal(outs[r], src[r * n:(r + 1) * n]), (shape, dt, n, root, ccl, r)
                max_per = ccl // p // 128 * 128 // unit
                moved, left = 0, n
                while left > 0:
                    cur = max_per if left * unit * p > ccl else left
                    block = cur * unit
                    moved += 2 * p * block + (servers * (servers - 1) // 2) * D * block + servers * (D * (D - 1) // 2) * block
                    left -= cur
                assert touched == 2 * moved, (shape, dt, n, root, ccl)


PRUNED_PORTS = ([0], [5], [0, 4], [2, 3], [1, 6], [0, 2, 4, 6], [1, 2, 3, 7], [4, 5, 6, 7])


def test_ring_pruned_allreduce_matches_closed_form(orc):
    # 8 ranks, fewer network ports than ranks: every slice of run j is the ring chain ending at the j-th port rank
    for dt in (FP32, BF16, INT32):
        unit = orc.dtype_size(dt)
        for nic in PRUNED_PORTS:
            for n in (1, 8, 1000, 5003):
                for op in (SUM, MAX):
                    ins = _inputs(dt, 8, n, len(nic) * 100 + n + op)
                    for ccl in (200 << 20, 2048):
                        want = cf.ring_pruned_allreduce(dt, op, ins, unit, ccl, 128, nic)
                        for flags in (0, orc.DIRECT, orc.DIRECT | orc.ZERO_STAGING):
                            got = orc.allreduce_ring_pruned([x.copy() for x in ins], dt, op, nic, ccl_bytes=ccl, flags=flags)
                            for r in range(8):
                                assert _eq(dt, got[r], want[r]), (dt, nic, n, op, ccl, flags, r)


def _pruned_kat():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "order_sensitive_ring_pruned_fp32.json")) as f:
        return json.load(f)


def test_ring_pruned_order_sensitive_known_answers(orc):
    kat = _pruned_kat()
    n = kat["elements"]
    ins = [np.full(n, v, np.float32) for v in kat["inputs_per_rank"]]
    per = n // 8
    for case in kat["cases"]:
        want = np.repeat(np.array(case["slice_values"], np.float32), per)
        got = orc.allreduce_ring_pruned([x.copy() for x in ins], FP32, SUM, case["nic_ranks"])
        for r in range(8):
            assert np.array_equal(got[r], want), (case["nic_ranks"], r)
    plain = np.repeat(np.array(kat["plain_ring"]["slice_values"], np.float32), per)
    got = orc.allreduce([x.copy() for x in ins], FP32, SUM, algo=RING)
    assert all(np.array_equal(g, plain) for g in got)            # and the plain ring differs where the chains end elsewhere


def test_ring_pruned_send_lists_match_the_hand_derived_ones(orc):
    # ReduceScatterSlicesPrep for ports {0, 4} (chunks of 4 slices): rank r sends the chunk of every port rank other
    # than itself, the nearest port rank behind it first.  Checked through the traffic: integer sums are right only if
    # every slice passes every rank once; the per-rank send order decides nothing else, so it is pinned by running
    # with snapshot messages (flags 0), where a wrong order deadlocks or mismatches message lengths.
    rng = np.random.default_rng(4)
    for nic in PRUNED_PORTS:
        sizes = rng.integers(1, 4000, 3)
        for n in sizes:
            ins = [rng.integers(-1000, 1000, int(n)).astype(np.int32) for _ in range(8)]
            got = orc.allreduce_ring_pruned([x.copy() for x in ins], INT32, SUM, nic)
            assert all(np.array_equal(g, sum(ins)) for g in got), (nic, n)
