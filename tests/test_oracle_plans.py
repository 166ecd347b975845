"""Pins the checker's slice / chunk planners against hand-derived vectors and invariants."""
import json
import os

import pytest

import closed_forms as cf

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "slice_plans.json")))


@pytest.mark.parametrize("case", GOLD["ring"])
def test_ring_slices_golden(orc, case):
    off, size = orc.ring_slices(case["total"], case["p"], case["align"])
    assert off == case["off"] and size == case["size"]


@pytest.mark.parametrize("case", GOLD["rhd_params"])
def test_rhd_params_golden(orc, case):
    assert orc.rhd_params(case["p"]) == (case["block"], case["part1"])


@pytest.mark.parametrize("case", GOLD["rhd_slices"])
def test_rhd_slices_golden(orc, case):
    off, size = orc.rhd_slices(case["total"], case["block"], case["align"])
    assert off == case["off"] and size == case["size"]


@pytest.mark.parametrize("case", GOLD["pieces"])
def test_pieces_golden(orc, case):
    got = orc.cut_pieces(case["off"], case["size"], case["n"], case["align"])
    assert [[list(x) for x in row] for row in got] == case["pieces"]


@pytest.mark.parametrize("case", GOLD["chunks"])
def test_chunk_plan_golden(orc, case):
    got = orc.chunk_plan(case["kind"], case["count"], case["unit"], case["p"], case["ccl"], case["align"])
    assert got == case["counts"]


@pytest.mark.parametrize("align", [1, 4, 128, 512])
def test_ring_slices_invariants(orc, align):
    for p in range(1, 34):
        for total in (0, 1, 4, 127, 128, 129, 1000, 4096, 65537, 1 << 20):
            off, size = orc.ring_slices(total, p, align)
            assert len(off) == p and sum(size) == total
            pos = 0
            for o, s in zip(off, size):
                assert o == pos            # slices tile [0, total) in order; empty ones sit at `total`
                pos += s
            nonempty = [s for s in size if s]
            assert all(s % align == 0 for s in nonempty[:-1])
            assert list(zip(off, size)) == cf.slice_plan(total, p, align)


def test_rhd_params_invariants(orc):
    for p in range(1, 200):
        block, part1 = orc.rhd_params(p)
        assert block & (block - 1) == 0 and block <= p < 2 * block
        assert part1 == 2 * (p - block)
        assert (block, part1) == cf.rhd_params(p)
