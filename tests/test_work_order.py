"""The work order of the attention launches (dl4s_amd/csrc/work_order.h), compiled for the host: whatever the pair
count, the units per pair, the longest-first flag and the round reversal, the grid of 8 * ceil(total / 8) workgroups
must hand out every (pair, unit) item exactly once and mark the rest as padding; a pair must stay on one XCD
(workgroup index % 8), which is what lets its workgroups share K and V in one L2."""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def shim():
    out = os.path.join(tempfile.mkdtemp(prefix="dl4s_work_order_"), "libwork_order.so")
    subprocess.check_call(["g++", "-O1", "-shared", "-fPIC", "-std=c++17", "-o", out, os.path.join(HERE, "work_order_shim.cpp")])
    lib = C.CDLL(out)
    lib.work_item_at.argtypes = [C.c_int] * 5 + [C.POINTER(C.c_int)] * 2
    lib.work_item_at.restype = C.c_int
    return lib


def items(lib, npairs, nunits, lpt, snake):
    total = npairs * nunits
    grid = (total + 7) // 8 * 8
    bh, unit = C.c_int(), C.c_int()
    got = []
    for block in range(grid):
        if lib.work_item_at(block, nunits, total, lpt, snake, C.byref(bh), C.byref(unit)):
            got.append((block, bh.value, unit.value))
    return total, got


@pytest.mark.parametrize("lpt", [0, 1])
@pytest.mark.parametrize("snake", [0, 32, 5])
def test_every_item_once(shim, lpt, snake):
    rng = np.random.default_rng(lpt * 10 + snake)
    cases = [(1, 1), (1, 7), (8, 1), (8, 16), (128, 16), (5, 3), (15, 40), (21, 40), (3, 100), (16, 1), (24, 5), (7, 64), (9, 9)]
    cases += [(int(rng.integers(1, 70)), int(rng.integers(1, 50))) for _ in range(40)]
    for npairs, nunits in cases:
        total, got = items(shim, npairs, nunits, lpt, snake)
        assert len(got) == total, (npairs, nunits)
        assert sorted((b, u) for _, b, u in got) == [(b, u) for b in range(npairs) for u in range(nunits)], (npairs, nunits)


@pytest.mark.parametrize("lpt", [0, 1])
def test_a_pair_stays_on_one_xcd_when_the_pair_count_divides_by_eight(shim, lpt):
    for npairs, nunits in [(8, 16), (128, 16), (32, 5), (16, 33)]:
        _, got = items(shim, npairs, nunits, lpt, 32 if lpt else 0)
        xcd_of = {}
        for block, b, _ in got:
            assert xcd_of.setdefault(b, block % 8) == block % 8
        assert all(x == b % 8 for b, x in xcd_of.items())        # XCD x takes the pairs x, x + 8, ...


def test_longest_first_hands_out_units_in_ascending_order_per_xcd(shim):
    """With the flag, an XCD's workgroups (ascending index) take unit 0 of all its pairs, then unit 1, ...: the callers
    number a pair's units longest first."""
    for npairs, nunits in [(128, 16), (8, 4), (21, 40), (5, 3)]:
        _, got = items(shim, npairs, nunits, 1, 0)
        for x in range(8):
            units = [u for block, _, u in got if block % 8 == x]
            assert units == sorted(units), (npairs, nunits, x)


def test_round_reversal_pairs_long_with_short(shim):
    """Two rounds of 32 CUs on an XCD (config 2's key-split launch: 4 pairs of 16 units per XCD): CU c holds local items
    c and 32 + c, whose units must add up to the same length everywhere."""
    npairs, nunits = 32, 16
    _, got = items(shim, npairs, nunits, 1, 32)
    for x in range(8):
        local = {block // 8: u for block, _, u in got if block % 8 == x}
        sums = {local[c] + local[32 + c] for c in range(32)}
        assert sums == {nunits - 1}


@pytest.mark.parametrize("nsplit", [1, 2, 3, 5, 8])
def test_adjacent_shares_hand_out_every_item_and_share_once(shim, nsplit):
    """split_item_at: over the grid (x = items padded to a multiple of 8, y = shares) every (item, share) exactly once, an item
    on the XCD of its index, and in an XCD's dispatch sequence the shares of an item next to each other, items ascending."""
    shim.split_item_at.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_int)] * 2
    shim.split_item_at.restype = None
    blk, sp = C.c_int(), C.c_int()
    for gx in (8, 16, 64, 256, 520):
        got = []
        for by in range(nsplit):
            for bx in range(gx):
                shim.split_item_at(bx, by, gx, nsplit, C.byref(blk), C.byref(sp))
                got.append((by * gx + bx, blk.value, sp.value))
        assert sorted((b, s) for _, b, s in got) == [(b, s) for b in range(gx) for s in range(nsplit)], gx
        assert all(lin % 8 == b % 8 for lin, b, _ in got)
        for x in range(8):
            seq = [(b, s) for lin, b, s in got if lin % 8 == x]      # dispatch order on that XCD
            assert seq == sorted(seq), (gx, x)
