"""Checks of gemmBroadcast / getGemmType that do not restate the reference's code, shared by the tests of the oracle
(tests/test_oracle.py) and of the product's C ABI and C++ layer (tests/test_abi.py, tests/test_cpp_ops.py).

Two independent sources:
  * tests/golden/shape_logic_cases.json: cases traced by hand through utils.cpp:293-396, at least one per branch,
    including the shapes of the reference's own unit tests;
  * the meaning of a matrix product: for every operand pair that torch.matmul accepts and whose batch dims are all 1,
    the class must be the one read off the real product [m,k] x [k,n] (a vector has exactly one dim other than 1),
    each operand keeps its element count, and the padded shapes are [1,1,m,k] and [1,1,k,n] - except where the source
    says otherwise, and each exception is stated below with the lines it comes from.

An implementation is handed in as (broadcast, gemm_type):
  broadcast(s1, s2) -> (status, o1, o2) with status in {"ok", "short", "abort", "out_of_range"}
  gemm_type(o1, o2) -> one of "VV", "MV", "VM", "MM"
"""
import itertools
import json
import os

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "shape_logic_cases.json")

# GEMM_TYPE of the reference, runtime/include/executor/utils/utils.h:30-36: UNKNOW, VV, MV, VM, MM.
TYPE_NAMES = {1: "VV", 2: "MV", 3: "VM", 4: "MM"}


def hand_traced_cases():
    return json.load(open(GOLDEN))["cases"]


def check_hand_traced(broadcast, gemm_type, undefined_may_refuse=False):
    """Every case of the table.  `undefined_may_refuse`: where the reference reads out of range, the product only has
    to stay in bounds (any status); the oracle has to report exactly that."""
    seen_lines = set()
    for c in hand_traced_cases():
        status, o1, o2 = broadcast(c["s1"], c["s2"])
        tag = (c["s1"], c["s2"], c["lines"])
        if c["status"] == "out_of_range":
            assert undefined_may_refuse or status == "out_of_range", tag
            continue
        assert status == c["status"], (tag, status)
        if c["status"] == "abort":
            continue
        assert (list(o1), list(o2)) == (c["o1"], c["o2"]), (tag, o1, o2)
        if c["status"] == "ok":
            assert gemm_type(o1, o2) == c["type"], tag
        seen_lines.add(c["lines"].split()[0])
    return len(seen_lines)


def _matrix_view(s1, s2):
    """[m, k] x [k2, n] of the real product (torch.matmul: a rank-1 first operand is a row, a rank-1 second a column)."""
    m, k = (1, s1[0]) if len(s1) == 1 else (s1[-2], s1[-1])
    k2, n = (s2[0], 1) if len(s2) == 1 else (s2[-2], s2[-1])
    return m, k, k2, n


def _class_of_product(m, k, n):
    a = (m != 1) + (k != 1)
    b = (k != 1) + (n != 1)
    return {(1, 1): "VV", (1, 2): "VM", (2, 1): "MV"}.get((a, b), "MM")


def _numel(s):
    r = 1
    for d in s:
        r *= d
    return r


def check_matmul_semantics(broadcast, gemm_type, dims=(1, 2, 3, 5)):
    """All rank-1..4 pairs over `dims` with batch dims 1 that torch.matmul accepts."""
    import torch

    def shapes():
        for r in range(1, 5):
            for s in itertools.product(dims, repeat=r):
                if all(d == 1 for d in s[:-2]):
                    yield list(s)

    n_checked = n_padded_as_product = 0
    exceptions = {"rank1_rank1": 0, "rank1_leading_match": 0, "square_behind_rank4_row": 0, "short": 0, "undefined": 0}
    for s1 in shapes():
        for s2 in shapes():
            m, k, k2, n = _matrix_view(s1, s2)
            if k != k2:
                continue
            # the real product exists and has the expected number of elements
            assert _numel(torch.matmul(torch.zeros(s1), torch.zeros(s2)).shape) == m * n
            status, o1, o2 = broadcast(s1, s2)
            r1, r2 = len(s1), len(s2)
            if (r1, r2) == (1, 3):
                # utils.cpp:320-330 inserts two ones and does not recurse: rank 1 + 2 = 3, getGemmType is undefined
                assert status in ("short", "out_of_range"), (s1, s2)
                exceptions["short"] += 1
                continue
            if (r1, r2) == (1, 4):
                assert status == "abort", (s1, s2)  # utils.cpp:331-333
                continue
            if (r1, r2) == (3, 1):
                # utils.cpp:344-345 reads shape1[3] of a rank-3 shape
                exceptions["undefined"] += 1
                continue
            assert status == "ok", (s1, s2, status)
            assert len(o1) == 4 and len(o2) == 4
            # each operand keeps its elements (the gap-3 branch, utils.cpp:356-366, copies shape1's batch dims into
            # shape2, which changes nothing here because they are 1)
            assert _numel(o1) == _numel(s1) and _numel(o2) == _numel(s2), (s1, s2, o1, o2)
            got = gemm_type(o1, o2)
            want = _class_of_product(m, k, n)
            n_checked += 1
            if r1 == 4 and r2 == 2 and s2[0] == s2[1] and s1[3] == s2[1] and s2[0] != 1:
                # utils.cpp:345-346 then 353-354: shape1[3] == shape2[1] appends a one to a SQUARE weight, and
                # shape1[0] = 1 != shape2[0] puts the second one in front: [1,K,K,1], batch dim K, hence MM.
                assert (o1, o2, got) == (s1, [1, s2[0], s2[1], 1], "MM"), (s1, s2, o1, o2, got)
                exceptions["square_behind_rank4_row"] += 1
                continue
            assert got == want, (s1, s2, o1, o2, got, want)
            if r1 == 1 and r2 == 1:
                # utils.cpp:299-310: both vectors become rows [1,1,1,K]
                assert (o1, o2) == ([1, 1, 1, k], [1, 1, 1, k])
                exceptions["rank1_rank1"] += k != 1
                continue
            if r1 == 1 and r2 == 2:
                # utils.cpp:314-315: shape1[0] == shape2[0] always holds for a valid product, so the one goes BEHIND
                # the vector's length: a column [1,1,K,1] in front of [1,1,K,N]
                assert (o1, o2) == ([1, 1, k, 1], [1, 1, k, n])
                exceptions["rank1_leading_match"] += k != 1
                continue
            assert (o1, o2) == ([1, 1, m, k], [1, 1, k, n]), (s1, s2, o1, o2)
            n_padded_as_product += 1
    return n_checked, n_padded_as_product, exceptions
