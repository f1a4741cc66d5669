#!/usr/bin/env python3
"""Writes reference_test_vectors.json: the inputs and expected outputs the reference's own operator tests
assert (test/test_opr.cpp), restated from their closed forms.  The reference holds no fixture files; its
tests build inputs and expectations from these formulas (N = 3 ranks, fp32) and compare with 4-ulp
tolerance (test/test_base.h:59) - every value here is a small integer, so the comparison is exact.

Nothing of the reference is run or imported: the formulas are re-derived below, each with the lines of
test/test_opr.cpp it restates.  Run from the repository root:  python tests/golden/make_reference_vectors.py
"""
import json
import os

N = 3


def all_reduce(op):
    # test/test_opr.cpp:286-359: in[i][j] = (i+1)(j+1), len = 10; SUM -> 6(j+1) (:321-330), MAX -> 3(j+1),
    # MIN -> (j+1) (:334-358); every rank expects the same
    length = 10
    ins = [[(i + 1) * (j + 1) for j in range(length)] for i in range(N)]
    factor = {"SUM": 6, "MAX": 3, "MIN": 1}[op]
    out = [factor * (j + 1) for j in range(length)]
    return {"collective": "all_reduce", "op": op, "len": length, "inputs": ins, "expected": [out] * N,
            "cites": "test/test_opr.cpp:286-359"}


def reduce_scatter(op):
    # test/test_opr.cpp:361-438: in[i][m] = (i+1)(m+1) for m < N*recvlen, recvlen = 10;
    # rank k expects factor * (k*recvlen + j + 1)
    recvlen = 10
    ins = [[(i + 1) * (m + 1) for m in range(N * recvlen)] for i in range(N)]
    factor = {"SUM": 6, "MAX": 3, "MIN": 1}[op]
    outs = [[factor * (k * recvlen + j + 1) for j in range(recvlen)] for k in range(N)]
    return {"collective": "reduce_scatter", "op": op, "len": recvlen, "inputs": ins, "expected": outs,
            "cites": "test/test_opr.cpp:361-438"}


def all_gather():
    # test/test_opr.cpp:243-284: in[i][j] = (i+1)(j+1), sendlen = 10; out[k][i*sendlen + j] = in[i][j] for every k
    sendlen = 10
    ins = [[(i + 1) * (j + 1) for j in range(sendlen)] for i in range(N)]
    out = [v for row in ins for v in row]
    return {"collective": "all_gather", "len": sendlen, "inputs": ins, "expected": [out] * N,
            "cites": "test/test_opr.cpp:243-284"}


def all_to_all():
    # test/test_opr.cpp:198-241: in[i][j*len + k] = (i+1)(j+2)(k+3), len = 6; out[j][i*len + k] = in[i][j*len + k]
    length = 6
    ins = [[(i + 1) * (j + 2) * (k + 3) for j in range(N) for k in range(length)] for i in range(N)]
    outs = [[(i + 1) * (j + 2) * (k + 3) for i in range(N) for k in range(length)] for j in range(N)]
    return {"collective": "all_to_all", "len": length, "inputs": ins, "expected": outs,
            "cites": "test/test_opr.cpp:198-241"}


def scatter():
    # test/test_opr.cpp:101-146: root 1 holds (i+1)(j+2) for block i, recvlen = 10; rank i receives block i
    length, root = 10, 1
    root_in = [(i + 1) * (j + 2) for i in range(N) for j in range(length)]
    outs = [[(i + 1) * (j + 2) for j in range(length)] for i in range(N)]
    return {"collective": "scatter", "len": length, "root": root, "inputs": [root_in if r == root else None for r in range(N)],
            "expected": outs, "cites": "test/test_opr.cpp:101-146"}


def gather():
    # test/test_opr.cpp:148-196: the inverse; only the root has an expectation
    length, root = 10, 1
    ins = [[(i + 1) * (j + 2) for j in range(length)] for i in range(N)]
    out = [(i + 1) * (j + 2) for i in range(N) for j in range(length)]
    return {"collective": "gather", "len": length, "root": root, "inputs": ins,
            "expected": [out if r == root else None for r in range(N)], "cites": "test/test_opr.cpp:148-196"}


def broadcast():
    # test/test_opr.cpp:440-480: root 1's (i+1)(j+1) row arrives on every rank
    length, root = 10, 1
    ins = [[(i + 1) * (j + 1) for j in range(length)] for i in range(N)]
    return {"collective": "broadcast", "len": length, "root": root, "inputs": ins, "expected": [ins[root]] * N,
            "cites": "test/test_opr.cpp:440-480"}


def reduce(op):
    # test/test_opr.cpp:482-551: in[i][j] = (i+1)(j+1), root 1 expects 6(j+1) / 3(j+1) / (j+1)
    length, root = 10, 1
    ins = [[(i + 1) * (j + 1) for j in range(length)] for i in range(N)]
    factor = {"SUM": 6, "MAX": 3, "MIN": 1}[op]
    out = [factor * (j + 1) for j in range(length)]
    return {"collective": "reduce", "op": op, "len": length, "root": root, "inputs": ins,
            "expected": [out if r == root else None for r in range(N)], "cites": "test/test_opr.cpp:482-551"}


def main():
    cases = [all_reduce(op) for op in ("SUM", "MAX", "MIN")]
    cases += [reduce_scatter(op) for op in ("SUM", "MAX", "MIN")]
    cases += [all_gather(), all_to_all(), scatter(), gather(), broadcast()]
    cases += [reduce(op) for op in ("SUM", "MAX", "MIN")]
    doc = {"dtype": "FLOAT32", "nranks": N, "tolerance_ulps_in_reference": 4, "cases": cases}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_test_vectors.json")
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    print(path, len(cases), "cases")


if __name__ == "__main__":
    main()
