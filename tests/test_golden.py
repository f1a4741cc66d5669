"""The committed fixture tests/golden/reference_test_vectors.json - the inputs and expectations of the
reference's own operator tests (test/test_opr.cpp), written by tests/golden/make_reference_vectors.py -
against the CPU oracle (no GPU) and against the HIP path through the C ABI (GPU)."""
import json
import os

import numpy as np
import pytest

import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_test_vectors.json")) as f:
    FIXTURE = json.load(f)
CASES = FIXTURE["cases"]
OPS = {"SUM": orc.SUM, "MAX": orc.MAX, "MIN": orc.MIN}


def arr(values):
    return None if values is None else np.array(values, dtype=np.float32)


def case_id(case):
    return case["collective"] + ("_" + case["op"] if "op" in case else "")


def check(outs, case, what):
    for r, want in enumerate(case["expected"]):
        if want is not None:
            assert np.array_equal(np.asarray(outs[r]), arr(want)), f"{what} {case_id(case)} rank {r} ({case['cites']})"


def test_fixture_is_what_the_generator_writes(tmp_path):
    import runpy
    mod = runpy.run_path(os.path.join(HERE, "golden", "make_reference_vectors.py"))
    fresh = [mod["all_reduce"](op) for op in ("SUM", "MAX", "MIN")] + [mod["reduce_scatter"](op) for op in ("SUM", "MAX", "MIN")]
    fresh += [mod["all_gather"](), mod["all_to_all"](), mod["scatter"](), mod["gather"](), mod["broadcast"]()]
    fresh += [mod["reduce"](op) for op in ("SUM", "MAX", "MIN")]
    assert json.loads(json.dumps(fresh)) == CASES
    assert FIXTURE["nranks"] == 3 and FIXTURE["dtype"] == "FLOAT32"


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_oracle_reproduces_the_reference_vectors(case):
    ins = [arr(x) for x in case["inputs"]]
    kind, dt = case["collective"], orc.FLOAT32
    if kind == "all_reduce":
        op = OPS[case["op"]]
        for outs in (orc.ucx_all_reduce(ins, dt, op), orc.shm_all_reduce(ins, dt, op), orc.test_all_reduce_f32(ins, op),
                     orc.fold_all_reduce(ins, dt, op, orc.ORDER_UCX), orc.fold_all_reduce(ins, dt, op, orc.ORDER_SHM),
                     orc.fold_all_reduce(ins, dt, op, orc.ORDER_RANK0)):
            check(outs, case, "oracle")
    elif kind == "reduce_scatter":
        op = OPS[case["op"]]
        for outs in (orc.ucx_reduce_scatter(ins, dt, op), orc.shm_reduce_scatter(ins, dt, op),
                     orc.test_reduce_scatter_f32(ins, op), orc.fold_reduce_scatter(ins, dt, op, orc.ORDER_UCX),
                     orc.fold_reduce_scatter(ins, dt, op, orc.ORDER_SHM)):
            check(outs, case, "oracle")
    elif kind == "all_gather":
        check(orc.ucx_all_gather(ins, dt), case, "oracle ucx")
        check(orc.shm_all_gather(ins, dt), case, "oracle shm")
    elif kind == "all_to_all":
        check(orc.ucx_all_to_all(ins, dt), case, "oracle ucx")
        check(orc.shm_all_to_all(ins, dt), case, "oracle shm")
    elif kind == "scatter":
        check(orc.ucx_scatter(ins, dt, case["root"]), case, "oracle")
    elif kind == "gather":
        check(orc.ucx_gather(ins, dt, case["root"]), case, "oracle")
    elif kind == "broadcast":
        check(orc.ucx_broadcast(ins, dt, case["root"]), case, "oracle")
    else:
        check(orc.ucx_reduce(ins, dt, OPS[case["op"]], case["root"]), case, "oracle")


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_hip_path_reproduces_the_reference_vectors(case):
    torch = pytest.importorskip("torch")
    import megray_amd as mr
    from gpu_util import empty_device, to_device, to_host

    n, length, kind = FIXTURE["nranks"], case["len"], case["collective"]
    ins = [arr(x) for x in case["inputs"]]
    d_in = [None if x is None else to_device(x) for x in ins]
    dt = mr.DType.FLOAT32
    root = case.get("root", 0)
    op = OPS.get(case.get("op", "SUM"))

    def host(views):
        torch.cuda.synchronize()
        return [None if v is None else to_host(v, np.float32) for v in views]

    if kind == "all_reduce":
        for order in (mr.FoldOrder.UCX, mr.FoldOrder.SHM, mr.FoldOrder.RANK0):
            for sched in (mr.Schedule.FUSED, mr.Schedule.TWO_PHASE):
                d_out = [empty_device(length * 4) for _ in range(n)]
                mr.all_reduce(d_in, d_out, length, dt, op, order, sched)
                check(host(d_out), case, f"hip order={order} sched={sched}")
    elif kind == "reduce_scatter":
        for order in (mr.FoldOrder.UCX, mr.FoldOrder.SHM):
            d_out = [empty_device(length * 4) for _ in range(n)]
            mr.reduce_scatter(d_in, d_out, length, dt, op, order)
            check(host(d_out), case, f"hip order={order}")
    elif kind == "all_gather":
        d_out = [empty_device(n * length * 4) for _ in range(n)]
        mr.all_gather(d_in, d_out, length, dt)
        check(host(d_out), case, "hip")
    elif kind == "all_to_all":
        d_out = [empty_device(n * length * 4) for _ in range(n)]
        mr.all_to_all(d_in, d_out, length, dt)
        check(host(d_out), case, "hip")
    elif kind == "scatter":
        d_out = [empty_device(length * 4) for _ in range(n)]
        mr.scatter(d_in[root], d_out, length, dt, root)
        check(host(d_out), case, "hip")
    elif kind == "gather":
        d_root = empty_device(n * length * 4)
        mr.gather(d_in, d_root, length, dt, root)
        check(host([d_root if r == root else None for r in range(n)]), case, "hip")
    elif kind == "broadcast":
        d_out = [empty_device(length * 4) for _ in range(n)]
        mr.broadcast(d_in[root], d_out, length, dt, root)
        check(host(d_out), case, "hip")
    else:
        d_root = empty_device(length * 4)
        mr.reduce_to_root(d_in, d_root, length, dt, op, root)
        check(host([d_root if r == root else None for r in range(n)]), case, "hip")
