"""Runs the golden known-answer cases (tests/golden/backend_kats.json) on any backend."""
import json
import os

import numpy as np

from catgrad_amd import _abi as A

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "backend_kats.json")) as f:
    KATS = json.load(f)

NP = {"f32": np.float32, "u32": np.uint32}
DT = {"f32": A.F32, "u32": A.U32}


def make(be, spec):
    arr = np.array(spec["data"], dtype=NP[spec["dtype"]]).reshape(spec["shape"])
    return be.from_numpy(arr)


def apply(be, case):
    op, args = case["op"], case.get("args", {})
    xs = [make(be, s) for s in case["inputs"]]
    if op == "zeros":
        return [be.zeros(args["shape"], DT[args["dtype"]])]
    if op in ("reshape", "broadcast"):
        return [getattr(be, op)(xs[0], args["shape"])]
    if op == "cast":
        return [be.cast(xs[0], DT[args["dtype"]])]
    if op == "topk":
        return list(be.topk(xs[0], args["k"]))
    return [getattr(be, op)(*xs)]


def check_case(be, case):
    outs = apply(be, case)
    assert len(outs) == len(case["expect"])
    for got, exp in zip(outs, case["expect"]):
        assert got.dtype == DT[exp["dtype"]], case["name"]
        assert list(got.shape) == exp["shape"], case["name"]
        g = be.to_numpy(got)
        e = np.array(exp["data"], dtype=np.float64).reshape(exp["shape"])
        if exp["dtype"] == "u32" or ("rtol" not in case and "atol" not in case):
            np.testing.assert_array_equal(g.astype(np.float64), e.astype(NP[exp["dtype"]]).astype(np.float64), err_msg=case["name"])
        else:
            np.testing.assert_allclose(g, e, rtol=case.get("rtol", 0), atol=case.get("atol", 0), err_msg=case["name"])
