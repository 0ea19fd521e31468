"""The reference's shape-semantics fixtures (the 21 tests of its shape-only backend,
catgrad/src/interpreter/backend/shape_only.rs:325-534, transcribed as data in
golden/shape_cases.json) replayed on the oracle (CPU) and on the device: result shapes, dtype tags,
and a refusal wherever the reference panics."""
import json
import os

import numpy as np
import pytest

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "shape_cases.json")))["cases"]


def _operand(be, cg, shape, dtype="F32"):
    n = int(np.prod(shape)) if len(shape) else 1
    # all equal values: `compare` then depends on the shapes alone, as in the shape-only backend
    a = np.ones(n, np.float32 if dtype == "F32" else np.uint32)
    return be.ndarray_from_vec_f32(a, shape) if dtype == "F32" else be.ndarray_from_vec_u32(a, shape)


def _tag(cg, t):
    return "F32" if t.dtype == cg.F32 else "U32"


def run_case(be, cg, c):
    op = c["op"]
    if op == "zeros":
        for dt in c["dtypes"]:
            t = be.zeros(c["shape"], cg.F32 if dt == "F32" else cg.U32)
            assert list(t.shape) == c["expect_shape"] and _tag(cg, t) == dt
            assert not be.to_vec(t).any()
        return
    if op == "from_vec":
        for dt in c["dtypes"]:
            a = np.asarray(c["data"], np.float32 if dt == "F32" else np.uint32)
            t = be.ndarray_from_vec_f32(a, c["shape"]) if dt == "F32" else be.ndarray_from_vec_u32(a, c["shape"])
            assert list(t.shape) == c["expect_shape"] and _tag(cg, t) == dt
            assert np.array_equal(be.to_vec(t), a)
        return
    x = _operand(be, cg, c["x"])
    if op == "compare":
        assert be.compare(x, _operand(be, cg, c["y"])) is c["expect_bool"]
        return

    def call():
        if op in ("add", "mul", "matmul"):
            return getattr(be, op)(x, _operand(be, cg, c["y"]))
        if op == "broadcast":
            return be.broadcast(x, c["to"])
        if op == "reshape":
            return be.reshape(x, c["to"])
        if op in ("sum", "max", "neg"):
            return getattr(be, op)(x)
        if op == "cast":
            return be.cast(x, cg.U32 if c["to_dtype"] == "U32" else cg.F32)
        if op == "topk":
            return be.topk(x, c["k"])
        raise AssertionError(op)
    if "expect_panic" in c or "ndarray_panics" in c:
        with pytest.raises(cg.BackendPanic) as e:
            r = call()
            be.to_vec(r)
        if c.get("expect_panic") == "Shape mismatch":
            assert isinstance(e.value, cg.ShapeError)
        return
    r = call()
    outs = r if isinstance(r, tuple) else (r,)
    for i, t in enumerate(outs):
        assert list(t.shape) == c["expect_shape"], c["name"]
        be.to_vec(t)                                       # the value exists, not only its shape
    if "expect_dtype" in c:
        assert _tag(cg, outs[0]) == c["expect_dtype"]
    if "expect_dtypes" in c:
        assert [_tag(cg, t) for t in outs] == c["expect_dtypes"]


def test_the_fixture_holds_all_21_cases():
    assert len(CASES) == 21 and len({c["name"] for c in CASES}) == 21


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_shape_case_on_oracle(oracle, cg, case):
    run_case(oracle, cg, case)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["lazy", "eager", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_shape_case_on_device(hip, hip_eager, hip_bf16, cg, case, mode):
    run_case({"lazy": hip, "eager": hip_eager, "bf16": hip_bf16}[mode], cg, case)
