"""The oracle's statistics and index reductions (variance / stdev / logsumexp / norms / argmax / argmin): checked against the known
answers the reference's Cuda tests hold (tests/golden/reference_reduce_stat_vectors.json) and against what the mathematics fixes
(float64 numpy: var with ddof, logaddexp.reduce, vector norms, first-occurrence argmax; hand-made tie / NaN / infinity cases)."""
import json
import os

import numpy as np
import pytest

from oracle import cpu
from oracle.meta import MetaTensor, TensorError

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "reference_reduce_stat_vectors.json")))["cases"]


def row_major(shape):
    strides, acc = [], 1
    for s in reversed(shape):
        strides.append(acc); acc *= s
    return list(reversed(strides))


def run(dtype, op, data, shape, dim, offset=0):
    code = cpu.DTYPE_BY_NAME[dtype]
    buf = np.ascontiguousarray(data, dtype=cpu.NP_DTYPE[code]).reshape(-1)
    meta = MetaTensor(list(shape), row_major(shape), offset)
    if op in cpu.ARG_OPS:
        return cpu.argmax(code, op, buf, meta, dim)
    return cpu.reduce_stat(code, op, buf, meta, dim)


@pytest.mark.parametrize("case", CASES, ids=[f"{c['op']}-{c['dim']}-{c['dtype']}" for c in CASES])
def test_reference_known_answers(case):
    got = run(case["dtype"], case["op"], case["data"], case["shape"], case["dim"])
    if case["op"] in cpu.ARG_OPS:
        assert got.tolist() == case["want"]
    else:
        rel = 1e-6 if case["dtype"] == "f32" else 1e-14        # the Cuda tests assert equality; a tree order may differ in the last bits
        assert np.allclose(got.astype(np.float64), case["want"], rtol=rel, atol=0)


def closed_form(op, x, axis):
    x = x.astype(np.float64)
    if op == "var": return x.var(axis=axis, ddof=1)
    if op == "pop_var": return x.var(axis=axis, ddof=0)
    if op == "std": return x.std(axis=axis, ddof=1)
    if op == "pop_std": return x.std(axis=axis, ddof=0)
    if op == "logsumexp": return np.logaddexp.reduce(x, axis=axis)
    if op == "l1_norm": return np.abs(x).sum(axis=axis)
    if op == "l2_norm": return np.sqrt((x * x).sum(axis=axis))
    raise AssertionError(op)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_against_float64_closed_forms(dtype):
    rng = np.random.default_rng(5)
    rel = 2e-5 if dtype == "f32" else 1e-12
    for shape, dim in (((7, 33, 5), 1), ((50, 3), 0), ((4, 1000), 1), ((1, 1, 9), 2), ((6, 2, 2), 0)):
        x = (rng.normal(size=shape) * 3 + 10).astype(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]])       # mean well away from 0
        for op in cpu.STAT_OPS:
            want = closed_form(op, x, dim).reshape(-1)
            got = run(dtype, op, x, shape, dim).astype(np.float64)
            assert np.allclose(got, want, rtol=rel, atol=0), (op, shape, dim)
            want_all = closed_form(op, x.reshape(-1), 0)
            got_all = run(dtype, op, x, shape, None).astype(np.float64)
            assert np.allclose(got_all, want_all, rtol=rel, atol=0), (op, shape, "total")
        for op, f in (("argmax", np.argmax), ("argmin", np.argmin)):
            assert run(dtype, op, x, shape, dim).tolist() == f(x, axis=dim).reshape(-1).tolist()
            assert run(dtype, op, x, shape, None).tolist() == [int(f(x))]


def test_offset_is_honoured_and_non_contiguous_is_refused():
    x = np.arange(30, dtype=np.float64)
    got = run("f64", "var", x, (2, 5), 1, offset=7)                         # rows 7..11 and 12..16
    assert np.allclose(got, [2.5, 2.5])
    assert run("f64", "argmax", x, (2, 5), 1, offset=7).tolist() == [4, 4]
    with pytest.raises(TensorError):
        cpu.reduce_stat(cpu.F64, "var", x, MetaTensor([5, 2], [1, 5], 0), 0)


def test_ties_nan_infinities_and_degenerate_counts():
    nan, inf = float("nan"), float("inf")
    # the first extremum wins; NaN never wins; nothing beats the starting value -> 0
    assert run("f64", "argmax", [1, 5, 5, 2], (4,), None).tolist() == [1]
    assert run("f64", "argmin", [3, 1, 1, 2], (4,), None).tolist() == [1]
    assert run("f64", "argmax", [nan, 2, nan, 7, 7], (5,), None).tolist() == [3]
    assert run("f64", "argmax", [nan, nan], (2,), None).tolist() == [0]
    assert run("f64", "argmax", [-inf, -inf], (2,), None).tolist() == [0]    # -inf does not beat lowest() either
    assert run("f32", "argmin", [inf, 4, -inf, -inf], (4,), None).tolist() == [2]
    assert run("i32", "argmax", [3, -7, 9, 9, 0], (5,), None).tolist() == [2]
    assert run("u8", "argmin", [3, 0, 9, 0], (4,), None).tolist() == [1]
    # logsumexp: infinities follow the limits, NaN propagates, an empty run is log(0)
    assert run("f64", "logsumexp", [-inf, -inf], (2,), None).tolist() == [-inf]
    assert run("f64", "logsumexp", [1.0, inf, 2.0], (3,), None).tolist() == [inf]
    assert np.isnan(run("f64", "logsumexp", [1.0, nan], (2,), None)[0])
    assert run("f64", "logsumexp", [], (0,), None).tolist() == [-inf]
    assert np.isclose(run("f64", "logsumexp", [1000.0, 1000.0], (2,), None)[0], 1000.0 + np.log(2.0), rtol=1e-15)   # no overflow
    assert np.isclose(run("f64", "logsumexp", [-1000.0, -1001.0], (2,), None)[0], -1000.0 + np.log1p(np.exp(-1.0)), rtol=1e-15)
    # one sample: population variance 0, sample variance 0 / 0
    assert run("f64", "pop_var", [4.0], (1,), None).tolist() == [0.0]
    assert np.isnan(run("f64", "var", [4.0], (1,), None)[0])
    # a large common offset does not cancel (this is what Welford's update is for): var of 1e9 + {0, 1, 2}
    assert np.isclose(run("f64", "var", [1e9, 1e9 + 1, 1e9 + 2], (3,), None)[0], 1.0, rtol=1e-12)
    # kinds the reference bounds on float types
    with pytest.raises(TensorError):
        run("i32", "var", [1, 2, 3], (3,), None)
    with pytest.raises(TensorError):
        run("bool", "argmax", [True, False], (2,), None)
