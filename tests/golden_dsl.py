"""Interpreter for the small program format of tests/golden/*.json.

A case is `inputs` (named row-major tensors), a `program` (one step per line: [result, op, operands...]) and
`expect` entries.  The same case runs against any tensor implementation that offers the reference's surface
(from_buf, slice, view_as, reshape, permute, transpose, unsqueeze_at, squeeze, + - * /, in-place forms, unary, reductions, matmul);
`factory(dtype_name, values, shape)` creates an owned tensor, `TensorError` is that implementation's error type.
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)["cases"]


def _slice(spec, SliceCls):
    if "slice" in spec:
        s, e, st = spec["slice"]
        return SliceCls(s, e, st)
    if "range" in spec:
        return SliceCls.range(*spec["range"])
    if "range_inclusive" in spec:
        return SliceCls.range_inclusive(*spec["range_inclusive"])
    if "index" in spec:
        return SliceCls.index(spec["index"])
    raise KeyError(spec)


def run_case(case, factory, SliceCls, ErrorCls):
    """Returns (env, error_kind).  `env` maps names to tensors; error_kind is None unless a step raised ErrorCls."""
    env = {}
    paths = {}
    for name, t in case["inputs"].items():
        env[name] = factory(case["dtype"], t["values"], t["shape"])
    try:
        for step in case["program"]:
            dst, op, *args = step
            if op == "slice":
                env[dst] = env[args[0]].slice(args[1], _slice(args[2], SliceCls))
            elif op == "permute":
                env[dst] = env[args[0]].permute(args[1])
            elif op == "transpose":
                env[dst] = env[args[0]].transpose()
            elif op == "unsqueeze":
                env[dst] = env[args[0]].unsqueeze_at(args[1])
            elif op == "view_as":
                env[dst] = env[args[0]].view_as(args[1])
            elif op == "reshape":
                env[dst] = env[args[0]].reshape(args[1])
            elif op == "squeeze":
                env[dst] = env[args[0]].squeeze() if len(args) == 1 else env[args[0]].squeeze_at(args[1])
            elif op in ("add", "sub", "mul", "div"):
                a, b = env[args[0]], env[args[1]]
                env[dst] = {"add": a.__add__, "sub": a.__sub__, "mul": a.__mul__, "div": a.__truediv__}[op](b)
            elif op in ("iadd", "isub", "imul", "idiv"):
                a, b = env[args[0]], env[args[1]]
                env[dst] = {"iadd": a.__iadd__, "isub": a.__isub__, "imul": a.__imul__, "idiv": a.__itruediv__}[op](b)
            elif op in ("add_scalar", "sub_scalar", "mul_scalar", "div_scalar"):
                a = env[args[0]]
                env[dst] = {"add_scalar": a.__add__, "sub_scalar": a.__sub__, "mul_scalar": a.__mul__,
                            "div_scalar": a.__truediv__}[op](args[1])
            elif op in ("iadd_scalar", "isub_scalar", "imul_scalar", "idiv_scalar"):            # `view += 5` and friends
                a = env[args[0]]
                env[dst] = {"iadd_scalar": a.__iadd__, "isub_scalar": a.__isub__, "imul_scalar": a.__imul__,
                            "idiv_scalar": a.__itruediv__}[op](args[1])
            elif op == "fill":                                                                   # view.fill(value)
                env[args[0]].fill(args[1])
                env[dst] = env[args[0]]
            elif op == "owned":
                env[dst] = env[args[0]].owned()
            elif op == "set":                                                                    # view.set(coord, value)
                env[args[0]].set(args[1], args[2])
                env[dst] = env[args[0]]
            elif op == "unary":
                env[dst] = env[args[0]].unary(args[1])
            elif op == "unary_inplace":
                env[dst] = env[args[0]].unary_inplace(args[1])
                paths[dst] = getattr(env[dst], "last_path", None)
            elif op == "scalar_inplace":
                env[dst] = env[args[0]].scalar_op_inplace(args[1], args[2])
            elif op in ("matmul", "dot", "outer"):
                env[dst] = getattr(env[args[0]], op)(env[args[1]])
            elif op in ("sum", "mean", "max", "min", "prod"):
                env[dst] = env[args[0]].reduce(op, args[1])
            else:
                raise KeyError(op)
    except ErrorCls as e:
        return env, getattr(e, "kind", type(e).__name__)
    return env, None


def check_case(case, env, err, to_numpy, get, meta_of):
    """Asserts every `expect` entry.  `to_numpy(t)` -> row-major ndarray, `get(t, idx)`, `meta_of(t)` -> (shape, strides, offset, contiguous)."""
    for exp in case["expect"]:
        if "error" in exp:
            assert err == exp["error"], f"{case['name']}: expected error {exp['error']}, got {err}"
            continue
        assert err is None, f"{case['name']}: unexpected error {err}"
        t = env[exp["t"]]
        shape, strides, offset, contiguous = meta_of(t)
        if "shape" in exp:
            assert list(shape) == exp["shape"], f"{case['name']}: shape {shape} != {exp['shape']}"
        if "strides" in exp:
            assert list(strides) == exp["strides"], f"{case['name']}: strides {strides} != {exp['strides']}"
        if "offset" in exp:
            assert offset == exp["offset"], f"{case['name']}: offset {offset} != {exp['offset']}"
        if "contiguous" in exp:
            assert contiguous == exp["contiguous"], f"{case['name']}: contiguity"
        if "path" in exp:
            assert getattr(t, "last_path", None) == exp["path"], f"{case['name']}: dispatched to {getattr(t, 'last_path', None)}"
        if "values" in exp:
            got = to_numpy(t).reshape(-1)
            want = np.array(exp["values"], dtype=got.dtype)
            if "tol" in exp:
                assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= exp["tol"]), f"{case['name']}: {got} vs {want}"
            else:
                assert got.tobytes() == want.tobytes() or np.array_equal(got, want), f"{case['name']}: {got} vs {want}"
        for idx, val in exp.get("get", []):
            assert get(t, idx) == val, f"{case['name']}: get{idx} = {get(t, idx)} != {val}"
