"""The C++ host layer (tensors, views, operators, reductions, autograd step) on the GPU against the oracle, and the
BASELINE configurations at their full sizes through size-independent properties."""
import numpy as np
import pytest

import golden_dsl
from oracle import cpu
from oracle.meta import Slice as OSlice, TensorError as OErr
from oracle.tensor import OTensor, train_step as oracle_train_step

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    from rtensors_amd import tensor
    return tensor


@pytest.fixture(scope="module")
def be(T):
    return T.Backend(0)


CASES = (golden_dsl.load("reference_vectors.json") + golden_dsl.load("reference_scalar_vectors.json") + golden_dsl.load("reference_view_vectors.json") + golden_dsl.load("reference_operand_vectors.json") + golden_dsl.load("reference_meta_vectors.json") +
         golden_dsl.load("reference_matmul_vectors.json"))


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_reference_vectors_through_host_layer(T, be, case):
    def slice_cls(start, end, step):
        return T.Slice(start, end, step)
    slice_cls.range = T.Slice.range
    slice_cls.range_inclusive = T.Slice.range_inclusive
    slice_cls.index = T.Slice.index
    env, err = golden_dsl.run_case(case, lambda dt, v, s: T.Tensor.from_buf(be, dt, v, s), slice_cls, T.TensorError)
    for exp in case["expect"]:
        exp.pop("path", None)

    def meta_of(t):
        i = t._info()
        return i["shape"], i["strides"], i["offset"], i["contiguous"]
    golden_dsl.check_case(case, env, err, lambda t: t.to_numpy(), lambda t, idx: t.get(idx), meta_of)


def rand_values(dtype, n, rng):
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    if npd.kind == "f":
        return rng.standard_normal(n).astype(npd)
    return rng.integers(-100, 100, size=n).astype(npd)


def test_random_programs_match_oracle(T, be):
    rng = np.random.default_rng(21)
    for trial in range(60):
        dtype = ["f32", "f64", "i32", "i64"][trial % 4]
        rank = int(rng.integers(1, 5))
        shape = [int(rng.integers(1, 9)) for _ in range(rank)]
        sb = [d if rng.random() < 0.6 else 1 for d in shape][int(rng.integers(0, rank)):]
        va, vb = rand_values(dtype, int(np.prod(shape)), rng), rand_values(dtype, int(np.prod(sb)), rng)
        o, g = OTensor.from_buf(dtype, va, shape), T.Tensor.from_buf(be, dtype, va, shape)
        ob, gb = OTensor.from_buf(dtype, vb, sb), T.Tensor.from_buf(be, dtype, vb, sb)
        ov, gv = o, g
        for _ in range(int(rng.integers(0, 3))):
            r = len(ov.meta.shape)
            d = int(rng.integers(0, r))
            k = int(rng.integers(0, 3))
            if k == 0 and ov.meta.strides[d] > 0 and ov.meta.shape[d] > 1:
                step = int(rng.choice([1, 2, -1]))
                ov, gv = ov.slice(d, OSlice(None, None, step)), gv.slice(d, T.Slice(None, None, step))
            elif k == 1 and r > 1:
                p = [int(v) for v in rng.permutation(r)]
                ov, gv = ov.permute(p), gv.permute(p)
            else:
                ov, gv = ov.unsqueeze_at(d), gv.unsqueeze_at(d)
        try:
            want = ((ov + ob) * 3 - ob).unary("relu")
        except OErr:
            continue
        got = ((gv + gb) * 3 - gb).unary("relu")
        assert got.shape == want.meta.shape
        assert got.to_numpy().tobytes() == want.to_numpy().tobytes(), (trial, dtype, ov.meta, sb)
        if ov.meta.shape == want.meta.shape and not (ov.meta.is_contiguous() and any(s < 0 for s in ov.meta.strides)):
            ov -= ob; gv -= gb
            ov.unary_inplace("abs"); gv.unary_inplace("abs")
            assert g.dump_buffer().tobytes() == o.buf.tobytes()
        if want.meta.rank() and dtype in ("i32", "i64"):
            for ax in range(want.meta.rank()):
                assert got.sum_at(ax).to_numpy().tobytes() == want.sum_at(ax).to_numpy().tobytes()
            assert got.max().to_numpy().tobytes() == want.max().to_numpy().tobytes()


def test_expressions_fuse_and_match_the_eager_operators(T, be):
    """`lazy(a) * 3 + b ...`: the recorded expression must give, bit for bit, what the same operators give when each runs as its own
    backend call (the oracle's OTensor), whether it is issued as fused launches (same-shape forward runs) or falls back to the
    operators (broadcast operands, stepped views, steps a chain does not have)."""
    rng = np.random.default_rng(77)
    for trial in range(48):
        dtype = ["f32", "f64", "i32", "i64", "u8", "i16"][trial % 6]
        flt = dtype[0] == "f"
        shape = [int(rng.integers(1, 20)) for _ in range(int(rng.integers(1, 4)))]
        n = int(np.prod(shape))
        mode = trial % 4                # 0, 1: same-shape operands; 2: b needs broadcasting; 3: a is a stepped view
        sb = shape if mode != 2 else ([1] * (len(shape) - 1) + [shape[-1]])
        va, vb, vc = rand_values(dtype, n, rng), rand_values(dtype, int(np.prod(sb)), rng), rand_values(dtype, n, rng)
        if dtype == "u8":
            va, vb, vc = np.abs(va).astype(np.uint8), np.abs(vb).astype(np.uint8), np.abs(vc).astype(np.uint8)
        oa, ob, oc = OTensor.from_buf(dtype, va, shape), OTensor.from_buf(dtype, vb, sb), OTensor.from_buf(dtype, vc, shape)
        ga, gb, gc = T.Tensor.from_buf(be, dtype, va, shape), T.Tensor.from_buf(be, dtype, vb, sb), T.Tensor.from_buf(be, dtype, vc, shape)
        if mode == 3 and shape[0] > 1:
            oa, ga = oa.slice(0, OSlice(None, None, 2)), ga.slice(0, T.Slice(None, None, 2))
            oc, gc = oc.slice(0, OSlice(None, None, 2)), gc.slice(0, T.Slice(None, None, 2))
            if mode != 2:
                ob, gb = ob.slice(0, OSlice(None, None, 2)), gb.slice(0, T.Slice(None, None, 2))
        # ((a * 3 + b).relu() - 1) * c - a, then |.|, then (floats) sqrt -- nine or ten steps: more than one launch when fused
        want = ((((oa * 3) + ob).unary("relu") - 1) * oc - oa).unary("abs")
        e = ((((T.lazy(ga) * 3) + gb).relu() - 1) * gc - ga).abs()
        want = want * 2 + oc
        e = e * 2 + gc
        want = (want - ob) if mode != 2 else want
        e = (e - gb) if mode != 2 else e
        if flt:
            want = want.unary("abs").unary("sqrt").unary("ln")           # `ln` is not available in a chain: the operator runs it
            e = e.abs().unary("sqrt").unary("ln")
        with np.errstate(all="ignore"):
            got = e.eval()
        assert got.shape == want.meta.shape
        g, w = got.to_numpy().reshape(-1), want.to_numpy().reshape(-1)
        if flt:
            ok = np.isclose(g.astype(np.float64), w.astype(np.float64), rtol=1e-5, atol=1e-5, equal_nan=True)       # through ln: the reference's 1e-5
            assert ok.all(), (trial, dtype, mode)
            # the exact part, without the logarithm, bit for bit
            e2 = (((((T.lazy(ga) * 3) + gb).relu() - 1) * gc - ga).abs() * 2 + gc)
            w2 = (((((oa * 3) + ob).unary("relu") - 1) * oc - oa).unary("abs") * 2 + oc)
            assert e2.eval().to_numpy().tobytes() == w2.to_numpy().tobytes(), (trial, dtype, mode)
            fused = e2.fused_launches
        else:
            assert g.tobytes() == w.tobytes(), (trial, dtype, mode)
            fused = e.fused_launches
        if mode in (0, 1):
            assert fused >= 1, (trial, dtype, "same-shape forward runs must take the fused path")
        if mode == 3 and shape[0] > 2 and len(shape) > 1:
            assert e.fused_launches is not None
    # an expression without steps is a copy; a single unfusable step is just the operator
    a = T.Tensor.from_buf(be, "f32", np.arange(6, dtype=np.float32), [2, 3])
    assert T.lazy(a).eval().to_numpy().tobytes() == a.to_numpy().tobytes()
    ev = T.lazy(a).unary("sin")
    assert np.allclose(ev.eval().to_numpy(), np.sin(np.arange(6, dtype=np.float32)).reshape(2, 3), rtol=1e-5, atol=1e-6) and ev.fused_launches == 0
    # an operand that is first named after a step the chain does not have: the steps before the logarithm are one launch (which must
    # not read b), the logarithm is the operator, the addition is a launch of its own
    b = T.Tensor.from_buf(be, "f32", np.arange(6, dtype=np.float32) * 0.25, [2, 3])
    ev = (T.lazy(a) + 1).unary("ln") + b
    want = np.log(np.arange(6, dtype=np.float32) + 1) + np.arange(6, dtype=np.float32) * 0.25
    assert np.allclose(ev.eval().to_numpy().reshape(-1), want, rtol=1e-5, atol=1e-6) and ev.fused_launches == 2


def test_reduce_of_noncontiguous_and_reversed_views(T, be):
    x = np.arange(24, dtype=np.float64) * 0.5 - 3
    o, g = OTensor.from_buf("f64", x, [2, 3, 4]), T.Tensor.from_buf(be, "f64", x, [2, 3, 4])
    assert np.array_equal(g.transpose().sum_at(0).to_numpy(), o.transpose().sum_at(0).to_numpy())
    assert np.array_equal(g.permute([1, 2, 0]).max_at(1).to_numpy(), o.permute([1, 2, 0]).max_at(1).to_numpy())
    # a reversed view is |stride|-contiguous; the reference then reduces from the wrong offset (Cpu: ignores it).  Here it
    # is gathered first, so the result is the reduction of the viewed values.
    rv = g.slice(0, T.Slice(None, None, -1))
    assert np.array_equal(rv.sum_at(2).to_numpy().reshape(2, 3), x.reshape(2, 3, 4)[::-1].sum(axis=2))


def test_statistic_and_index_reductions_through_host_layer(T, be):
    """var / pop_var / std / norm / logsumexp / argmax / argmin (ops/reduction/mod.rs:411-500): shapes of the outputs (kept dim, rank-0
    totals, u64 for the index kinds), views gathered first, and the reference's Cuda known answers."""
    import json, os
    cases = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_reduce_stat_vectors.json")))["cases"]
    for c in cases:
        x = np.array(c["data"], dtype=cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[c["dtype"]]])
        g, o = T.Tensor.from_buf(be, c["dtype"], x, c["shape"]), OTensor.from_buf(c["dtype"], x, c["shape"])
        got, want = g.reduce(c["op"], c["dim"]), o.reduce(c["op"], c["dim"])
        assert list(got.shape) == list(want.meta.shape) == ([] if c["dim"] is None else [1, 2])
        if c["op"] in cpu.ARG_OPS:
            assert got.dtype == cpu.U64 and got.to_numpy().reshape(-1).tolist() == c["want"]
        else:
            assert np.allclose(got.to_numpy().reshape(-1).astype(np.float64), c["want"], rtol=1e-6 if c["dtype"] == "f32" else 1e-14, atol=0)
    rng = np.random.default_rng(9)
    x = (rng.normal(size=(6, 5, 7)) * 2 + 4)
    g, o = T.Tensor.from_buf(be, "f64", x.reshape(-1), [6, 5, 7]), OTensor.from_buf("f64", x.reshape(-1), [6, 5, 7])
    gv, ov = g.permute([2, 0, 1]).slice(1, T.Slice(None, None, -2)), o.permute([2, 0, 1]).slice(1, OSlice(None, None, -2))
    for axis in (0, 1, 2):
        for name, args in (("var_at", ()), ("pop_var_at", ()), ("std_at", (True,)), ("std_at", (False,)), ("norm_at", ("L1",)), ("norm_at", ("L2",)),
                           ("logsumexp_at", ())):
            got, want = getattr(gv, name)(axis, *args), getattr(ov, name)(axis, *args)
            assert list(got.shape) == list(want.meta.shape)
            assert np.allclose(got.to_numpy(), want.to_numpy(), rtol=1e-12, atol=0), (name, axis)
        for name in ("argmax_at", "argmin_at"):
            got, want = getattr(gv, name)(axis), getattr(ov, name)(axis)
            assert np.array_equal(got.to_numpy(), want.to_numpy()), (name, axis)
    assert np.isclose(gv.var().to_numpy(), ov.var().to_numpy(), rtol=1e-12) and np.isclose(gv.std(False).to_numpy(), ov.std(False).to_numpy(), rtol=1e-12)
    assert np.isclose(gv.logsumexp().to_numpy(), ov.logsumexp().to_numpy(), rtol=1e-12) and np.isclose(gv.norm("L2").to_numpy(), ov.norm("L2").to_numpy(), rtol=1e-12)
    assert int(gv.argmax().to_numpy()) == int(ov.argmax().to_numpy()) and int(gv.argmin().to_numpy()) == int(ov.argmin().to_numpy())
    # closed form on the viewed values
    xv = x.transpose(2, 0, 1)[:, ::-2]
    assert np.allclose(gv.var_at(2).to_numpy().reshape(xv.shape[0], xv.shape[1]), xv.var(axis=2, ddof=1), rtol=1e-12)
    assert np.array_equal(gv.argmax_at(1).to_numpy().reshape(xv.shape[0], xv.shape[2]), xv.argmax(axis=1))


def test_constructors_and_into_dtype(T, be):
    """`scalar`, `column`, `row`, `max`, `min`, `zeros`, `ones` (core/primitives.rs:418-506; the reference's tests core/mod.rs:839-867 hold
    the shapes) and `into_dtype` (core/primitives.rs:527-539: whole buffer converted, meta kept, a partial view refused)."""
    col, row, sc = T.Tensor.column(be, "i32", [1, 2, 3]), T.Tensor.row(be, "i32", [1, 2, 3]), T.Tensor.scalar(be, "i32", 42)
    assert list(col.shape) == [3] and [col.get([i]) for i in range(3)] == [1, 2, 3]                       # core/mod.rs:839-845
    assert list(row.shape) == [1, 3] and [row.get([0, i]) for i in range(3)] == [1, 2, 3]                 # core/mod.rs:848-856
    assert list(sc.shape) == [] and sc.get([]) == 42                                                       # core/mod.rs:859-867
    for name in ("u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64"):
        info = np.iinfo(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[name]])
        assert T.Tensor.max_of(be, name, [2, 3]).to_numpy().reshape(-1).tolist() == [info.max] * 6
        assert T.Tensor.min_of(be, name, [5]).to_numpy().reshape(-1).tolist() == [info.min] * 5
    for name in ("f32", "f64"):
        info = np.finfo(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[name]])
        assert T.Tensor.max_of(be, name, [4]).to_numpy().tolist() == [info.max] * 4 and T.Tensor.min_of(be, name, [4]).to_numpy().tolist() == [info.min] * 4
    assert T.Tensor.max_of(be, "bool", [3]).to_numpy().astype(np.uint8).tolist() == [1, 1, 1]
    assert T.Tensor.zeros(be, "f64", [2, 2]).to_numpy().reshape(-1).tolist() == [0.0] * 4 and T.Tensor.ones(be, "u16", [3]).to_numpy().tolist() == [1, 1, 1]
    x = np.array([0.4, 0.5, 1.5, -0.5, -1.5, 300.7, -2.5, 1e10, -1e10, 7.0, np.nan, 2.5], dtype=np.float32)
    t = T.Tensor.from_buf(be, "f32", x, [3, 4])
    as_i32 = t.into_dtype("i32")
    assert as_i32.dtype == cpu.I32 and list(as_i32.shape) == [3, 4] and list(as_i32.strides) == [4, 1]
    assert as_i32.to_numpy().reshape(-1).tolist() == [0, 1, 2, -1, -2, 301, -3, 2 ** 31 - 1, -2 ** 31, 7, 0, 3]   # round half away from zero, saturate, NaN -> 0
    assert t.into_dtype("f64").to_numpy().reshape(-1).tobytes() == x.astype(np.float64).tobytes()
    tv = t.transpose()                                                  # a view of the whole buffer keeps its meta
    tvi = tv.into_dtype("i64")
    assert list(tvi.shape) == [4, 3] and list(tvi.strides) == [1, 4] and tvi.get([1, 2]) == 7
    with pytest.raises(T.TensorError) as e:                             # a view of part of the buffer: size != buffer length
        t.slice(0, T.Slice(0, 2, 1)).into_dtype("i32")
    assert e.value.kind == "SizeMismatch"


def test_view_as_and_reshape(T, be):
    """`view_as` (core/tensor.rs:328-355) and `reshape` (238-243) through the host layer: shared storage, the two error kinds, reshape of
    permuted views, and the one place where the host layer departs from the reference: a fully reversed view keeps its element order."""
    x = np.arange(24, dtype=np.int32)
    t = T.Tensor.from_buf(be, "i32", x, [2, 3, 4])
    v = t.view_as([6, 4])
    assert list(v.shape) == [6, 4] and list(v.strides) == [4, 1] and np.array_equal(v.to_numpy(), x.reshape(6, 4))
    v.set([5, 3], 99)                                                    # same storage
    assert t.get([1, 2, 3]) == 99
    v.set([5, 3], 23)
    row = t.slice(0, 1).slice(0, 2)                                      # contiguous run at an offset
    assert np.array_equal(row.view_as([2, 2]).to_numpy(), x.reshape(2, 3, 4)[1, 2].reshape(2, 2)) and row.view_as([2, 2]).offset == 20
    with pytest.raises(T.TensorError) as e:
        t.transpose().view_as([24])
    assert e.value.kind == "ContiguityError"
    with pytest.raises(T.TensorError) as e:
        t.view_as([5, 5])
    assert e.value.kind == "InvalidShape"
    r = t.transpose().reshape([6, 4])                                    # gathers first
    assert not r._info()["is_view"]
    assert np.array_equal(r.to_numpy(), x.reshape(2, 3, 4).transpose(2, 1, 0).reshape(6, 4)) and list(r.strides) == [4, 1]
    assert np.array_equal(t.reshape([4, 6]).to_numpy(), x.reshape(4, 6))
    flat = T.Tensor.from_buf(be, "i32", x, [24])
    rev = flat.slice(0, T.Slice(None, None, -1))                         # |stride| contiguous, offset 23
    rv = rev.view_as([4, 6])
    assert list(rv.strides) == [-6, -1] and rv.offset == 23 and np.array_equal(rv.to_numpy(), x[::-1].reshape(4, 6))
    assert np.array_equal(rev.reshape([2, 12]).to_numpy(), x[::-1].reshape(2, 12))
    half = t.slice(2, T.Slice(None, None, -1))                           # reversed along the last dim only
    with pytest.raises(T.TensorError) as e:
        half.view_as([24])
    assert e.value.kind == "ContiguityError"
    assert np.array_equal(half.reshape([24]).to_numpy(), x.reshape(2, 3, 4)[:, :, ::-1].reshape(24))


def test_out_of_scope_methods_report_unsupported(T, be):
    g = T.Tensor.from_buf(be, "i32", np.ones(4, np.int32), [4])
    with pytest.raises(T.TensorError) as e:
        g.var()                                               # WeightValue kinds on an integer tensor
    assert e.value.kind == "UnsupportedOperation"
    with pytest.raises(T.TensorError):
        g._new(T._h.rth_reduce, 11, T.C.c_int64(-1))          # not a reduction op code


# ---- autograd step (config 5 at reduced size) ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("mode", ["sum", "reference_literal"])
@pytest.mark.parametrize("seed_with_loss", [True, False])
def test_train_step_matches_oracle(T, be, dtype, mode, seed_with_loss):
    from rtensors_amd import datagen
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    n, d = 384, 96
    x = datagen.normal(npd, n * d, 4, 0)
    bias = datagen.normal(npd, d, 4, 1, 0.1)
    target = datagen.uniform(npd, n * d, 4, 2)
    ox, ob, ot = OTensor.from_buf(dtype, x, [n, d]), OTensor.from_buf(dtype, bias, [d]), OTensor.from_buf(dtype, target, [n, d])
    gx, gb, gt = T.Tensor.from_buf(be, dtype, x, [n, d]), T.Tensor.from_buf(be, dtype, bias, [d]), T.Tensor.from_buf(be, dtype, target, [n, d])
    oloss, ograd = oracle_train_step(ox, ob, ot, 0.01, mode, seed_with_loss)
    gloss, ggrad = T.train_step(gx, gb, gt, 0.01, mode, seed_with_loss)
    tol = (1e-5 if dtype == "f32" else 1e-12)
    # loss = mean |y - t|: a float reduction, within rel tol of sum|x|/N
    absdiff_sum = float(np.abs(np.maximum(x.reshape(n, d).astype(np.float64) + bias, 0) - target.reshape(n, d)).sum())
    assert abs(float(gloss.to_numpy()) - float(oloss.buf[0])) <= tol * absdiff_sum / (n * d) + 1e-30
    assert ggrad.shape == ograd.meta.shape == [d]
    # d(bias): elementwise maps are bit-exact; the column sum is a float reduction (tolerance relative to sum|g|)
    scale = abs(float(oloss.buf[0])) if seed_with_loss else 1.0
    gtol = tol * scale * n / (n * d) * 4 + 1e-30 if mode == "sum" else 1e-6 * scale
    assert np.max(np.abs(ggrad.to_numpy().astype(np.float64) - ograd.buf.astype(np.float64))) <= gtol
    assert np.max(np.abs(gb.to_numpy().astype(np.float64) - ob.buf.astype(np.float64))) <= 0.01 * gtol + np.finfo(npd).eps
    if mode == "sum" and not seed_with_loss:
        # closed form: d(bias)[j] = (1/N) * sum_i [x_ij + b_j > 0] * sign(y_ij - t_ij),  N = n*d
        pre = (x.reshape(n, d) + bias.astype(npd)).astype(npd)
        y = np.maximum(pre, 0)
        closed = ((pre > 0) * np.sign((y - target.reshape(n, d)).astype(npd))).astype(np.float64).sum(axis=0) / (n * d)
        assert np.max(np.abs(ggrad.to_numpy() - closed)) < 1e-6
    if mode == "reference_literal":
        # the literal engine keeps row 0 of the upstream gradient instead of the batch sum
        ob2 = OTensor.from_buf(dtype, bias, [d])
        _, gsum = oracle_train_step(OTensor.from_buf(dtype, x, [n, d]), ob2, OTensor.from_buf(dtype, target, [n, d]), 0.01, "sum", seed_with_loss)
        assert not np.allclose(gsum.buf, ograd.buf)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("seed_with_loss", [True, False])
def test_fused_train_step_matches_oracle(T, be, dtype, seed_with_loss):
    """The three fused passes against the oracle's literal sequence: y and the L1 gradient map bit for bit (through the C ABI), the
    loss and d(bias) within the reduction tolerance, the updated bias as the tape leaves it; and the host layer's fused step against
    its own tape."""
    from rtensors_amd import datagen, hip as H
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    tol = 1e-5 if dtype == "f32" else 1e-12
    for n, d in ((384, 96), (1000, 260), (7, 4), (5, 6), (4100, 4096)):
        x = datagen.normal(npd, n * d, 4, 0)
        bias = datagen.normal(npd, d, 4, 1, 0.1)
        target = datagen.uniform(npd, n * d, 4, 2)
        x[::97] = 0; bias[::5] = 0; target[::89] = 0                     # ties: pre == 0, y == t
        ox, ob, ot = OTensor.from_buf(dtype, x, [n, d]), OTensor.from_buf(dtype, bias, [d]), OTensor.from_buf(dtype, target, [n, d])
        # element-wise pieces of the literal sequence, op by op, on the oracle
        oy = (ox + ob).unary("relu")
        odiff = oy - ot
        ogmap = odiff.unary("sign") / float(np.float32(n * d))
        absdiff = np.abs(odiff.buf.astype(np.float64))
        fits = d % (4 if dtype == "f32" else 2) == 0
        # the same through the C ABI
        hip = H.Hip.new(0) if fits else None
        if not fits:
            terms = None
        if fits:
            code = H.DTYPE_BY_NAME[dtype]
            hx, hb, ht = hip.alloc_from_slice(code, x), hip.alloc_from_slice(code, bias), hip.alloc_from_slice(code, target)
            hy, hg, hl, hd = hip.alloc(code, n * d), hip.alloc(code, n * d), hip.alloc(code, 1), hip.alloc(code, d)
            hip.fused_bias_relu(hx, hb, hy, n, d)
            hip.fused_l1_forward(hy, ht, hg, hl, n * d)
            assert hip.dump(hy).tobytes() == oy.buf.tobytes(), (dtype, n, d, "y")
            assert hip.dump(hg).tobytes() == ogmap.buf.tobytes(), (dtype, n, d, "gmap")
            loss = hip.dump(hl)[0]
            assert abs(float(loss) - absdiff.sum() / float(np.float32(n * d))) <= tol * absdiff.sum() / (n * d) + 1e-300
            up = hl if seed_with_loss else hip.alloc_from_slice(code, np.ones(1, npd))
            hip.fused_l1_relu_backward(hg, hy, up, hd, n, d)
            upv = loss if seed_with_loss else npd.type(1)
            terms = ((oy.buf > 0).astype(npd) * (ogmap.buf * upv).astype(npd)).astype(npd).reshape(n, d).astype(np.float64)
            assert np.all(np.abs(hip.dump(hd).astype(np.float64) - terms.sum(axis=0)) <= tol * np.abs(terms).sum(axis=0) + 1e-300), (dtype, n, d)
            # the two-pass form: the same y bit for bit, the same loss and d(bias) within the tolerance of a sum, no gradient map stored
            hy2, hl2, hd2 = hip.alloc(code, n * d), hip.alloc(code, 1), hip.alloc(code, d)
            hip.fused_bias_relu_l1(hx, hb, ht, hy2, hl2, n, d)
            assert hip.dump(hy2).tobytes() == oy.buf.tobytes(), (dtype, n, d, "y, two passes")
            loss2 = hip.dump(hl2)[0]
            assert abs(float(loss2) - absdiff.sum() / float(np.float32(n * d))) <= tol * absdiff.sum() / (n * d) + 1e-300
            up2 = hl2 if seed_with_loss else up
            hip.fused_l1_relu_backward_t(hy2, ht, up2, hd2, n, d)
            upv2 = loss2 if seed_with_loss else npd.type(1)
            terms2 = ((oy.buf > 0).astype(npd) * (ogmap.buf * upv2).astype(npd)).astype(npd).reshape(n, d).astype(np.float64)
            assert np.all(np.abs(hip.dump(hd2).astype(np.float64) - terms2.sum(axis=0)) <= tol * np.abs(terms2).sum(axis=0) + 1e-300), (dtype, n, d)
            hip.close()
        # host layer: fused step against the tape and the oracle's step
        gx, gt = T.Tensor.from_buf(be, dtype, x, [n, d]), T.Tensor.from_buf(be, dtype, target, [n, d])
        gb3, gb2 = T.Tensor.from_buf(be, dtype, bias, [d]), T.Tensor.from_buf(be, dtype, bias, [d])
        tloss, tgrad = T.train_step(gx, gb2, gt, 0.01, "sum", seed_with_loss)
        floss3, fgrad3, used3 = T.train_step_fused(gx, gb3, gt, 0.01, seed_with_loss, passes=3)
        gb1 = T.Tensor.from_buf(be, dtype, bias, [d])
        floss, fgrad, used = T.train_step_fused(gx, gb1, gt, 0.01, seed_with_loss)          # two passes (the default)
        assert used3 == fits
        assert abs(float(floss3.to_numpy()) - float(floss.to_numpy())) <= 2 * tol * absdiff.sum() / (n * d) + 1e-300
        assert used == fits
        assert abs(float(floss.to_numpy()) - absdiff.sum() / float(np.float32(n * d))) <= tol * absdiff.sum() / (n * d) + 1e-300
        assert fgrad.shape == [d]
        if terms is None:
            upv = npd.type(floss.to_numpy()) if seed_with_loss else npd.type(1)
            terms = ((oy.buf > 0).astype(npd) * (ogmap.buf * upv).astype(npd)).astype(npd).reshape(n, d).astype(np.float64)
        gtol = 2 * tol * np.abs(terms).sum(axis=0) + 1e-300
        assert np.all(np.abs(fgrad.to_numpy().astype(np.float64) - tgrad.to_numpy().astype(np.float64)) <= gtol)
        assert np.all(np.abs(fgrad3.to_numpy().astype(np.float64) - tgrad.to_numpy().astype(np.float64)) <= gtol)
        assert np.max(np.abs(gb1.to_numpy().astype(np.float64) - gb2.to_numpy().astype(np.float64))) <= 0.01 * gtol.max() + np.finfo(npd).eps
        assert np.max(np.abs(gb3.to_numpy().astype(np.float64) - gb2.to_numpy().astype(np.float64))) <= 0.01 * gtol.max() + np.finfo(npd).eps
        if n * d <= 300000:
            # the oracle's whole step (its loss is a sequential f32 sum, which is itself only good to about 1e-7 * n: small shapes only)
            oloss, ograd = oracle_train_step(ox, ob, ot, 0.01, "sum", seed_with_loss)
            assert abs(float(floss.to_numpy()) - float(oloss.buf[0])) <= tol * absdiff.sum() / (n * d) + 1e-300
            assert ograd.meta.shape == [d]
            assert np.all(np.abs(fgrad.to_numpy().astype(np.float64) - ograd.buf.astype(np.float64)) <= gtol)
            assert np.max(np.abs(gb1.to_numpy().astype(np.float64) - ob.buf.astype(np.float64))) <= 0.01 * gtol.max() + np.finfo(npd).eps


def test_fused_passes_refuse_what_they_do_not_take(be):
    from rtensors_amd import hip as H
    hip = H.Hip.new(0)
    a, b, c = hip.alloc(H.F32, 4 * 6), hip.alloc(H.F32, 6), hip.alloc(H.F32, 4 * 6)
    with pytest.raises(H.TensorError) as e:
        hip.fused_bias_relu(a, b, c, 4, 6)                                # rows of 6 f32 are not whole vectors
    assert e.value.status == 1
    with pytest.raises(H.TensorError) as e:
        hip.fused_bias_relu(a, b, c, 5, 8)                                # more than the buffers hold
    assert e.value.kind == "IdxOutOfBounds"
    i = hip.alloc(H.I32, 16)
    with pytest.raises(H.TensorError) as e:
        hip.fused_bias_relu(i, i, i, 2, 8)
    assert e.value.kind == "UnsupportedOperation"
    # outputs that overlap an input: in place on the very same run is fine, anything else is refused
    x = hip.alloc_from_slice(H.F32, np.arange(-16, 16, dtype=np.float32))
    bias = hip.alloc_from_slice(H.F32, np.ones(8, np.float32))
    hip.fused_bias_relu(x, bias, x, 4, 8)
    assert np.array_equal(hip.dump(x), np.maximum(np.arange(-16, 16, dtype=np.float32) + 1, 0))
    shifted = H.HipBuf(None, x.ptr + 16, 24, H.F32)                        # a window into x, not owned
    with pytest.raises(H.TensorError) as e:
        hip.fused_bias_relu(x, bias, shifted, 2, 8)
    assert e.value.status == 1 and "overlaps" in str(e.value)
    loss = hip.alloc(H.F32, 1)
    with pytest.raises(H.TensorError):
        hip.fused_l1_forward(x, c, shifted, loss, 24)
    with pytest.raises(H.TensorError):
        hip.fused_l1_relu_backward(x, x, loss, H.HipBuf(None, x.ptr, 8, H.F32), 4, 8)
    hip.close()


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("seed_with_loss", [True, False])
def test_linear_step_matches_oracle(T, be, dtype, seed_with_loss):
    """y = x @ w, mean L1 loss, backward through the MatMul node (d(w) = x^T @ upstream), SGD on w."""
    from rtensors_amd import datagen
    from oracle.tensor import linear_step as oracle_linear_step
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    n, d, h = 200, 48, 24
    x = datagen.normal(npd, n * d, 5, 0)
    w = datagen.normal(npd, d * h, 5, 1, 0.2)
    target = datagen.uniform(npd, n * h, 5, 2)
    ox, ow, ot = OTensor.from_buf(dtype, x, [n, d]), OTensor.from_buf(dtype, w, [d, h]), OTensor.from_buf(dtype, target, [n, h])
    gx, gw, gt = T.Tensor.from_buf(be, dtype, x, [n, d]), T.Tensor.from_buf(be, dtype, w, [d, h]), T.Tensor.from_buf(be, dtype, target, [n, h])
    oloss, ograd = oracle_linear_step(ox, ow, ot, 0.01, seed_with_loss)
    gloss, ggrad = T.linear_step(gx, gw, gt, 0.01, seed_with_loss)
    tol = 1e-5 if dtype == "f32" else 1e-12
    X, W, Tg = x.reshape(n, d).astype(np.float64), w.reshape(d, h).astype(np.float64), target.reshape(n, h).astype(np.float64)
    Y = X @ W
    assert abs(float(gloss.to_numpy()) - float(oloss.buf[0])) <= 50 * tol * (np.abs(X) @ np.abs(W) + np.abs(Tg)).sum() / (n * h)
    assert ggrad.shape == ograd.meta.shape == [d, h]
    scale = abs(float(oloss.buf[0])) if seed_with_loss else 1.0
    bound = 50 * tol * scale * np.abs(X).sum(axis=0)[:, None] / (n * h) + 1e-30
    # sign(y - t) can flip where a float matmul result lands on the other side of the target: compare away from such ties
    stable = np.abs(Y - Tg) > 1e-3
    if stable.all():
        assert (np.abs(ggrad.to_numpy().astype(np.float64) - ograd.buf.reshape(d, h).astype(np.float64)) <= bound).all()
    closed = scale * (X.T @ np.sign(Y - Tg)) / (n * h)
    assert np.max(np.abs(ggrad.to_numpy().astype(np.float64) - closed)) <= 1e-4 * scale * (1.0 + (~stable).sum())
    assert np.max(np.abs(gw.to_numpy().astype(np.float64) - (W - 0.01 * closed))) <= 1e-5 * (1.0 + (~stable).sum())


# ---- BASELINE configurations at full size ---------------------------------------------------------------------------------------
def test_config1_full_vs_oracle(be, T):
    from rtensors_amd import datagen
    n = 4096
    for dtype in ("f32", "i32"):
        if dtype == "f32":
            a, b = datagen.uniform(np.float32, n, 0, 0), datagen.uniform(np.float32, n, 0, 1)
        else:
            a, b = datagen.integers(n, 0, 2, -1000, 1000), datagen.integers(n, 0, 3, -1000, 1000)
        oc = OTensor.from_buf(dtype, a, [1, n]) + OTensor.from_buf(dtype, b, [n, 1])
        gc = T.Tensor.from_buf(be, dtype, a, [1, n]) + T.Tensor.from_buf(be, dtype, b, [n, 1])
        assert gc.shape == [n, n] and gc.to_numpy().tobytes() == oc.buf.tobytes()
        os_, gs = oc.sum_at(1), gc.sum_at(1)
        assert gs.shape == [n, 1]
        if dtype == "i32":
            assert gs.to_numpy().tobytes() == os_.buf.tobytes()
            assert np.array_equal(gs.to_numpy().reshape(-1).astype(np.int64), a.astype(np.int64).sum() + n * b.astype(np.int64))   # closed form
        else:
            tol = 1e-5 * np.abs(oc.buf.astype(np.float64)).reshape(n, n).sum(axis=1)
            assert np.all(np.abs(gs.to_numpy().reshape(-1).astype(np.float64) - os_.buf.astype(np.float64)) <= tol)


def test_config2_chain_full_size(be, T):
    """c = relu(a * 3 + b); c -= 1 at 2^28 f32 (2^27 f64, 2^28 i32): a strided sample of the result is compared with the
    same chain in numpy (each step is one IEEE / wrapping operation, so the comparison is bit-exact)."""
    from rtensors_amd import datagen
    for dtype, n in (("f32", 1 << 28), ("f64", 1 << 27), ("i32", 1 << 28)):
        npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
        chunk = 1 << 22
        def gen(stream, start, m):
            if dtype == "i32":
                return datagen.integers(m, 1, stream, -(1 << 20), 1 << 20, start)
            return datagen.normal(npd, m, 1, stream, 1.0, start)
        # only the sampled windows are generated on the host; the device tensors come from the device generator
        from rtensors_amd import hip as H
        hb = H.Hip.new(0)
        code = H.DTYPE_BY_NAME[dtype]
        da, db = hb.alloc_uninit(code, n), hb.alloc_uninit(code, n)
        if dtype == "i32":
            datagen.fill_device(da, "int", 1, 0, -(1 << 20), 1 << 20); datagen.fill_device(db, "int", 1, 1, -(1 << 20), 1 << 20)
        else:
            datagen.fill_device(da, "normal", 1, 0); datagen.fill_device(db, "normal", 1, 1)
        three, one = (3, 1) if dtype == "i32" else (3.0, 1.0)
        t = hb.copy(da)                                   # `a * 3.0` = owned() + in-place mul
        hb.scalar_contiguous("mul", t, three, 0, n)
        u = hb.alloc_uninit(code, n)
        m = (0, [n], [1])
        hb.broadcast((t, m), (db, m), (u, m), "add")
        c = hb.copy(u)                                    # `.relu()` = owned() + in-place relu
        hb.unary_contiguous("relu", c, 0, n)
        hb.scalar_contiguous("sub", c, one, 0, n)
        for start in (0, 12345 * 4, n // 2 + 3, n - chunk):
            tmp = hb.alloc_uninit(code, chunk)
            hb.copy_range_within(tmp, c, 0, start, chunk)
            got = hb.dump(tmp)
            ha, hbv = gen(0, start, chunk), gen(1, start, chunk)
            with np.errstate(over="ignore"):
                want = (np.maximum((ha * npd.type(three)).astype(npd) + hbv, 0).astype(npd) - npd.type(one)).astype(npd)
            assert got.tobytes() == want.tobytes(), (dtype, start)
        del da, db, t, u, c
        hb.sync()
    # the same expression through the host layer's lazy form: one fused launch, the same bits as the operators one by one
    rng = np.random.default_rng(2)
    n = (1 << 24) + 3
    for dtype in ("f32", "f64", "i32"):
        va, vb = rand_values(dtype, n, rng), rand_values(dtype, n, rng)
        a, b = T.Tensor.from_buf(be, dtype, va, [n]), T.Tensor.from_buf(be, dtype, vb, [n])
        eager = ((a * 3.0) + b).relu()
        eager -= 1.0
        e = ((T.lazy(a) * 3.0) + b).relu() - 1.0
        fusedv = e.eval()
        assert e.fused_launches == 1
        assert fusedv.equals(eager)
        npd = va.dtype
        want = (np.maximum((va * npd.type(3)).astype(npd) + vb, 0).astype(npd) - npd.type(1)).astype(npd)
        assert fusedv.to_numpy().tobytes() == want.tobytes()


def test_config3_both_variants_agree_and_match_formula(be, T):
    """z = x + y -> (16,64,512,1024) with x contiguous, and with x given as the permuted / reversed / unsqueezed view of a
    (16,1024,512) tensor holding the same values: both must produce the same 2 GiB, checked on sampled rows against
    numpy, and checked equal to each other in full on the device."""
    from rtensors_amd import datagen, hip as H
    hb = H.Hip.new(0)
    B, J, K, L = 16, 64, 512, 1024
    x = datagen.normal(np.float32, B * K * L, 2, 0).reshape(B, K, L)
    y = datagen.uniform(np.float32, J * L, 2, 1).reshape(J, L)
    gx = hb.alloc_from_slice(H.F32, x.reshape(-1))
    gy = hb.alloc_from_slice(H.F32, y.reshape(-1))
    shape = [B, J, K, L]
    zs = [J * K * L, K * L, L, 1]
    z1 = hb.alloc_uninit(H.F32, B * J * K * L)
    hb.broadcast((gx, (0, shape, [K * L, 0, L, 1])), (gy, (0, shape, [0, L, 0, 1])), (z1, (0, shape, zs)), "add")
    # variant b: base[b, l, K-1-k] = x[b, k, l]; view = base.permute([0,2,1]).slice(1, step -1).unsqueeze_at(1)
    base = np.ascontiguousarray(np.transpose(x, (0, 2, 1))[:, :, ::-1])
    gbase = hb.alloc_from_slice(H.F32, base.reshape(-1))
    from oracle.meta import MetaTensor                                # metadata only: derive the view's layout with the oracle rules
    mv = OTensor(cpu.F32, np.zeros(1, np.float32), MetaTensor.row_major([B, L, K])).permute([0, 2, 1]).slice(1, OSlice(None, None, -1)).unsqueeze_at(1)
    assert mv.meta.shape == [B, 1, K, L] and mv.meta.strides == [K * L, -K, -1, K] and mv.meta.offset == K - 1
    z2 = hb.alloc_uninit(H.F32, B * J * K * L)
    hb.broadcast((gbase, (mv.meta.offset, shape, [K * L, 0, -1, K])), (gy, (0, shape, [0, L, 0, 1])), (z2, (0, shape, zs)), "add")
    assert z1 == z2                                                   # device-side equality over all 2^29 elements
    # each result on its own against the formula: whole (b, j) slabs of K rows -- 12 slabs = 6144 rows per variant, drawn
    # separately for the two, every b and both ends of j among them -- and 64 single rows anywhere
    rng = np.random.default_rng(0)
    slab = hb.alloc_uninit(H.F32, K * L)
    for name, z in (("contiguous x", z1), ("permuted x", z2)):
        pairs = {(0, 0), (B - 1, J - 1), (0, J - 1), (B - 1, 0)}
        while len(pairs) < 12:
            pairs.add((int(rng.integers(0, B)), int(rng.integers(0, J))))
        for b, j in sorted(pairs):
            hb.copy_range_within(slab, z, 0, (b * J + j) * K * L, K * L)
            assert hb.dump(slab).tobytes() == (x[b] + y[j][None, :]).tobytes(), (name, b, j)
        row = hb.alloc_uninit(H.F32, L)
        for _ in range(64):
            b, j, k = int(rng.integers(0, B)), int(rng.integers(0, J)), int(rng.integers(0, K))
            hb.copy_range_within(row, z, 0, ((b * J + j) * K + k) * L, L)
            assert hb.dump(row).tobytes() == (x[b, k] + y[j]).tobytes(), (name, b, j, k)
    # a checksum over everything: sum over (j, k) of z[b, j, k, :] = J * sum_k x[b, k, :] + K * sum_j y[j, :], evaluated by the
    # device's own axis reductions on the 2 GiB result and compared with float64 on the host within the reduction tolerance
    for z in (z1, z2):
        part = hb.alloc(H.F32, B * J * L)
        hb.apply_reduce_contiguous_nd((z, (0, [B * J, K, L], [K * L, L, 1])), part, 1, "sum")
        tot = hb.alloc(H.F32, B * L)
        hb.apply_reduce_contiguous_nd((part, (0, [B, J, L], [J * L, L, 1])), tot, 1, "sum")
        want = J * x.astype(np.float64).sum(axis=1) + K * y.astype(np.float64).sum(axis=0)[None, :]
        bound = 2e-5 * (J * np.abs(x.astype(np.float64)).sum(axis=1) + K * np.abs(y.astype(np.float64)).sum(axis=0)[None, :])
        assert np.all(np.abs(hb.dump(tot).reshape(B, L).astype(np.float64) - want) <= bound)
    hb.sync()


def test_config4_full_size_reductions(be, T):
    from rtensors_amd import datagen, hip as H
    hb = H.Hip.new(0)
    R, Cc = 8192, 32768
    t = hb.alloc_uninit(H.F32, R * Cc)
    datagen.fill_device(t, "normal", 3, 0)
    host = hb.dump(t).reshape(R, Cc)
    h64 = host.astype(np.float64)
    meta = (0, [R, Cc], [Cc, 1])
    def run(op, dim, n_out):
        out = hb.alloc(H.F32, n_out)
        hb.apply_reduce_contiguous_nd((t, meta), out, dim, op)
        return hb.dump(out)
    rows_abs = np.abs(h64).sum(axis=1); cols_abs = np.abs(h64).sum(axis=0)
    assert np.all(np.abs(run("sum", 1, R) - h64.sum(axis=1)) <= 1e-5 * rows_abs)
    assert np.all(np.abs(run("mean", 1, R) - h64.mean(axis=1)) <= 1e-5 * rows_abs / Cc + 1e-12)
    assert run("max", 1, R).tobytes() == host.max(axis=1).tobytes()
    assert np.all(np.abs(run("sum", 0, Cc) - h64.sum(axis=0)) <= 1e-5 * cols_abs)
    out = hb.alloc(H.F32, 1)
    hb.apply_reduce_contiguous_flat(t, out, 0, R * Cc, "sum")
    assert abs(float(hb.dump(out)[0]) - h64.sum()) <= 1e-5 * np.abs(h64).sum()
    # a checksum of checksums: summing the row sums equals summing the column sums equals the full sum, within tolerance
    assert abs(run("sum", 1, R).astype(np.float64).sum() - run("sum", 0, Cc).astype(np.float64).sum()) <= 2e-5 * np.abs(h64).sum()
    del host, h64
    ti = hb.alloc_uninit(H.I32, R * Cc)
    datagen.fill_device(ti, "int", 3, 1, -1000, 1000)
    hi = hb.dump(ti).reshape(R, Cc)
    def runi(op, dim, n_out):
        out = hb.alloc(H.I32, n_out)
        hb.apply_reduce_contiguous_nd((ti, meta), out, dim, op)
        return hb.dump(out)
    assert np.array_equal(runi("sum", 1, R), hi.sum(axis=1, dtype=np.int64).astype(np.int32))
    assert np.array_equal(runi("sum", 0, Cc), hi.sum(axis=0, dtype=np.int64).astype(np.int32))
    assert np.array_equal(runi("max", 1, R), hi.max(axis=1)) and np.array_equal(runi("min", 0, Cc), hi.min(axis=0))
    assert np.array_equal(runi("min", 1, R), hi.min(axis=1)) and np.array_equal(runi("max", 0, Cc), hi.max(axis=0))
    hb.sync()


def test_config5_full_size_step(be, T):
    """x (65536,4096), bias (4096,), target (65536,4096), lr 0.01: d(bias) against the closed form evaluated in numpy."""
    from rtensors_amd import datagen
    n, d = 65536, 4096
    x = datagen.normal(np.float32, n * d, 4, 0)
    bias = datagen.normal(np.float32, d, 4, 1, 0.1)
    target = datagen.uniform(np.float32, n * d, 4, 2)
    gx, gb, gt = T.Tensor.from_buf(be, "f32", x, [n, d]), T.Tensor.from_buf(be, "f32", bias, [d]), T.Tensor.from_buf(be, "f32", target, [n, d])
    gb_fused = T.Tensor.from_buf(be, "f32", bias, [d])
    gloss, ggrad = T.train_step(gx, gb, gt, 0.01, "sum", True)
    floss, fgrad, used = T.train_step_fused(gx, gb_fused, gt, 0.01, True)
    assert used
    gb_fused3 = T.Tensor.from_buf(be, "f32", bias, [d])
    floss3, fgrad3, used3 = T.train_step_fused(gx, gb_fused3, gt, 0.01, True, passes=3)
    assert used3
    pre = x.reshape(n, d) + bias
    y = np.maximum(pre, 0)
    diff = y - target.reshape(n, d)
    loss = np.abs(diff.astype(np.float64)).mean()
    got_loss = float(gloss.to_numpy())
    assert abs(got_loss - loss) <= 1e-5 * loss
    N = np.float32(np.float32(n * d))
    gm = (np.sign(diff) / N).astype(np.float32)                       # sign(sign(d)) / N
    up = (gm * np.float32(got_loss)).astype(np.float32) * (pre > 0)   # L1 backward seeded with the loss, then ReLU backward
    closed = up.astype(np.float64).sum(axis=0)
    tol = 1e-5 * np.abs(up.astype(np.float64)).sum(axis=0) + 1e-30
    g = ggrad.to_numpy().astype(np.float64)
    assert np.all(np.abs(g - closed) <= tol)
    new_bias = gb.to_numpy()
    want_bias = bias - (ggrad.to_numpy() * np.float32(0.01)).astype(np.float32)
    assert new_bias.tobytes() == want_bias.astype(np.float32).tobytes()
    # the fused passes: the same loss and gradient within the same bounds, the same update rule
    assert abs(float(floss.to_numpy()) - loss) <= 1e-5 * loss
    up_f = (gm * np.float32(float(floss.to_numpy()))).astype(np.float32) * (pre > 0)
    assert np.all(np.abs(fgrad.to_numpy().astype(np.float64) - up_f.astype(np.float64).sum(axis=0)) <= 1e-5 * np.abs(up_f.astype(np.float64)).sum(axis=0) + 1e-30)
    want_fused = bias - (fgrad.to_numpy() * np.float32(0.01)).astype(np.float32)
    assert gb_fused.to_numpy().tobytes() == want_fused.astype(np.float32).tobytes()
    assert abs(float(floss3.to_numpy()) - loss) <= 1e-5 * loss
    up_3 = (gm * np.float32(float(floss3.to_numpy()))).astype(np.float32) * (pre > 0)
    assert np.all(np.abs(fgrad3.to_numpy().astype(np.float64) - up_3.astype(np.float64).sum(axis=0)) <= 1e-5 * np.abs(up_3.astype(np.float64)).sum(axis=0) + 1e-30)
    want_fused3 = bias - (fgrad3.to_numpy() * np.float32(0.01)).astype(np.float32)
    assert gb_fused3.to_numpy().tobytes() == want_fused3.astype(np.float32).tobytes()
