"""Pins the CPU oracle against an independent evaluation: numpy's own strided-view machinery
(np.lib.stride_tricks.as_strided) and numpy's elementwise / sequential-accumulate routines.  A wrong sign, index,
stride or a transposed operand in the oracle fails here."""
import zlib
import numpy as np
import pytest
from numpy.lib.stride_tricks import as_strided

from oracle import cpu
from oracle.meta import MetaTensor, Slice, compute_broadcasted_params
from oracle.tensor import OTensor

RNG = np.random.default_rng(1234)


def np_view(buf, meta):
    """The elements `meta` addresses inside `buf`, as a numpy strided view."""
    item = buf.dtype.itemsize
    base = buf[meta.offset:] if meta.offset < buf.size else buf[:0]
    # as_strided with negative strides needs a base pointer at the offset element
    return as_strided(buf[meta.offset:meta.offset + 1] if buf.size else base, shape=meta.shape,
                      strides=[s * item for s in meta.strides], writeable=False)


def random_view(t: OTensor, rng):
    """Random chain of slices / permutes on `t` (owned, rank >= 1)."""
    v = t.view()
    for _ in range(rng.integers(1, 4)):
        r = v.meta.rank()
        if r == 0:
            break
        k = rng.integers(0, 3)
        d = int(rng.integers(0, r))
        n = v.meta.shape[d]
        if k == 0 and v.meta.strides[d] > 0:     # (chained slicing of an already reversed dim follows a reference quirk; kept out of the numpy comparison)
            step = int(rng.choice([1, 2, 3, -1, -2]))
            if step > 0:
                a = int(rng.integers(0, n)); b = int(rng.integers(a + 1, n + 1))
                v = v.slice(d, Slice(a, b, step))
            else:
                a = int(rng.integers(0, n)); b = int(rng.integers(-1, a))
                v = v.slice(d, Slice(a, None if b < 0 else b, step))
        elif k == 1 and r > 1:
            v = v.permute(list(rng.permutation(r)))
        elif k == 2:
            v = v.unsqueeze_at(d)
    return v


DTYPES = ["f32", "f64", "i32", "i64", "u8", "i16", "u32"]


def rand_values(dtype, n, rng):
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    if npd.kind == "f":
        return rng.standard_normal(n).astype(npd)
    info = np.iinfo(npd)
    return rng.integers(max(info.min, -1000), min(info.max, 1000), size=n, dtype=np.int64).astype(npd)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", ["add", "sub", "mul"])
def test_broadcast_vs_numpy(dtype, op, oracle_lib):
    rng = np.random.default_rng(zlib.crc32((dtype + op).encode()))
    for trial in range(40):
        rank = int(rng.integers(1, 5))
        full = [int(rng.integers(1, 6)) for _ in range(rank)]
        sa = [d if rng.random() < 0.7 else 1 for d in full]
        sb = [d if rng.random() < 0.7 else 1 for d in full]
        sb = sb[int(rng.integers(0, rank)):] if rng.random() < 0.3 else sb
        a = OTensor.from_buf(dtype, rand_values(dtype, int(np.prod(sa)), rng), sa)
        b = OTensor.from_buf(dtype, rand_values(dtype, int(np.prod(sb)), rng), sb)
        va = a.slice(0, Slice(None, None, -1)) if (sa[0] > 1 and rng.random() < 0.5) else a
        vb = b.transpose() if rng.random() < 0.3 and len(sb) == len(sa) and sb == sb[::-1] else b
        got = getattr(va, {"add": "__add__", "sub": "__sub__", "mul": "__mul__"}[op])(vb)
        na, nb = np_view(a.buf, va.meta), np_view(b.buf, vb.meta)
        with np.errstate(over="ignore"):
            want = {"add": np.add, "sub": np.subtract, "mul": np.multiply}[op](na, nb)
        assert got.meta.shape == list(want.shape)
        assert got.to_numpy().tobytes() == np.ascontiguousarray(want).tobytes(), (dtype, op, sa, sb)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_broadcast_div_vs_numpy(dtype, oracle_lib):
    rng = np.random.default_rng(7)
    a = OTensor.from_buf(dtype, rand_values(dtype, 60, rng), [3, 4, 5])
    b = OTensor.from_buf(dtype, rand_values(dtype, 5, rng), [5])
    got = (a.permute([1, 0, 2]) / b).to_numpy()
    want = np_view(a.buf, a.permute([1, 0, 2]).meta) / b.buf
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()


def test_integer_division_truncates_and_faults(oracle_lib):
    a = OTensor.from_buf("i32", [7, -7, 7, -7], [4])
    b = OTensor.from_buf("i32", [2, 2, -2, -2], [4])
    assert (a / b).buf.tolist() == [3, -3, -3, 3]          # Rust `/` truncates toward zero
    from oracle.meta import TensorError
    with pytest.raises(TensorError):
        a / OTensor.from_buf("i32", [1, 0, 1, 1], [4])   # the reference panics on a zero divisor
    with pytest.raises(TensorError):
        OTensor.from_buf("i32", [-2 ** 31], [1]) / OTensor.from_buf("i32", [-1], [1])


def test_inplace_through_random_views(oracle_lib):
    rng = np.random.default_rng(99)
    for trial in range(60):
        rank = int(rng.integers(1, 5))
        shape = [int(rng.integers(1, 7)) for _ in range(rank)]
        dtype = DTYPES[trial % len(DTYPES)]
        vals = rand_values(dtype, int(np.prod(shape)), rng)
        t = OTensor.from_buf(dtype, vals, shape)
        v = random_view(t, rng)
        ref = vals.copy()
        nv = as_strided(ref[v.meta.offset:v.meta.offset + 1], shape=v.meta.shape,
                        strides=[s * ref.dtype.itemsize for s in v.meta.strides])
        which = trial % 3
        with np.errstate(over="ignore"):
            if which == 0:
                v += 3
                nv += ref.dtype.type(3)
            elif which == 1:
                v.unary_inplace("relu")
                np.maximum(nv, 0, out=nv)
            else:
                v.fill(7)
                nv[...] = 7
        assert t.buf.tobytes() == ref.tobytes(), (trial, dtype, v.meta)


UNARY_NP = {
    "neg": np.negative, "abs": np.abs, "square": lambda x: x * x, "cube": lambda x: x * x * x,
    "reciprocal": lambda x: x.dtype.type(1) / x, "sqrt": np.sqrt, "floor": np.floor, "ceil": np.ceil, "trunc": np.trunc,
    "sign": np.sign,
}


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("op", sorted(UNARY_NP))
def test_exact_unary_vs_numpy(dtype, op, oracle_lib):
    rng = np.random.default_rng(5)
    x = rand_values(dtype, 1000, rng)
    x[:6] = [0.0, -0.0, 1.5, -2.5, 0.5, -0.5]
    t = OTensor.from_buf(dtype, x, [1000])
    with np.errstate(invalid="ignore", divide="ignore"):
        want = UNARY_NP[op](x)
    got = t.unary(op).buf
    if op == "sign":
        assert np.array_equal(got, want)                    # -0.0 -> 0 either sign compares equal; NaN-free input
    else:
        assert got.tobytes() == want.astype(x.dtype).tobytes(), op


def test_special_values(oracle_lib):
    nan, inf = np.float32("nan"), np.float32("inf")
    x = np.array([nan, -0.0, 0.0, -inf, inf, -1.0], dtype=np.float32)
    t = OTensor.from_buf("f32", x, [6])
    relu = t.unary("relu").buf                               # `x > 0 ? x : 0` (backend/cpu.rs:650-657): NaN -> 0, -0.0 -> +0.0
    assert relu.tobytes() == np.array([0.0, 0.0, 0.0, 0.0, inf, 0.0], dtype=np.float32).tobytes()
    sign = t.unary("sign").buf                               # backend/cpu.rs:548-557: NaN -> 0
    assert sign.tobytes() == np.array([0.0, 0.0, 0.0, -1.0, 1.0, -1.0], dtype=np.float32).tobytes()
    ab = t.unary("abs").buf                                  # f32::abs clears the sign bit
    assert np.signbit(ab).sum() == 0 and np.isnan(ab[0])
    lr = OTensor.from_buf("f32", x, [6]).scalar_op_inplace("leaky_relu", 0.5).buf   # `x > 0 ? x : x * s`
    assert np.isnan(lr[0]) and np.signbit(lr[1]) and not np.signbit(lr[2]) and lr[3] == -inf and lr[5] == -0.5
    i = OTensor.from_buf("i32", [-2 ** 31, -5, 0, 7], [4])
    assert i.unary("abs").buf.tolist() == [-2 ** 31, 5, 0, 7]      # i32::MIN.abs() wraps in release builds
    assert i.unary("neg").buf.tolist() == [-2 ** 31, 5, 0, -7]
    assert i.unary("relu").buf.tolist() == [0, 0, 0, 7]


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "i64", "u8"])
def test_leaky_relu_gradient_map(dtype, oracle_lib):
    # ops/scalar/mod.rs:149-166: `if val > 0 { 1 } else { scalar }`, element by element
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    x = np.array([3, 0, 1, 0, 7, 2, 0, 9], dtype=npd) if dtype == "u8" else np.array([3, -2, 0, -0.0, 7, -9, 1, -1], dtype=npd)
    s = npd.type(0.25) if dtype[0] == "f" else npd.type(5)
    if dtype[0] == "f":
        x[5] = np.nan                                        # NaN > 0 is false -> slope
    t = OTensor.from_buf(dtype, x, [8])
    got = t.scalar_op_inplace("leaky_grad", s).buf
    want = np.where(x > 0, npd.type(1), s).astype(npd)
    assert got.tobytes() == want.tobytes()
    v = OTensor.from_buf(dtype, x, [8]).slice(0, Slice(None, None, -3))      # elements 7, 4, 1 through a reversed view
    v.scalar_op_inplace("leaky_grad", s)
    want2 = x.copy(); want2[[7, 4, 1]] = want[[7, 4, 1]]
    assert v.buf.tobytes() == want2.tobytes()


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_transcendental_unary_within_reference_tolerance(dtype, oracle_lib):
    # bit parity of these is unpinned (platform libm on both sides); the reference's own tests use 1e-5
    rng = np.random.default_rng(11)
    x = (rng.random(500) * 1.8 - 0.9).astype(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]])
    t = OTensor.from_buf(dtype, x, [500])
    x64 = x.astype(np.float64)
    table = {"exp": np.exp, "sin": np.sin, "cos": np.cos, "tan": np.tan, "asin": np.arcsin, "acos": np.arccos,
             "atan": np.arctan, "sinh": np.sinh, "cosh": np.cosh, "tanh": np.tanh, "asinh": np.arcsinh,
             "atanh": np.arctanh, "expm1": np.expm1, "ln1p": np.log1p,
             "sigmoid": lambda v: 1 / (1 + np.exp(-v)), "silu": lambda v: v / (1 + np.exp(-v))}
    for op, f in table.items():
        got = t.unary(op).buf.astype(np.float64)
        assert np.max(np.abs(got - f(x64))) < 1e-5, op
    pos = OTensor.from_buf(dtype, np.abs(x) + 1.5, [500])
    p64 = pos.buf.astype(np.float64)
    assert np.max(np.abs(pos.unary("ln").buf - np.log(p64))) < 1e-5
    assert np.max(np.abs(pos.unary("acosh").buf - np.arccosh(p64))) < 1e-5
    assert np.max(np.abs(pos.unary("rsqrt").buf - 1 / np.sqrt(p64))) < 1e-5
    assert np.max(np.abs(pos.owned().scalar_op_inplace("log", 10.0).buf - np.log10(p64))) < 1e-5
    assert np.max(np.abs(pos.owned().scalar_op_inplace("log1p", 10.0).buf - np.log1p(p64) / np.log(10.0))) < 1e-5
    e = t.owned().scalar_op_inplace("elu", 0.3).buf
    assert np.max(np.abs(e - np.where(x64 >= 0, x64, 0.3 * np.expm1(x64)))) < 1e-5


def sequential(op, x):
    """Strict left-to-right fold with numpy scalar arithmetic (ufunc.accumulate is sequential by definition)."""
    if op in ("sum", "mean"):
        with np.errstate(over="ignore"):
            s = np.add.accumulate(x, dtype=x.dtype)[-1]
        if op == "mean":
            if x.dtype.kind == "f":
                return s / x.dtype.type(np.float32(x.size))
            # The reference's Mean accumulator instantiated at an integer type: the wrapped sum, divided (Rust `/`, truncating toward
            # zero) by T::from_usize(n) = (n as f32) as T, a cast that saturates (core/value.rs:54-56; ops/reduction/mod.rs:112-137).
            # Written with Python integers, not with the oracle's C++ expression.
            info = np.iinfo(x.dtype)
            width = 2 ** (8 * x.dtype.itemsize)
            total = sum(int(v) for v in x)
            total = (total - info.min) % width + info.min                       # wrap into T
            count = min(max(int(np.float32(x.size)), info.min), info.max)       # saturating float -> int cast
            q = abs(total) // abs(count)
            return -q if (total < 0) != (count < 0) else q
        return s
    if op == "prod":
        with np.errstate(over="ignore"):
            return np.multiply.accumulate(x, dtype=x.dtype)[-1]
    if op == "max":
        return max(np.finfo(x.dtype).min if x.dtype.kind == "f" else np.iinfo(x.dtype).min, x.max())
    return min(np.finfo(x.dtype).max if x.dtype.kind == "f" else np.iinfo(x.dtype).max, x.min())


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "i64", "u8"])
@pytest.mark.parametrize("op", ["sum", "prod", "max", "min", "mean"])
def test_reduce_vs_sequential_numpy(dtype, op, oracle_lib):
    rng = np.random.default_rng(3)
    for shape in ([7], [4, 5], [3, 4, 5], [2, 3, 4, 5], [1, 6], [6, 1], [257, 3]):
        x = rand_values(dtype, int(np.prod(shape)), rng)
        if op == "prod" and x.dtype.kind == "f":
            x = (x * 0.1 + 1).astype(x.dtype)
        t = OTensor.from_buf(dtype, x, shape)
        full = t.reduce(op).buf[0]
        assert full.tobytes() == np.asarray(sequential(op, x)).astype(x.dtype).tobytes(), (dtype, op, shape, "flat")
        xs = x.reshape(shape)
        for axis in range(len(shape)):
            got = t.reduce(op, axis)
            assert got.meta.shape == [1 if d == axis else shape[d] for d in range(len(shape))]
            want = np.apply_along_axis(lambda v: sequential(op, np.ascontiguousarray(v)), axis, xs)
            assert got.buf.tobytes() == np.ascontiguousarray(want).astype(x.dtype).tobytes(), (dtype, op, shape, axis)


def test_int_sum_is_sum_mod_2w(oracle_lib):
    rng = np.random.default_rng(8)
    x = rng.integers(-2 ** 31, 2 ** 31, size=5000, dtype=np.int64).astype(np.int32)
    got = int(cpu.reduce_flat(cpu.I32, "sum", x, 0, x.size)[0])
    want = (int(x.astype(np.int64).sum()) + 2 ** 31) % 2 ** 32 - 2 ** 31
    assert got == want


def test_max_min_corner_cases(oracle_lib):
    nan, inf = float("nan"), float("inf")
    f = lambda vals, op: cpu.reduce_flat(cpu.F32, op, np.array(vals, dtype=np.float32), 0, len(vals))[0]
    assert f([nan, 1.0, nan, 3.0, 2.0], "max") == 3.0                       # `if value > max`: NaN never wins
    assert f([nan, nan], "max") == np.finfo(np.float32).min                  # stays at T::MIN (lowest finite)
    assert f([-inf, -inf], "max") == np.finfo(np.float32).min
    assert f([inf, nan], "min") == np.finfo(np.float32).max
    assert np.signbit(f([-0.0, 0.0], "max")) and not np.signbit(f([0.0, -0.0], "max"))   # first of equals stays
    assert not np.signbit(f([0.0, -0.0], "min")) and np.signbit(f([-0.0, 0.0], "min"))


def test_reduce_nd_offset_behaviour(oracle_lib):
    # backend/cpu.rs:434 has no offset term (reference-acknowledged bug, backend/remote/server.rs:327-330);
    # honour_offset=True is the Cuda behaviour (backend/cuda.rs:1934) and the one the product implements.
    x = np.arange(24, dtype=np.float64)
    m = MetaTensor([2, 3], [3, 1], 6)            # rows 2..3 of an (8,3) buffer
    lit = cpu.reduce_nd(cpu.F64, "sum", x, m, 1, honour_offset=False)
    hon = cpu.reduce_nd(cpu.F64, "sum", x, m, 1, honour_offset=True)
    assert lit.tolist() == [3.0, 12.0] and hon.tolist() == [21.0, 30.0]


def test_noncontiguous_reduce_goes_through_contiguous(oracle_lib):
    x = np.arange(12, dtype=np.float32)
    t = OTensor.from_buf("f32", x, [3, 4])
    got = t.transpose().sum_at(0)
    assert got.meta.shape == [1, 3] and got.buf.tolist() == x.reshape(3, 4).sum(axis=1).tolist()


def test_gather_and_equal(oracle_lib):
    x = np.arange(24, dtype=np.int32)
    t = OTensor.from_buf("i32", x, [2, 3, 4])
    v = t.permute([2, 0, 1]).slice(0, Slice(None, None, -1))
    assert np.array_equal(v.to_numpy(), np.transpose(x.reshape(2, 3, 4), (2, 0, 1))[::-1])
    a = np.array([1.0, np.nan], dtype=np.float32)
    assert not cpu.equal(cpu.F32, a, a.copy())               # NaN != NaN, as for Box<[f32]> ==
    assert cpu.equal(cpu.F32, np.array([0.0], np.float32), np.array([-0.0], np.float32))


def test_bool_and_128bit(oracle_lib):
    a = OTensor.from_buf("bool", [1, 0, 1, 0], [4]); b = OTensor.from_buf("bool", [1, 1, 0, 0], [4])
    assert (a + b).buf.tolist() == [True, True, True, False]      # OR
    assert (a - b).buf.tolist() == [False, True, True, False]     # XOR
    assert (a * b).buf.tolist() == [True, False, False, False]    # AND
    big = 2 ** 127 - 1
    x = OTensor.from_buf("i128", [big, -5, 3], [3])
    y = OTensor.from_buf("i128", [1, 7, 2 ** 100], [3])
    assert cpu.to_ints(cpu.I128, (x + y).buf) == [-2 ** 127, 2, 3 + 2 ** 100]
    assert cpu.to_ints(cpu.I128, (x * y).buf) == [big, -35, 3 * 2 ** 100]
    u = OTensor.from_buf("u128", [2 ** 128 - 1, 10], [2])
    assert cpu.to_ints(cpu.U128, (u + OTensor.from_buf("u128", [2, 5], [2])).buf) == [1, 15]
    assert cpu.to_ints(cpu.U128, (u / OTensor.from_buf("u128", [2 ** 64, 3], [2])).buf) == [2 ** 64 - 1, 3]


def test_dispatch_paths(oracle_lib):
    t = OTensor.from_buf("f32", np.arange(16, dtype=np.float32), [4, 4])
    assert t.meta.dispatch()[0] == "contiguous"
    assert t.slice(1, Slice.index(1)).meta.dispatch() == ("1d_strided", (1, 4, 4))
    assert t.slice(0, Slice(None, None, 2)).slice(1, Slice(None, None, 2)).meta.dispatch()[0] == "nd"
    # |stride| contiguity (core/meta.rs:536): a fully reversed view is "contiguous" and the Cpu loop then slices
    # buf[offset..offset+len] with offset = index of the *last* element -> out-of-bounds panic in the reference.
    rev = OTensor.from_buf("f32", np.arange(4, dtype=np.float32), [4]).slice(0, Slice(None, None, -1))
    assert rev.meta.is_contiguous() and rev.meta.dispatch() == ("contiguous", (3, 4))
    from oracle.meta import TensorError
    with pytest.raises(TensorError):
        rev.unary_inplace("relu")
