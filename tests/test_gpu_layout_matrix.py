"""Every in-place op through every layout entry point of the C ABI, against the Cpu loops of the reference as the oracle restates them.

The trait gives each of the 31 unary ops, the 8 scalar ops and fill three methods -- `_contiguous(start, len)`, `_1d_strided(offset,
stride, len)`, `_nd(offset, shape, strides)` (backend/mod.rs:96-213, 239-294) -- and a dispatching method that picks one of them
(backend/mod.rs:15-94).  Here all three entry points (rt_unary_*, rt_scalar_*, rt_fill_*) are called directly, for every op the trait
admits for a dtype: f32 / f64 all of them, the integers (u16 / u32 / u64 / i8 / u128 / i128 included) relu, abs, neg, the gradient
maps, scalar add / sub / mul / div / leaky_relu and fill.  Layouts: runs that start on and off the 16-byte grid; strides +2, +3, -1,
-2 at a non-zero offset; the reference's own fixtures (testing/mod.rs:6-195: (2, 1) contiguous, (3, 1) with step 2, (4, 4, 1) with
step 2 x 2); a view with long rows; a rank-10 view with every dim sliced.  Results are bit for bit the oracle's for the exact ops and
within the reference's 1e-5 for the transcendental ones; every element outside the view must keep its bits."""
import zlib

import numpy as np
import pytest

from oracle import cpu
from oracle.meta import MetaTensor

pytestmark = pytest.mark.gpu

UNARY_EXACT = ["neg", "relu", "abs", "sqrt", "floor", "ceil", "round", "trunc", "reciprocal", "square", "cube", "sign"]
UNARY_TOL = ["sigmoid", "silu", "tanh", "ln", "expm1", "ln1p", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "asinh",
             "acosh", "atanh", "rsqrt", "exp"]
SCALAR_FLOAT = {"add": 3.0, "sub": 7.0, "mul": 3.0, "div": 0.7, "log": 10.0, "log1p": 10.0, "leaky_relu": 0.1, "elu": 0.3}
SCALAR_INT = {"add": 3, "sub": 7, "mul": 3, "div": 3, "leaky_relu": 2}
INT_DTYPES = ["u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64", "u128", "i128"]


@pytest.fixture(scope="module")
def hip():
    from rtensors_amd import hip as H
    b = H.Hip.new(0)
    yield b
    b.sync()


def layouts(n):
    """(entry point, MetaTensor) pairs over a buffer of n elements (n >= 59049)."""
    out = []
    for start, ln in ((0, n), (1, n - 3), (5, 1000), (n - 7, 7), (3, 0)):
        out.append(("contiguous", MetaTensor([ln], [1], start)))
    for stride, off, ln in ((2, 3, (n - 3) // 2), (3, 1, (n - 1) // 3), (-1, n - 2, n - 5), (-2, n - 1, (n - 1) // 2), (7, 11, 100), (-1, 40, 1)):
        out.append(("1d_strided", MetaTensor([ln], [stride], off)))
    out.append(("1d_strided", MetaTensor([2], [2], 0)))                                         # testing/mod.rs: (3, 1) sliced with step 2
    out.append(("nd", MetaTensor([2, 2, 1], [8, 2, 1], 0)))                                     # testing/mod.rs: (4, 4, 1) step 2 x 2
    out.append(("nd", MetaTensor([2, 1], [1, 1], 0)))                                           # testing/mod.rs: the (2, 1) contiguous fixture through nd
    rows, pitch = 37, 1040
    out.append(("nd", MetaTensor([rows, 1031], [pitch, 1], 5)))                                 # long unit-stride rows off the vector grid
    out.append(("nd", MetaTensor([rows, 512], [-pitch, 2], (rows - 1) * pitch + 3)))            # rows walked backwards, stepped columns
    out.append(("nd", MetaTensor([6, 5, 40], [40, 6 * 40 * 33, 1], 17)))                        # permuted outer dims
    # rank 10: a (3,) * 10 tensor (59049 elements) with every dim sliced at step 2, forwards and backwards in turn -> (2,) * 10
    st = [3 ** (9 - i) for i in range(10)]
    strides10 = [s * 2 if k % 2 == 0 else -s * 2 for k, s in enumerate(st)]
    off10 = sum(-s for s in strides10 if s < 0)
    out.append(("nd", MetaTensor([2] * 10, strides10, off10)))
    return out


def elements(meta):
    """Buffer indices a view addresses."""
    idx = np.array([meta.offset], dtype=np.int64)
    for d, s in zip(meta.shape, meta.strides):
        idx = (idx[:, None] + (np.arange(d, dtype=np.int64) * s)[None, :]).reshape(-1)
    return idx


def oracle_view(meta):
    """The same elements as a view the reference's dispatch walks correctly.  Its contiguity test compares |stride| (core/meta.rs:536),
    so a fully reversed view would reach the contiguous loop with the offset of its last element; elementwise ops do not depend on
    the order of the elements, so such a view is handed to the oracle walked forwards."""
    if meta.rank() == 1 and meta.strides[0] == -1 and meta.shape[0] > 1:
        return MetaTensor([meta.shape[0]], [1], meta.offset - (meta.shape[0] - 1))
    return meta


def call(hip, family, entry, op, buf, value, meta):
    if entry == "contiguous":
        args = (meta.offset, meta.shape[0])
    elif entry == "1d_strided":
        args = (meta.offset, meta.strides[0], meta.shape[0])
    else:
        args = (meta.offset, list(meta.shape), list(meta.strides))
    if family == "unary":
        getattr(hip, f"unary_{entry}")(op, buf, *args)
    elif family == "scalar":
        getattr(hip, f"scalar_{entry}")(op, buf, value, *args)
    else:
        getattr(hip, f"fill_{entry}")(buf, value, *args)


def float_input(npd, n, op, rng):
    x = (rng.standard_normal(n) * 0.6).astype(npd)
    x[:14] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1.0, -1.0, 0.5, -0.5, 2.5, np.finfo(npd).tiny / 4, -np.finfo(npd).tiny / 4, np.finfo(npd).tiny, np.finfo(npd).max]
    if op in ("ln", "ln1p", "sqrt", "rsqrt", "acosh", "log", "log1p"):
        x = np.abs(x) + (1.0 if op in ("acosh", "log", "log1p") else 0.0)
        x[2:5] = [1.0, 2.0, 3.0]
    if op in ("asin", "acos", "atanh"):
        x = np.clip(x, -0.95, 0.95)
        x[2] = 0.25
    return x.astype(npd)


def check_float(got, want, before, idx, exact, what):
    mask = np.zeros(got.size, dtype=bool)
    mask[idx] = True
    assert got[~mask].tobytes() == before[~mask].tobytes(), (what, "elements outside the view changed")
    g, w = got[mask], want[mask]
    if exact:
        both_nan = np.isnan(g) & np.isnan(w)
        u = np.uint32 if g.dtype == np.float32 else np.uint64
        assert np.all(both_nan | (g.view(u) == w.view(u))), what
    else:
        ok = np.isclose(g.astype(np.float64), w.astype(np.float64), rtol=1e-5, atol=1e-5, equal_nan=True)
        assert ok.all(), (what, g[~ok][:4], w[~ok][:4])


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_float_ops_through_every_entry_point(hip, dtype):
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 1)
    n = 65_536
    lay = layouts(n)
    assert {e for e, _ in lay} == {"contiguous", "1d_strided", "nd"} and any(m.rank() == 10 for _, m in lay)
    cases = [("unary", op, None) for op in UNARY_EXACT + UNARY_TOL] + [("scalar", op, v) for op, v in SCALAR_FLOAT.items()] + [("fill", "fill", 1.5)]
    for family, op, value in cases:
        x = float_input(npd, n, op, rng)
        exact = family == "fill" or (family == "unary" and op in UNARY_EXACT) or (family == "scalar" and op not in ("log", "log1p", "elu"))
        for entry, meta in lay:
            want = x.copy()
            om = oracle_view(meta)
            with np.errstate(all="ignore"):
                if family == "unary":
                    cpu.unary(code, op, want, om)
                elif family == "scalar":
                    cpu.scalar(code, op, want, value, om)
                else:
                    cpu.fill(code, want, value, om)
            g = hip.alloc_from_slice(code, x)
            call(hip, family, entry, op, g, value, meta)
            check_float(hip.dump(g), want, x, elements(meta), exact, (dtype, family, op, entry, meta))


def int_values(dtype, n, rng):
    code = cpu.DTYPE_BY_NAME[dtype]
    if dtype in ("u128", "i128"):
        lo, hi = (0, (1 << 128) - 1) if dtype == "u128" else (-(1 << 127), (1 << 127) - 1)
        vals = [int(rng.integers(-1000, 1000)) for _ in range(n)]
        for i in range(0, n, 7):
            vals[i] = (int(rng.integers(0, 1 << 62)) << 64) | int(rng.integers(0, 1 << 62))
            if dtype == "i128" and i % 14 == 0:
                vals[i] = -vals[i]
        vals[:4] = [lo, hi, 0, 1]
        if dtype == "u128":
            vals = [abs(v) for v in vals]
        return cpu.from_ints(code, vals)
    npd = cpu.NP_DTYPE[code]
    info = np.iinfo(npd)
    x = rng.integers(max(info.min, -1000), min(info.max, 1000) + 1, size=n, dtype=np.int64).astype(npd)
    x[:4] = [info.min, info.max, 0, 1]
    return x


@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_integer_ops_through_every_entry_point(hip, dtype):
    from rtensors_amd import hip as H
    code = cpu.DTYPE_BY_NAME[dtype]
    signed = dtype[0] == "i"
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 2)
    n = 65_536
    lay = layouts(n)
    x = int_values(dtype, n, rng)
    cases = [("unary", op, None) for op in ("relu", "abs") + (("neg",) if signed else ())]
    cases += [("scalar", op, v) for op, v in SCALAR_INT.items()] + [("fill", "fill", 5)]
    if signed:
        cases.append(("scalar", "mul", -3))
    for family, op, value in cases:
        for entry, meta in lay:
            want = x.copy()
            om = oracle_view(meta)
            if family == "unary":
                cpu.unary(code, op, want, om)
            elif family == "scalar":
                cpu.scalar(code, op, want, value, om)
            else:
                cpu.fill(code, want, value, om)
            g = hip.alloc_from_slice(code, x)
            call(hip, family, entry, op, g, value, meta)
            assert hip.dump(g).tobytes() == want.tobytes(), (dtype, family, op, entry, meta)
    # the gradient maps (no loop of their own in the Cpu backend: x > 0 ? 1 : 0 / -1 / slope, ops/unary/mod.rs:213-252, ops/scalar/mod.rs:149-166)
    ints = cpu.to_ints(code, x)
    maps = [("unary", "step", None, lambda v: 1 if v > 0 else 0), ("scalar", "leaky_grad", 3, lambda v: 1 if v > 0 else 3)]
    if signed:
        maps.append(("unary", "abs_grad", None, lambda v: 1 if v > 0 else -1))
    for family, op, value, rule in maps:
        for entry, meta in lay:
            idx = elements(meta)
            want = list(ints)
            for i in idx.tolist():
                want[i] = rule(ints[i])
            g = hip.alloc_from_slice(code, x)
            call(hip, family, entry, op, g, value, meta)
            assert hip.dump(g).tobytes() == cpu.from_ints(code, want).tobytes(), (dtype, op, entry, meta)
    # ops the trait bounds on f32 / f64 are refused for every entry point alike
    g = hip.alloc_from_slice(code, x)
    for entry, meta in (lay[0], lay[6], lay[-1]):
        with pytest.raises(H.TensorError) as e:
            call(hip, "unary", entry, "sqrt", g, None, meta)
        assert e.value.kind == "UnsupportedOperation"
        with pytest.raises(H.TensorError) as e:
            call(hip, "scalar", entry, "elu", g, 1, meta)
        assert e.value.kind == "UnsupportedOperation"
    assert hip.dump(g).tobytes() == x.tobytes()


def test_bool_ops_through_every_entry_point(hip):
    """bool: + is OR, - is XOR, * is AND (core/value.rs:650-765); relu / abs are the identity; fill."""
    code = cpu.BOOL
    rng = np.random.default_rng(9)
    n = 65_536
    x = rng.integers(0, 2, size=n).astype(np.bool_)
    for family, op, value in [("scalar", "add", True), ("scalar", "add", False), ("scalar", "sub", True), ("scalar", "mul", False), ("scalar", "mul", True),
                              ("unary", "relu", None), ("unary", "abs", None), ("fill", "fill", True)]:
        for entry, meta in layouts(n):
            want = x.copy()
            om = oracle_view(meta)
            if family == "unary":
                cpu.unary(code, op, want, om)
            elif family == "scalar":
                cpu.scalar(code, op, want, value, om)
            else:
                cpu.fill(code, want, value, om)
            g = hip.alloc_from_slice(code, x)
            call(hip, family, entry, op, g, value, meta)
            assert hip.dump(g).tobytes() == want.tobytes(), (family, op, value, entry, meta)
