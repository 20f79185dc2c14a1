"""GPU parity: every kernel family of the HIP backend, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Bit-exact for integers, for f32/f64 elementwise results, and for max/min; float sum/prod/mean within
rel 1e-5 (f32) / 1e-12 (f64) of sum|x|; transcendental unaries within the reference's own 1e-5."""
import os
import zlib
import numpy as np
import pytest

import golden_dsl
from oracle import cpu
from oracle.meta import MetaTensor, Slice, TensorError as OErr
from oracle.tensor import OTensor

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from rtensors_amd import hip as H
    b = H.Hip.new(0)
    yield b
    b.sync()


def G(hip, dtype, values, shape):
    from gpu_tensor import GTensor
    return GTensor.from_buf(hip, dtype, values, shape)


def rand_values(dtype, n, rng, lo=-1000, hi=1000):
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    if npd.kind == "f":
        return rng.standard_normal(n).astype(npd)
    if npd.kind == "b":
        return rng.integers(0, 2, size=n).astype(npd)
    info = np.iinfo(npd)
    return rng.integers(max(info.min, lo), min(info.max, hi) + 1, size=n, dtype=np.int64).astype(npd)


ALL_DTYPES = ["u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64", "f32", "f64", "bool"]
NUM_DTYPES = [d for d in ALL_DTYPES if d != "bool"]


def random_view(t, rng, allow_rev=True):
    v = t.view()
    for _ in range(int(rng.integers(0, 4))):
        r = v.meta.rank()
        if r == 0:
            break
        k = int(rng.integers(0, 3))
        d = int(rng.integers(0, r))
        n = v.meta.shape[d]
        if k == 0 and v.meta.strides[d] > 0:
            steps = [1, 2, 3, -1, -2] if allow_rev else [1, 2, 3]
            step = int(rng.choice(steps))
            if step > 0:
                a = int(rng.integers(0, n)); b = int(rng.integers(a + 1, n + 1))
                v = v.slice(d, Slice(a, b, step))
            else:
                a = int(rng.integers(0, n)); b = int(rng.integers(-1, a))
                v = v.slice(d, Slice(a, None if b < 0 else b, step))
        elif k == 1 and r > 1:
            v = v.permute([int(x) for x in rng.permutation(r)])
        elif k == 2:
            v = v.unsqueeze_at(d)
    return v


def replay(view_meta_src, g):
    """A GTensor view with the same layout as an oracle view."""
    return g._view(view_meta_src.meta.shape, view_meta_src.meta.strides, view_meta_src.meta.offset)


# ---------------------------------------------------------------------------------------------------------------------
def test_buffers_and_transfers(hip):
    from rtensors_amd import hip as H
    rng = np.random.default_rng(0)
    for dtype in ALL_DTYPES:
        code = H.DTYPE_BY_NAME[dtype]
        x = rand_values(dtype, 1000, rng)
        z = hip.alloc(code, 777)
        assert not hip.dump(z).any()                                      # Backend::alloc is zero-initialised
        b = hip.alloc_from_slice(code, x)
        assert hip.len(b) == 1000 and hip.dump(b).tobytes() == x.tobytes()
        assert hip.read(b, 123) == x[123]
        hip.write(b, 123, x[5])
        y = x.copy(); y[123] = x[5]
        assert hip.dump(b).tobytes() == y.tobytes()
        c = hip.copy(b)
        assert c == b and hip.dump(c).tobytes() == y.tobytes()
        hip.copy_range_within(c, b, 10, 500, 100)
        y2 = y.copy(); y2[10:110] = y[500:600]
        assert hip.dump(c).tobytes() == y2.tobytes()
        assert not (c == b)
        hip.copy_from_slice(c, x)
        assert hip.dump(c).tobytes() == x.tobytes()
        with pytest.raises(H.TensorError) as e:
            hip.copy_from_slice(c, x[:10])
        assert e.value.kind == "SizeMismatch"
        with pytest.raises(H.TensorError) as e:
            hip.read(b, 1000)
        assert e.value.kind == "IdxOutOfBounds"
        with pytest.raises(H.TensorError):
            hip.write(b, 1000, x[0])
        with pytest.raises(H.TensorError):
            hip.copy_range_within(c, b, 950, 0, 100)
    # device copies large enough for the vector copy kernel: equal and unequal 16-byte phases, ragged ends
    big = rng.integers(0, 256, size=100_003, dtype=np.uint8)
    src = hip.alloc_from_slice(H.U8, big)
    assert hip.dump(hip.copy(src)).tobytes() == big.tobytes()
    for dst_off, src_off, length in ((0, 0, 100_003), (16, 32, 70_001), (5, 21, 50_000), (3, 4, 60_000), (7, 7, 99_990), (1, 17, 4096), (9, 9, 15)):
        dst = hip.alloc(H.U8, 100_003)
        hip.copy_range_within(dst, src, dst_off, src_off, length)
        want = np.zeros(100_003, dtype=np.uint8); want[dst_off:dst_off + length] = big[src_off:src_off + length]
        assert hip.dump(dst).tobytes() == want.tobytes(), (dst_off, src_off, length)
    nan = hip.alloc_from_slice(H.F32, np.array([1.0, np.nan], np.float32))
    assert not (nan == hip.copy(nan))                                     # NaN != NaN, like Box<[f32]> ==
    pz = hip.alloc_from_slice(H.F32, np.array([0.0], np.float32)); nz = hip.alloc_from_slice(H.F32, np.array([-0.0], np.float32))
    assert pz == nz
    assert not (hip.alloc(H.F32, 3) == hip.alloc(H.F32, 4))


@pytest.mark.parametrize("dtype", ["u8", "i16", "f32", "f64"])
def test_copy_range_within_any_phase(hip, dtype):
    """`copy_range_within` (backend/mod.rs:227-229) with source and destination ranges in every 16-byte phase relative to each other and
    to the 128-byte lines the copy kernel aligns its body to; lengths from a single element to several blocks; the bytes outside the
    destination range stay untouched."""
    code = cpu.DTYPE_BY_NAME[dtype]
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 5)
    n = 6000
    x = rand_values(dtype, n, rng)
    src = hip.alloc_from_slice(code, x)
    for trial in range(60):
        ln = int(rng.choice([1, 2, 3, 15, 16, 17, 31, 127, 128, 129, 1000, 4097, 5000]))
        do, so = int(rng.integers(0, n - ln + 1)), int(rng.integers(0, n - ln + 1))
        if trial < 20:
            do, so = trial % 5, (trial * 3) % 7                                 # small offsets: every phase pair near the buffer start
            ln = min(ln, n - 8)
        y = rand_values(dtype, n, rng)
        dst = hip.alloc_from_slice(code, y)
        hip.copy_range_within(dst, src, do, so, ln)
        want = y.copy(); want[do:do + ln] = x[so:so + ln]
        assert hip.dump(dst).tobytes() == want.tobytes(), (dtype, do, so, ln)
    with pytest.raises(Exception):
        hip.copy_range_within(src, src, n - 3, 0, 4)


def test_allocator_reuses_blocks(hip):
    from rtensors_amd import hip as H
    hip.sync()
    a = hip.alloc(H.F32, 1 << 20); del a
    before = hip.mem_stats()["device_allocs"]
    for _ in range(20):
        b = hip.alloc(H.F32, 1 << 20); del b
    assert hip.mem_stats()["device_allocs"] == before


def test_large_transfers_round_trip(hip):
    """Host <-> device copies above 4 MiB go through the pinned staging ring in 8 MiB chunks split over four copy threads:
    sizes on and around every boundary must come back byte for byte, also when several threads transfer at once."""
    import threading
    from rtensors_amd import hip as H
    rng = np.random.default_rng(77)
    mib = 1 << 20
    sizes = [4 * mib - 1, 4 * mib, 4 * mib + 1, 8 * mib - 64, 8 * mib, 8 * mib + 3, 32 * mib, 32 * mib + 5, 41 * mib + 777]
    for n in sizes:
        x = rng.integers(0, 256, size=n, dtype=np.uint8)
        b = hip.alloc_from_slice(H.U8, x)
        assert hip.dump(b).tobytes() == x.tobytes(), n
        y = rng.integers(0, 256, size=n, dtype=np.uint8)
        hip.copy_from_slice(b, y)
        assert hip.dump(b).tobytes() == y.tobytes(), n
    x64 = rng.standard_normal(3 * mib + 11)                     # 24 MiB + 88 bytes of f64
    assert hip.dump(hip.alloc_from_slice(H.F64, x64)).tobytes() == x64.tobytes()
    errors = []
    def worker(seed):
        try:
            r = np.random.default_rng(seed)
            be = H.Hip.new(0)                                   # own context: own staging ring, shared copy threads
            for _ in range(3):
                v = r.integers(0, 256, size=9 * mib + seed, dtype=np.uint8)
                if be.dump(be.alloc_from_slice(H.U8, v)).tobytes() != v.tobytes():
                    errors.append(seed)
        except Exception as e:                                  # noqa: BLE001
            errors.append(repr(e))
    ts = [threading.Thread(target=worker, args=(s,)) for s in (1, 2, 3)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errors, errors


UNARY_EXACT = ["neg", "relu", "abs", "sqrt", "floor", "ceil", "round", "trunc", "reciprocal", "square", "cube", "sign"]
UNARY_TOL = ["sigmoid", "silu", "tanh", "ln", "expm1", "ln1p", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "asinh",
             "acosh", "atanh", "rsqrt", "exp"]


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_unary_contiguous_float(hip, dtype):
    rng = np.random.default_rng(1)
    n = 100_003
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    x = (rng.standard_normal(n) * 0.6).astype(npd)
    x[:10] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1.0, -1.0, 0.5, -0.5, 2.5]
    tiny = np.finfo(npd).tiny
    x[10:14] = [tiny / 4, -tiny / 4, tiny, np.finfo(npd).max]            # denormals must not be flushed
    for op in UNARY_EXACT + UNARY_TOL:
        xi = x.copy()
        if op in ("ln", "ln1p", "sqrt", "rsqrt", "acosh"):
            xi = np.abs(xi) + (1.0 if op == "acosh" else 0.0)
            xi[2:5] = [1.0, 2.0, 3.0]
        if op in ("asin", "acos", "atanh"):
            xi = np.clip(xi, -0.95, 0.95); xi[2] = 0.25
        for start in (0, 1, 3):                                          # unaligned starts exercise head/tail handling
            want = xi.copy()
            m = MetaTensor([n - start - 2], [1], start)
            with np.errstate(all="ignore"):
                cpu.unary(cpu.DTYPE_BY_NAME[dtype], op, want, m)
            g = hip.alloc_from_slice(cpu.DTYPE_BY_NAME[dtype], xi)
            hip.unary_contiguous(op, g, start, n - start - 2)
            got = hip.dump(g)
            if op in UNARY_EXACT:
                assert got.tobytes() == want.tobytes(), (op, start)
            else:
                ok = np.isclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-5, atol=1e-5, equal_nan=True)
                assert ok.all(), (op, start, got[~ok][:5], want[~ok][:5])
                assert got[:start].tobytes() == xi[:start].tobytes() and got[n - 2:].tobytes() == xi[n - 2:].tobytes()


@pytest.mark.parametrize("dtype", ["u8", "i8", "bool"])
def test_one_byte_types_every_pair(hip, dtype):
    """The vector kernels handle 1-byte elements four to a 32-bit word.  Every (a, b) byte pair, so every carry / borrow / sign
    combination inside a word: binary ops (contiguous, row-broadcast and in-place-row kernels), scalar ops and relu / neg / abs,
    against two's-complement arithmetic in numpy and against the oracle."""
    from rtensors_amd import hip as H
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    if dtype == "bool":
        a = np.repeat(np.arange(2, dtype=np.uint8), 2).astype(np.bool_); a = np.tile(a, 4096)
        b = np.tile(np.arange(2, dtype=np.uint8), 2).astype(np.bool_); b = np.tile(b, 4096)
        closed = {"add": a | b, "sub": a ^ b, "mul": a & b}
    else:
        a = np.repeat(np.arange(256, dtype=np.uint8), 256).view(npd)
        b = np.tile(np.arange(256, dtype=np.uint8), 256).view(npd)
        w = {"add": a.astype(np.int32) + b, "sub": a.astype(np.int32) - b, "mul": a.astype(np.int32) * b}
        closed = {k: v.astype(np.uint8 if dtype == "u8" else np.int8) for k, v in w.items()}      # astype wraps modulo 256
    n = a.size
    ga, gb = hip.alloc_from_slice(code, a), hip.alloc_from_slice(code, b)
    flat = (0, [n], [1])
    for op in ("add", "sub", "mul"):
        want = np.zeros(n, dtype=npd)
        cpu.broadcast(code, op, a.copy(), MetaTensor([n], [1], 0), b.copy(), MetaTensor([n], [1], 0), want, MetaTensor([n], [1], 0))
        assert want.tobytes() == closed[op].tobytes(), op                  # the oracle agrees with the closed form
        gd = hip.alloc(code, n)
        hip.broadcast((ga, flat), (gb, flat), (gd, flat), op)
        assert hip.dump(gd).tobytes() == want.tobytes(), op
        # rows kernel: right operand is one row of 256 repeated (b is exactly that)
        rows = (0, [n // 256, 256], [256, 1])
        gd2 = hip.alloc(code, n)
        hip.broadcast((ga, rows), (gb, (0, [n // 256, 256], [0, 1])), (gd2, rows), op)
        assert hip.dump(gd2).tobytes() == want.tobytes(), op
    if dtype != "bool":
        x = np.tile(np.arange(256, dtype=np.uint8), 64).view(npd)
        for v in (0, 1, 3, 127, 128, 200, 255):
            sv = int(np.array([v], dtype=np.uint8).view(npd)[0])
            for op in ("add", "sub"):
                g = hip.alloc_from_slice(code, x)
                hip.scalar_contiguous(op, g, sv, 0, x.size)
                wide = x.astype(np.int32) + sv if op == "add" else x.astype(np.int32) - sv
                assert hip.dump(g).tobytes() == wide.astype(npd).tobytes(), (op, v)
                # a view of whole rows inside a wider buffer takes the in-place row kernel
                g = hip.alloc_from_slice(code, x)
                hip.scalar_nd(op, g, sv, 16, [x.size // 64, 32], [64, 1])
                want = x.copy()
                cpu.scalar(code, op, want, sv, MetaTensor([x.size // 64, 32], [64, 1], 16))
                assert hip.dump(g).tobytes() == want.tobytes(), (op, v)
        for op in ("relu", "neg", "abs"):
            want = x.copy()
            try:
                cpu.unary(code, op, want, MetaTensor([x.size], [1], 0))
            except OErr:
                continue
            g = hip.alloc_from_slice(code, x)
            hip.unary_contiguous(op, g, 0, x.size)
            assert hip.dump(g).tobytes() == want.tobytes(), op
            xi = x.astype(np.int32)
            fixed = {"relu": np.maximum(xi, 0), "neg": -xi, "abs": np.abs(xi)}[op].astype(npd)
            assert want.tobytes() == fixed.tobytes(), op
    else:
        x = np.tile(np.array([0, 1, 1, 0, 1], dtype=np.bool_), 4000)
        for v in (False, True):
            for op, f in (("add", np.logical_or), ("sub", np.logical_xor), ("mul", np.logical_and)):
                g = hip.alloc_from_slice(code, x)
                hip.scalar_contiguous(op, g, v, 0, x.size)
                assert hip.dump(g).tobytes() == f(x, v).tobytes(), (op, v)


@pytest.mark.parametrize("dtype", [d for d in ALL_DTYPES if d not in ("f32", "f64")])
def test_unary_contiguous_int(hip, dtype):
    from rtensors_amd import hip as H
    rng = np.random.default_rng(2)
    code = cpu.DTYPE_BY_NAME[dtype]
    x = rand_values(dtype, 5000, rng)
    if dtype not in ("bool",):
        info = np.iinfo(x.dtype); x[:2] = [info.min, info.max]
    for op in ("relu", "abs", "neg", "square"):
        want = x.copy()
        g = hip.alloc_from_slice(code, x)
        try:
            cpu.unary(code, op, want, MetaTensor([5000], [1], 0))
        except OErr:
            with pytest.raises(H.TensorError) as e:                       # same refusal as the trait bounds
                hip.unary_contiguous(op, g, 0, 5000)
            assert e.value.kind == "UnsupportedOperation"
            continue
        hip.unary_contiguous(op, g, 0, 5000)
        assert hip.dump(g).tobytes() == want.tobytes(), op


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_scalar_and_fill_contiguous(hip, dtype):
    from rtensors_amd import hip as H
    rng = np.random.default_rng(3)
    code = cpu.DTYPE_BY_NAME[dtype]
    n = 70_001
    x = rand_values(dtype, n, rng)
    vals = {"add": 3, "sub": 7, "mul": 3, "div": 3, "leaky_relu": 2, "log": 10, "log1p": 10, "elu": 0.3}
    if dtype in ("f32", "f64"):
        vals.update({"mul": 3.0, "div": 0.7, "leaky_relu": 0.1})
    for op, v in vals.items():
        for start in (0, 5):
            want = np.abs(x) + 1 if op in ("log", "log1p") and x.dtype.kind == "f" else x.copy()
            g = hip.alloc_from_slice(code, want)
            m = MetaTensor([n - start - 1], [1], start)
            try:
                with np.errstate(all="ignore"):
                    cpu.scalar(code, op, want, v, m)
            except OErr:
                with pytest.raises(H.TensorError):
                    hip.scalar_contiguous(op, g, v, start, n - start - 1)
                continue
            hip.scalar_contiguous(op, g, v, start, n - start - 1)
            got = hip.dump(g)
            if op in ("log", "log1p", "elu"):
                assert np.allclose(got, want, rtol=1e-5, atol=1e-5), op
            else:
                assert got.tobytes() == want.tobytes(), (op, start)
    if dtype not in ("f32", "f64", "bool"):
        g = hip.alloc_from_slice(code, x)
        with pytest.raises(H.TensorError) as e:
            hip.scalar_contiguous("div", g, 0, 0, n)                       # the reference panics on integer / 0
        assert e.value.kind == "ArithmeticError"
    g = hip.alloc_from_slice(code, x)
    want = x.copy(); want[11:n - 3] = 1
    hip.fill_contiguous(g, 1, 11, n - 14)
    assert hip.dump(g).tobytes() == want.tobytes()


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "i64", "i8"])
def test_gradient_maps(hip, dtype):
    """The three maps the reference's autograd fills with one get/set per element (ops/unary/mod.rs:213-252,
    ops/scalar/mod.rs:149-166): relu -> x > 0 ? 1 : 0, abs -> x > 0 ? 1 : -1, leaky_relu -> x > 0 ? 1 : slope."""
    rng = np.random.default_rng(21)
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    n = 40_003
    x = rand_values(dtype, n, rng)
    if dtype[0] == "f":
        x[:6] = [0.0, -0.0, np.nan, np.inf, -np.inf, np.finfo(npd).tiny / 2]
    else:
        x[:3] = [0, 1, -1]
    slope = npd.type(0.125) if dtype[0] == "f" else npd.type(-3)
    one = npd.type(1)
    with np.errstate(invalid="ignore"):
        pos = x > 0
    cases = {"step": np.where(pos, one, npd.type(0)), "abs_grad": np.where(pos, one, npd.type(-1)), "leaky_grad": np.where(pos, one, slope)}
    for name, full in cases.items():
        full = full.astype(npd)
        for (off, shape, strides) in (([0], [n], [1]), ([5], [(n - 5) // 3], [3]), ([n - 99], [200, 50], [-150, 2])):
            m = MetaTensor(shape, strides, off[0])
            want = x.copy()
            idx = (off[0] + np.add.outer(*[np.arange(sz) * st for sz, st in zip(shape, strides)])).reshape(-1) if len(shape) == 2 \
                else off[0] + np.arange(shape[0]) * strides[0]
            want[idx] = full[idx]
            g = hip.alloc_from_slice(code, x)
            if name == "leaky_grad":
                hip.scalar_nd(name, g, slope, m.offset, m.shape, m.strides)
                chk = x.copy(); cpu.scalar(code, name, chk, slope, m)
                assert chk.tobytes() == want.tobytes()
            else:
                hip.unary_nd(name, g, m.offset, m.shape, m.strides)
            assert hip.dump(g).tobytes() == want.tobytes(), (name, shape, strides)


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i64", "i16"])
def test_inplace_ops_over_random_views(hip, dtype):
    rng = np.random.default_rng(4)
    code = cpu.DTYPE_BY_NAME[dtype]
    for trial in range(40):
        rank = int(rng.integers(1, 5))
        shape = [int(rng.integers(1, 40 if rank < 3 else 12)) for _ in range(rank)]
        vals = rand_values(dtype, int(np.prod(shape)), rng)
        o = OTensor.from_buf(dtype, vals, shape)
        g = G(hip, dtype, vals, shape)
        ov = random_view(o, rng)
        if ov.meta.is_contiguous() and any(s < 0 for s in ov.meta.strides):
            continue        # the reference's |stride| dispatch panics here (out-of-bounds slice); covered separately
        gv = replay(ov, g)
        which = trial % 4
        if which == 0:
            ov.unary_inplace("relu"); gv.unary_inplace("relu")
        elif which == 1:
            ov += 3; gv += 3
        elif which == 2:
            ov.fill(5); gv.fill(5)
        else:
            ov.scalar_op_inplace("leaky_relu", 2); gv.scalar_op_inplace("leaky_relu", 2)
        assert g.dump().tobytes() == o.buf.tobytes(), (trial, dtype, ov.meta)


@pytest.mark.parametrize("dtype", ["f32", "u8", "i16", "f64"])
def test_inplace_ops_on_long_row_views(hip, dtype):
    """Views whose rows hold 64 or more 16-byte vectors (the one-vector-per-lane row kernel): ragged row ends, rows that start
    off the vector and line grid, one and two outer dims, reversed and stepped outer dims.  Everything outside the view must stay
    untouched."""
    rng = np.random.default_rng(41)
    per_vec = 16 // np.dtype(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]).itemsize
    L0 = 135 * per_vec + 3
    for trial, (shape, cuts) in enumerate([
        ([9, 70 * per_vec + 3], [(1, Slice(1, 70 * per_vec, 1))]),
        ([9, L0], [(1, Slice(1, L0 - 2, 1))]),
        ([9, L0 + 13], [(1, Slice(5, 5 + 128 * per_vec, 1)), (0, Slice(None, None, -1))]),
        ([9, L0 + 13], [(1, Slice(3, 3 + 128 * per_vec + 2, 1))]),
        ([3, 6, L0], [(2, Slice(2, None, 1)), (1, Slice(0, None, 2))]),
        ([2, 3, 5, L0], [(3, Slice(0, L0 - 1, 1)), (1, Slice(None, None, -1)), (2, Slice(1, 5, 1))]),
        ([5, 4, 2 * L0], [(2, Slice(L0 // 2, L0 // 2 + 129 * per_vec + 1, 1)), (0, Slice(1, 4, 1))]),
        ([4, 128 * per_vec], [(0, Slice(0, 4, 1))]),
        ([6, 256 * per_vec], [(1, Slice(0, 128 * per_vec, 1))]),
        ([6, 256 * per_vec], [(1, Slice(1, 255 * per_vec, 1))]),
    ]):
        vals = rand_values(dtype, int(np.prod(shape)), rng)
        for which in range(4):
            o = OTensor.from_buf(dtype, vals.copy(), shape)
            g = G(hip, dtype, vals, shape)
            ov, gv = o, g
            for dim, sl in cuts:
                ov, gv = ov.slice(dim, sl), gv.slice(dim, sl)
            if which == 0:
                ov.unary_inplace("relu"); gv.unary_inplace("relu")
            elif which == 1:
                ov += 3; gv += 3
            elif which == 2:
                ov.fill(5); gv.fill(5)
            else:
                ov.scalar_op_inplace("leaky_relu", 2); gv.scalar_op_inplace("leaky_relu", 2)
            assert g.dump().tobytes() == o.buf.tobytes(), (trial, which, dtype, ov.meta)


def test_reversed_view_is_walked_backwards_not_out_of_bounds(hip):
    # Divergence kept on purpose: the reference's |stride| contiguity test (core/meta.rs:536) hands a fully reversed view
    # to the contiguous loop with start = offset of the last element, which panics on Cpu.  Here signed strides are used.
    x = np.arange(10, dtype=np.float32) - 5
    g = G(hip, "f32", x, [10])
    g.slice(0, Slice(None, None, -1)).unary_inplace("relu")
    assert np.array_equal(g.dump(), np.maximum(x, 0))
    o = OTensor.from_buf("f32", x, [10])
    with pytest.raises(OErr):
        o.slice(0, Slice(None, None, -1)).unary_inplace("relu")


CASES = golden_dsl.load("reference_vectors.json") + golden_dsl.load("reference_scalar_vectors.json") + golden_dsl.load("reference_view_vectors.json") + golden_dsl.load("reference_operand_vectors.json") + golden_dsl.load("reference_matmul_vectors.json")


@pytest.mark.parametrize("dispatch", ["nd", "three_way"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_reference_vectors_on_gpu(hip, case, dispatch, monkeypatch):
    """The reference's own known answers.  `nd`: every in-place op goes down as (offset, shape, strides); `three_way`: through the
    `_contiguous` / `_1d_strided` / `_nd` entry point that the trait's default dispatch (backend/mod.rs:15-94) would pick."""
    import copy
    import gpu_tensor
    from gpu_tensor import GTensor
    monkeypatch.setattr(gpu_tensor, "DISPATCH", dispatch)
    case = copy.deepcopy(case)
    env, err = golden_dsl.run_case(case, lambda dt, v, s: GTensor.from_buf(hip, dt, v, s), Slice, OErr)
    if dispatch == "nd":
        for exp in case["expect"]:
            exp.pop("path", None)             # which of the three loops ran is only defined for the three-way dispatch
    golden_dsl.check_case(case, env, err, lambda t: t.to_numpy(), lambda t, idx: t.get(idx),
                          lambda t: (t.meta.shape, t.meta.strides, t.meta.offset, t.meta.is_contiguous()))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_broadcast_random_vs_oracle(hip, dtype, op):
    from rtensors_amd import hip as H
    rng = np.random.default_rng(zlib.crc32((dtype + op).encode()))
    if dtype == "bool" and op == "div":
        pytest.skip("boolean division is todo!() in the reference")
    for trial in range(25):
        rank = int(rng.integers(1, 6))
        big = trial % 5 == 0
        full = [int(rng.integers(1, 7)) for _ in range(rank)]
        if big:
            full[-1] = int(rng.choice([64, 100, 257, 1024, 1500]))
        sa = [d if rng.random() < 0.7 else 1 for d in full]
        sb = [d if rng.random() < 0.7 else 1 for d in full]
        if rng.random() < 0.3:
            sb = sb[int(rng.integers(0, rank)):]
        va, vb = rand_values(dtype, int(np.prod(sa)), rng), rand_values(dtype, int(np.prod(sb)), rng)
        if op == "div" and vb.dtype.kind != "f" and trial % 3 != 0:
            vb[vb == 0] = 1                                                # every third trial keeps its zero divisors
        if op == "div" and vb.dtype.kind == "i" and trial % 6 == 3 and va.size and vb.size:
            va[rng.integers(0, va.size)] = np.iinfo(va.dtype).min          # MIN / -1 overflows
            vb[rng.integers(0, vb.size)] = -1
        oa, ob = OTensor.from_buf(dtype, va, sa), OTensor.from_buf(dtype, vb, sb)
        ga, gb = G(hip, dtype, va, sa), G(hip, dtype, vb, sb)
        ova, ovb = random_view(oa, rng), random_view(ob, rng)
        fault = False
        try:
            with np.errstate(all="ignore"):
                want = {"add": ova.__add__, "sub": ova.__sub__, "mul": ova.__mul__, "div": ova.__truediv__}[op](ovb)
        except OErr as e:
            if e.kind == "BroadcastError":
                continue
            assert e.kind == "ArithmeticPanic" and op == "div", e.kind
            fault = True                                                   # zero divisor or MIN / -1: the reference panics
        gva, gvb = replay(ova, ga), replay(ovb, gb)
        got = {"add": gva.__add__, "sub": gva.__sub__, "mul": gva.__mul__, "div": gva.__truediv__}[op](gvb)
        if fault:
            # the kernel has run; the fault comes back from the next call that waits for the stream, once
            with pytest.raises(H.TensorError) as e:
                got.dump()
            assert e.value.kind == "ArithmeticError", (trial, dtype, ova.meta, ovb.meta)
            hip.sync()
            continue
        assert got.meta.shape == want.meta.shape
        assert got.dump().tobytes() == want.buf.tobytes(), (trial, dtype, op, ova.meta, ovb.meta)
    hip.sync()                                                             # no fault may be left behind


@pytest.mark.parametrize("dtype", ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64"])
def test_integer_division_faults(hip, dtype):
    """A zero divisor or MIN / -1 inside a tensor: the reference panics (ops/base.rs:27-37), the oracle answers ArithmeticPanic, and the
    backend returns RT_E_ARITH from the next call that waits for the stream -- once -- for every kernel shape of the broadcast
    family; without a fault nothing is reported."""
    from rtensors_amd import hip as H
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 99)
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    signed = npd.kind == "i"
    # (shape of a, shape of b, view of b): contiguous, bias row, column, row kernel, transposed operand, strided generic
    layouts = [([4096], [4096], None), ([64, 256], [256], None), ([64, 256], [64, 1], None), ([8, 16, 1024], [16, 1], None),
               ([128, 256], [256, 128], "T"), ([33, 70], [33, 70], "step2"), ([3, 5, 7], [1], None)]
    for sa, sb, how in layouts:
        for kind in ("zero", "min_neg1", "clean"):
            if kind == "min_neg1" and not signed:
                continue
            va = rng.integers(1, 100, size=int(np.prod(sa))).astype(npd)
            vb = rng.integers(1, 10, size=int(np.prod(sb))).astype(npd)
            ia, ib = int(rng.integers(0, va.size)), int(rng.integers(0, vb.size))
            if kind == "zero":
                vb[ib] = 0
            elif kind == "min_neg1":
                va[:] = np.iinfo(npd).min                                  # wherever the -1 lands, it meets MIN
                vb[ib] = -1
            oa, ob = OTensor.from_buf(dtype, va, sa), OTensor.from_buf(dtype, vb, sb)
            ga, gb = G(hip, dtype, va, sa), G(hip, dtype, vb, sb)
            if how == "T":
                ob, gb = ob.transpose(), gb.transpose()
            elif how == "step2":
                oa, ga = oa.slice(1, Slice(None, None, 2)), ga.slice(1, Slice(None, None, 2))
                ob, gb = ob.slice(1, Slice(None, None, 2)), gb.slice(1, Slice(None, None, 2))
                if kind != "clean" and (ib % 70) % 2 == 1:
                    continue                                               # the planted element is not in the view
            try:
                want = oa / ob
                faulted = False
            except OErr as e:
                assert e.kind == "ArithmeticPanic"
                faulted = True
            assert faulted == (kind != "clean"), (dtype, sa, sb, how, kind)
            got = ga / gb                                                  # enqueued; nothing is known yet
            if faulted:
                with pytest.raises(H.TensorError) as e:
                    hip.sync()
                assert e.value.kind == "ArithmeticError" and e.value.status == 7
                hip.sync()                                                 # reported once, then clear
                out = got.dump()                                           # the other elements are still the quotients
                if kind == "zero" and how is None and sa == sb:
                    ref = np.where(vb == 0, 0, va // np.where(vb == 0, 1, vb)).astype(npd)
                    assert out.tobytes() == ref.tobytes()
            else:
                hip.sync()
                assert got.dump().tobytes() == want.buf.tobytes(), (dtype, sa, sb, how)
    # tensor / scalar: a zero scalar is refused at once; -1 faults only if MIN is present
    v = rng.integers(1, 100, size=1000).astype(npd)
    g = G(hip, dtype, v, [1000])
    with pytest.raises(H.TensorError) as e:
        g /= 0
    assert e.value.kind == "ArithmeticError"
    if signed:
        g /= -1
        hip.sync()
        assert g.dump().tobytes() == (-v).astype(npd).tobytes()
        v[17] = np.iinfo(npd).min
        g = G(hip, dtype, v, [1000])
        g /= -1
        with pytest.raises(H.TensorError) as e:
            g.dump()
        assert e.value.kind == "ArithmeticError"
        hip.sync()


@pytest.mark.parametrize("dtype", ["i8", "u8"])
def test_8_bit_division_every_pair(hip, dtype):
    """1-byte integers are divided through a table of multipliers in LDS (contiguous and long-row kernels) or through the float unit
    (every other kernel).  Every (dividend, divisor) pair through each: the contiguous kernel, the row kernel with the divisors as a
    repeated row, the element kernel (stepped views) and the scalar form; zero divisors and MIN / -1 give 0 / MIN and raise the fault."""
    from rtensors_amd import hip as H
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    info = np.iinfo(npd)
    vals = np.arange(256, dtype=np.uint8).view(npd).astype(np.int64)                   # every value of the type, in byte order

    def trunc_div(a, b):
        return ((np.abs(a) // np.abs(b)) * np.sign(a) * np.sign(b)).astype(npd)
    a = np.repeat(vals, 256); b = np.tile(vals, 256)
    clean = (b != 0) & ~((a == info.min) & (b == -1))
    bc = np.where(clean, b, 1)
    want = trunc_div(a, bc)
    n = a.size
    ga, gb = hip.alloc_from_slice(code, a.astype(npd)), hip.alloc_from_slice(code, bc.astype(npd))
    out = hip.alloc(code, n)
    flat = (0, [n], [1])
    hip.broadcast((ga, flat), (gb, flat), (out, flat), "div")                         # contiguous kernel
    hip.sync()
    assert hip.dump(out).tobytes() == want.tobytes()
    half = (0, [n // 2], [2])
    out2 = hip.alloc(code, n)
    hip.broadcast((ga, half), (gb, half), (out2, half), "div")                        # element kernel
    assert hip.dump(out2)[::2].tobytes() == want[::2].tobytes()
    # rows of 1024 divisors (every value four times) under 64 rows of dividends arranged so that every pair occurs
    cols = np.arange(1024)
    rows = np.arange(64)
    a2 = vals[(rows[:, None] * 4 + cols[None, :] // 256) % 256]
    b2 = vals[cols % 256]
    b2c = np.where(b2 == 0, 1, b2)
    keep = ~((a2 == info.min) & (b2c[None, :] == -1))
    a2c = np.where(keep, a2, 0)
    gra, grb = hip.alloc_from_slice(code, a2c.astype(npd).reshape(-1)), hip.alloc_from_slice(code, b2c.astype(npd))
    out3 = hip.alloc(code, 64 * 1024)
    shape = [64, 1024]
    hip.broadcast((gra, (0, shape, [1024, 1])), (grb, (0, shape, [0, 1])), (out3, (0, shape, [1024, 1])), "div")     # long-row kernel
    hip.sync()
    assert hip.dump(out3).tobytes() == trunc_div(a2c, b2c[None, :]).reshape(-1).tobytes()
    pairs = set(zip(a2c.reshape(-1).tolist(), np.broadcast_to(b2c[None, :], a2c.shape).reshape(-1).tolist()))
    assert len(pairs) >= 256 * 255 - 2
    # the faults: the same operands with their zero divisors (and MIN / -1) left in
    gb0 = hip.alloc_from_slice(code, b.astype(npd))
    hip.broadcast((ga, flat), (gb0, flat), (out, flat), "div")
    with pytest.raises(H.TensorError) as e:
        hip.sync()
    assert e.value.kind == "ArithmeticError"
    got = hip.dump(out)
    ref = np.where(b == 0, 0, trunc_div(a, np.where(b == 0, 1, b)).astype(np.int64)).astype(npd)         # MIN / -1 wraps to MIN
    assert got.tobytes() == ref.tobytes()
    grb0 = hip.alloc_from_slice(code, b2.astype(npd))
    hip.broadcast((gra, (0, shape, [1024, 1])), (grb0, (0, shape, [0, 1])), (out3, (0, shape, [1024, 1])), "div")
    with pytest.raises(H.TensorError):
        hip.sync()
    hip.sync()
    for d in [int(v) for v in vals if v not in (0, -1)][::5]:
        g = G(hip, dtype, vals.astype(npd), [256])
        g /= d
        assert g.dump().tobytes() == trunc_div(vals, np.int64(d)).tobytes(), d


@pytest.mark.parametrize("dtype", ["i16", "u16"])
def test_16_bit_division_every_dividend_and_every_divisor(hip, dtype):
    """Integers of at most 16 bits are divided through the float unit (reciprocal, multiply, truncate).  Every dividend against a
    set of divisors, and every divisor against a set of dividends, must equal the truncating quotient; so must the scalar form.
    (All 2^32 pairs were checked once when the kernel was written; 8-bit types have every pair in test_one_byte_types_every_pair.)"""
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    info = np.iinfo(npd)
    allv = np.arange(info.min, info.max + 1, dtype=np.int64)
    picks = [1, 2, 3, 5, 7, 10, 11, 13, 127, 128, 129, 181, 182, 255, 256, 257, 1000, 4681, 21845, 32766, 32767, info.max, info.max - 1]
    if info.min < 0:
        picks += [-p for p in picks] + [info.min, info.min + 1]
    else:
        picks += [32768, 32769, 43691, 65534]
    picks = np.array(sorted(set(picks)), dtype=np.int64)

    def trunc_div(a, b):
        return ((np.abs(a) // np.abs(b)) * np.sign(a) * np.sign(b)).astype(npd)
    divisors = picks[(picks != 0) & (picks != -1)]
    for av, bv in ((allv, divisors), (picks, allv[(allv != 0) & (allv != -1)])):
        a, b = hip.alloc_from_slice(cpu.DTYPE_BY_NAME[dtype], av.astype(npd)), hip.alloc_from_slice(cpu.DTYPE_BY_NAME[dtype], bv.astype(npd))
        R, C = av.size, bv.size
        out = hip.alloc_uninit(cpu.DTYPE_BY_NAME[dtype], R * C)
        hip.broadcast((a, (0, [R, C], [1, 0])), (b, (0, [R, C], [0, 1])), (out, (0, [R, C], [C, 1])), "div")
        got = hip.dump(out).reshape(R, C)
        want = trunc_div(av[:, None], bv[None, :])
        assert got.tobytes() == want.tobytes(), [(int(av[i]), int(bv[j]), int(got[i, j]), int(want[i, j])) for i, j in np.argwhere(got != want)[:3]]
    keep = allv[allv != info.min] if info.min < 0 else allv
    if info.min < 0:                                       # a divisor of -1 inside a tensor: every dividend but MIN (which faults)
        code = cpu.DTYPE_BY_NAME[dtype]
        a, b = hip.alloc_from_slice(code, keep.astype(npd)), hip.alloc_from_slice(code, np.full(keep.size, -1, dtype=npd))
        out = hip.alloc_uninit(code, keep.size)
        hip.broadcast((a, (0, [keep.size], [1])), (b, (0, [keep.size], [1])), (out, (0, [keep.size], [1])), "div")
        assert hip.dump(out).tobytes() == (-keep).astype(npd).tobytes()
    for d in divisors[::3]:
        g = G(hip, dtype, keep.astype(npd), [keep.size])
        g /= int(d)
        assert g.dump().tobytes() == trunc_div(keep, np.int64(d)).tobytes(), int(d)


@pytest.mark.parametrize("dtype", ["i32", "u32"])
def test_32_bit_division_edge_pairs_and_multiples(hip, dtype):
    """32-bit integers are divided through the f64 unit (reciprocal, one Newton step, multiply, truncate).  What a rounding error
    would break: dividends at and next to multiples of the divisor, quotients near the type's limits, powers of two and their
    neighbours -- all pairs of an edge set, and a million structured pairs, against integer arithmetic."""
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    code = cpu.DTYPE_BY_NAME[dtype]
    info = np.iinfo(npd)
    rng = np.random.default_rng(3232)
    E = {0, 1, 2, 3, 5, 7, 10, info.max, info.max - 1, info.max // 2, info.max // 2 + 1, info.max // 3, 46340, 46341, 65535, 65536, 65537}
    for k in range(1, 33):
        E |= {(1 << k) - 1, 1 << k, (1 << k) + 1}
    if info.min < 0:
        E |= {-e for e in E} | {info.min, info.min + 1}
    E = np.array(sorted(e for e in E if info.min <= e <= info.max), dtype=np.int64)
    A, B = [m.ravel() for m in np.meshgrid(E, E, indexing="ij")]
    m = 1 << 20
    b2 = (rng.integers(0, 1 << 62, size=m, dtype=np.int64) >> (62 - rng.integers(1, 32, size=m))) + 1
    q2 = (rng.random(m) * np.maximum(info.max // b2, 1)).astype(np.int64)
    a2 = q2 * b2 + rng.integers(-1, 2, size=m)
    if info.min < 0:
        a2 *= rng.choice([-1, 1], size=m); b2 *= rng.choice([-1, 1], size=m)
    a, b = np.concatenate([A, a2]), np.concatenate([B, b2])
    keep = (b != 0) & (a >= info.min) & (a <= info.max) & ~((a == info.min) & (b == -1))
    a, b = a[keep], b[keep]
    want = ((np.abs(a) // np.abs(b)) * np.sign(a) * np.sign(b)).astype(npd)
    ga, gb = hip.alloc_from_slice(code, a.astype(npd)), hip.alloc_from_slice(code, b.astype(npd))
    out = hip.alloc_uninit(code, a.size)
    hip.broadcast((ga, (0, [a.size], [1])), (gb, (0, [a.size], [1])), (out, (0, [a.size], [1])), "div")     # vector path
    got = hip.dump(out)
    assert got.tobytes() == want.tobytes(), [(int(a[i]), int(b[i]), int(got[i]), int(want[i])) for i in np.nonzero(got != want)[0][:3]]
    n2 = a.size // 2
    hip.broadcast((ga, (0, [n2], [2])), (gb, (0, [n2], [2])), (out, (0, [n2], [2])), "div")                 # element path
    assert hip.dump(out)[:2 * n2:2].tobytes() == want[:2 * n2:2].tobytes()


@pytest.mark.parametrize("dtype", ["u8", "i8", "i16", "f32", "f64", "bool"])
def test_broadcast_repeated_row_any_length(hip, dtype):
    """(rows, L) op (L,) for row lengths that are not a whole number of 16-byte vectors, so that vectors of the output straddle the
    end of the row (unaligned row loads, the two-load wrap-around, rows shorter than a vector), both operand orders, out of place
    and in place; plus the aligned lengths that take the flat row kernel."""
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 5)
    for L in (1, 2, 3, 5, 7, 15, 16, 17, 31, 33, 100, 250, 1000, 1001, 1024, 4099):
        rows = max(3, 40000 // L)
        va, vb = rand_values(dtype, rows * L, rng), rand_values(dtype, L, rng)
        oa, ob = OTensor.from_buf(dtype, va, [rows, L]), OTensor.from_buf(dtype, vb, [L])
        ga, gb = G(hip, dtype, va, [rows, L]), G(hip, dtype, vb, [L])
        for f in ("__add__", "__sub__", "__mul__"):
            with np.errstate(all="ignore"):
                w1, w2 = getattr(oa, f)(ob), getattr(ob, f)(oa)
            assert getattr(ga, f)(gb).dump().tobytes() == w1.buf.tobytes(), (dtype, L, f, "x op row")
            assert getattr(gb, f)(ga).dump().tobytes() == w2.buf.tobytes(), (dtype, L, f, "row op x")
        with np.errstate(all="ignore"):
            oa += ob
        ga += gb
        assert ga.dump().tobytes() == oa.buf.tobytes(), (dtype, L, "in place")


@pytest.mark.parametrize("dtype", ["f32", "i32", "f64", "u8"])
def test_broadcast_inplace_random(hip, dtype):
    rng = np.random.default_rng(17)
    for trial in range(30):
        rank = int(rng.integers(1, 5))
        shape = [int(rng.integers(1, 9)) for _ in range(rank)]
        if trial % 4 == 0:
            shape[-1] = int(rng.choice([64, 129, 512]))
        sb = [d if rng.random() < 0.6 else 1 for d in shape][int(rng.integers(0, rank)):]
        va, vb = rand_values(dtype, int(np.prod(shape)), rng), rand_values(dtype, int(np.prod(sb)), rng)
        oa, ob = OTensor.from_buf(dtype, va, shape), OTensor.from_buf(dtype, vb, sb)
        ga, gb = G(hip, dtype, va, shape), G(hip, dtype, vb, sb)
        ov = random_view(oa, rng)
        gv = replay(ov, ga)
        try:
            ov += ob
        except OErr:
            with pytest.raises(OErr):
                gv += gb
            continue
        gv += gb
        assert ga.dump().tobytes() == oa.buf.tobytes(), (trial, ov.meta, sb)


@pytest.mark.parametrize("dtype", ["f32", "i16"])
def test_broadcast_row_of_several_mib_repeated(hip, dtype):
    """A row-wise operand of more than 4 MiB per row that repeats along the rows: the row kernel walks bands of rows and groups of
    tiles instead of whole rows (ragged row length, a number of rows that is not a whole number of bands, an outer dim, both operand
    positions, in place).  Checked against numpy: one IEEE / wrapping operation per element."""
    rng = np.random.default_rng(77)
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    L = (4 << 20) // np.dtype(npd).itemsize + 4099
    for rows_shape in ([37], [2, 9]):
        shape = rows_shape + [L]
        n = int(np.prod(shape))
        va, vb = rand_values(dtype, n, rng), rand_values(dtype, L, rng)
        a, b = hip.alloc_from_slice(code, va), hip.alloc_from_slice(code, vb)
        out = hip.alloc_uninit(code, n)
        st = [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
        A, B, O = (a, (0, shape, st)), (b, (0, shape, [0] * len(rows_shape) + [1])), (out, (0, shape, st))
        with np.errstate(all="ignore"):
            hip.broadcast(A, B, O, "sub")
            assert hip.dump(out).tobytes() == (va.reshape(shape) - vb).astype(npd).tobytes(), (dtype, shape, "a - row")
            hip.broadcast(B, A, O, "sub")
            assert hip.dump(out).tobytes() == (vb - va.reshape(shape)).astype(npd).tobytes(), (dtype, shape, "row - a")
            hip.broadcast(A, B, A, "add")
            assert hip.dump(a).tobytes() == (va.reshape(shape) + vb).astype(npd).tobytes(), (dtype, shape, "a += row")


def _tol(dtype, x):
    return {"f32": 1e-5, "f64": 1e-12}[dtype] * float(np.abs(x.astype(np.float64)).sum())


@pytest.mark.parametrize("dtype", ["f32", "u8", "i16", "f64"])
def test_broadcast_long_rows(hip, dtype):
    """Rows of 64 or more 16-byte vectors with every pairing of row-wise and repeated operands (the one-vector-per-lane row kernel):
    ragged row ends, rows cut out of longer rows at odd offsets, one to three outer dims, reversed and stepped outer dims, an operand
    that does not move along an outer dim, in-place accumulation."""
    rng = np.random.default_rng(43)
    per_vec = 16 // np.dtype(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]).itemsize
    L = 66 * per_vec + 3
    def cut(t, cuts):
        for dim, sl in cuts:
            t = t.slice(dim, sl)
        return t
    cases = [
        # (shape of a, cuts of a, shape of b, cuts of b)
        ([7, L], [], [7, L], []),
        ([7, L], [], [L], []),
        ([7, 1], [], [7, L], []),
        ([9, L + 9], [(1, Slice(4, 4 + L, 1))], [L], []),
        ([5, 6, L], [(1, Slice(None, None, -1))], [6, L], []),
        ([5, 6, L], [(0, Slice(0, None, 2))], [3, 6, 1], []),
        ([2, 5, 4, L], [(2, Slice(None, None, -1)), (3, Slice(1, L, 1))], [5, 1, L - 1], []),
        ([2, 1, 4, L], [], [1, 5, 1, L], []),
        ([4, 64 * per_vec], [], [4, 1], []),
        ([6, 128 * per_vec], [(1, Slice(0, 64 * per_vec, 1))], [6, 128 * per_vec], [(1, Slice(64 * per_vec, None, 1))]),
        # dst rows off the 16-byte grid (the in-place leg writes through the view of a): every phase, ragged at both ends
        ([6, L + 5], [(1, Slice(1, 1 + L, 1))], [L], []),
        ([6, L + 5], [(1, Slice(2, 2 + L, 1))], [6, 1], []),
        ([3, 5, L + 4], [(2, Slice(3, 3 + L, 1)), (1, Slice(None, None, -1))], [5, L], []),
        ([8, 130 * per_vec + 1], [(1, Slice(1, None, 1))], [8, 130 * per_vec + 1], [(1, Slice(0, 130 * per_vec, 1))]),
        # five dims that do not merge (the third outer dim is folded into the grid's z)
        ([2, 3, 2, 5, L], [], [1, 3, 1, 5, 1], []),
        ([2, 3, 2, 5, L], [(3, Slice(None, None, -1)), (1, Slice(0, None, 2))], [2, 1, 2, 1, L], []),
        ([3, 1, 2, 1, 64 * per_vec], [], [1, 4, 1, 5, 1], []),
    ]
    for trial, (sa, ca, sb, cb) in enumerate(cases):
        va, vb = rand_values(dtype, int(np.prod(sa)), rng), rand_values(dtype, int(np.prod(sb)), rng)
        for op in ("add", "mul", "sub"):
            oa, ob = OTensor.from_buf(dtype, va, sa), OTensor.from_buf(dtype, vb, sb)
            ga, gb = G(hip, dtype, va, sa), G(hip, dtype, vb, sb)
            ova, ovb, gva, gvb = cut(oa, ca), cut(ob, cb), cut(ga, ca), cut(gb, cb)
            with np.errstate(all="ignore"):
                want = {"add": ova.__add__, "sub": ova.__sub__, "mul": ova.__mul__}[op](ovb)
                got = {"add": gva.__add__, "sub": gva.__sub__, "mul": gva.__mul__}[op](gvb)
                assert got.meta.shape == want.meta.shape
                assert got.dump().tobytes() == want.buf.tobytes(), (trial, dtype, op, "a op b")
                want2 = {"add": ovb.__add__, "sub": ovb.__sub__, "mul": ovb.__mul__}[op](ova)
                got2 = {"add": gvb.__add__, "sub": gvb.__sub__, "mul": gvb.__mul__}[op](gva)
                assert got2.dump().tobytes() == want2.buf.tobytes(), (trial, dtype, op, "b op a")
                if want.meta.shape == ova.meta.shape and all(st != 0 for st in ova.meta.strides):
                    if op == "add":
                        ova += ovb; gva += gvb
                    elif op == "sub":
                        ova -= ovb; gva -= gvb
                    else:
                        ova *= ovb; gva *= gvb
                    assert ga.dump().tobytes() == oa.buf.tobytes(), (trial, dtype, op, "in place")


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "i64", "u8", "i16", "u32"])
@pytest.mark.parametrize("op", ["sum", "prod", "max", "min", "mean"])
def test_reduce_random_vs_oracle(hip, dtype, op):
    rng = np.random.default_rng(zlib.crc32((dtype + op).encode()))
    shapes = [[1], [7], [63], [64], [1000], [70001], [4, 5], [3, 4, 5], [2, 3, 4, 5], [1, 6], [6, 1], [257, 3], [3, 257], [2, 4100],
              [4100, 2], [5, 64, 7], [300, 260], [17, 1024], [2, 1, 3], [33, 40000], [40000, 33], [3, 2048, 8]]
    for shape in shapes:
        x = rand_values(dtype, int(np.prod(shape)), rng, -100, 100)
        if op == "prod" and x.dtype.kind == "f":
            x = (x * 0.05 + 1).astype(x.dtype)
        if op == "mean" and x.dtype.kind != "f" and x.dtype.itemsize < 4:
            continue      # from_usize saturates for narrow ints; covered by test_int_mean_small
        o = OTensor.from_buf(dtype, x, shape)
        g = G(hip, dtype, x, shape)
        for axis in [None] + list(range(len(shape))):
            want = o.reduce(op, axis)
            got = g.reduce(op, axis)
            assert got.meta.shape == want.meta.shape
            a, b = got.dump(), want.buf
            if x.dtype.kind == "f" and op in ("sum", "mean", "prod"):
                if op == "prod":
                    assert np.allclose(a, b, rtol=1e-4 if dtype == "f32" else 1e-11), (shape, axis)
                else:
                    r = 1 if op == "sum" else (o.meta.size() if axis is None else shape[axis])
                    tol = _tol(dtype, x) / r + 1e-30
                    assert np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) <= tol, (dtype, op, shape, axis)
            else:
                assert a.tobytes() == b.tobytes(), (dtype, op, shape, axis)


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32"])
def test_reduce_rows_of_80_to_256_kib_unsplit(hip, dtype):
    """Rows of 80 ... 256 KiB, enough of them that no row is split: the block-per-row kernel with eight loads in flight per lane.
    Row lengths that leave 1 ... 7 vectors and a few elements for the last trip, and a contiguous offset view."""
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 80)
    es = np.dtype(cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]).itemsize
    rows = 2100
    for R in (81920 // es + 3, 98304 // es + 16 * 256 // es * 3 + 1, 131072 // es):
        x = rand_values(dtype, rows * R + 5, rng, -100, 100)
        for offset in (0, 5):
            o = OTensor.from_buf(dtype, x, [rows * R + 5]).slice(0, Slice(offset, offset + rows * R, 1))
            g = G(hip, dtype, x, [rows * R + 5]).slice(0, Slice(offset, offset + rows * R, 1))
            o = OTensor(o.dtype, o.buf, MetaTensor([rows, R], [R, 1], offset), is_view=True)
            g = type(g)(g.backend, g.buf, MetaTensor([rows, R], [R, 1], offset), is_view=True)
            for op in ("sum", "max", "min"):
                want, got = o.reduce(op, 1), g.reduce(op, 1)
                a, b = got.dump(), want.buf
                if x.dtype.kind == "f" and op == "sum":
                    xs = np.abs(x[offset:offset + rows * R].astype(np.float64)).reshape(rows, R).sum(axis=1)
                    tol = (1e-5 if dtype == "f32" else 1e-12) * xs + 1e-30
                    assert (np.abs(a.astype(np.float64) - b.astype(np.float64)).reshape(-1) <= tol).all(), (dtype, op, R, offset)
                else:
                    assert a.tobytes() == b.tobytes(), (dtype, op, R, offset)


def test_reduce_corner_values(hip):
    nan, inf = np.nan, np.inf
    lowest, highest = np.finfo(np.float32).min, np.finfo(np.float32).max
    cases = [([nan, 1.0, nan, 3.0, 2.0], "max", 3.0), ([nan, nan], "max", lowest), ([-inf, -inf], "max", lowest),
             ([inf, nan], "min", highest), ([nan, -2.0, 5.0], "min", -2.0)]
    for vals, op, want in cases:
        g = G(hip, "f32", np.array(vals, np.float32), [len(vals)])
        assert g.reduce(op).dump()[0] == np.float32(want), (vals, op)
    # sign of a zero extremum: the sequential loop keeps the first of equal values (`if value > max`)
    rng = np.random.default_rng(5)
    for n in (2, 64, 1000, 5000, 300000):
        for op in ("max", "min"):
            for first_neg in (True, False):
                x = (-np.abs(rng.standard_normal(n)) - 1).astype(np.float32) if op == "max" else (np.abs(rng.standard_normal(n)) + 1).astype(np.float32)
                i, j = sorted(rng.choice(n, size=2, replace=False))
                x[i], x[j] = (-0.0, 0.0) if first_neg else (0.0, -0.0)
                want = cpu.reduce_flat(cpu.F32, op, x, 0, n)
                got = G(hip, "f32", x, [n]).reduce(op).dump()
                assert got.tobytes() == want.tobytes(), (n, op, first_neg)
                cols = np.stack([x, x[::-1]], axis=1).copy()               # column reduce of the same data
                oc = OTensor.from_buf("f32", cols, [n, 2]).reduce(op, 0)
                gc = G(hip, "f32", cols, [n, 2]).reduce(op, 0)
                assert gc.dump().tobytes() == oc.buf.tobytes(), (n, op, first_neg, "cols")


def test_int_mean_small(hip):
    x = np.arange(1, 13, dtype=np.int32) * 7
    o, g = OTensor.from_buf("i32", x, [3, 4]), G(hip, "i32", x, [3, 4])
    for axis in (None, 0, 1):
        assert g.reduce("mean", axis).dump().tobytes() == o.reduce("mean", axis).buf.tobytes()


def test_reduce_offset_and_errors(hip):
    from rtensors_amd import hip as H
    x = np.arange(24, dtype=np.float64)
    g = hip.alloc_from_slice(H.F64, x)
    out = hip.alloc(H.F64, 2)
    hip.apply_reduce_contiguous_nd((g, (6, [2, 3], [3, 1])), out, 1, "sum")       # offset honoured (backend/cuda.rs:1934)
    assert hip.dump(out).tolist() == cpu.reduce_nd(cpu.F64, "sum", x, MetaTensor([2, 3], [3, 1], 6), 1, honour_offset=True).tolist()
    with pytest.raises(H.TensorError) as e:
        hip.apply_reduce_contiguous_nd((g, (0, [3, 2], [1, 3])), out, 1, "sum")   # non-contiguous source
    assert e.value.kind == "WrongDims"
    with pytest.raises(H.TensorError) as e:
        hip.apply_reduce_contiguous_nd((g, (0, [4, 6], [6, 1])), out, 1, "sum")   # needs 4 outputs, has 2
    assert e.value.kind == "IdxOutOfBounds"
    with pytest.raises(H.TensorError):
        hip.apply_reduce_contiguous_flat(g, out, 20, 5, "sum")
    with pytest.raises(H.TensorError):
        hip.apply_reduce_contiguous_nd((g, (0, [4, 6], [6, 1])), hip.alloc(H.F64, 4), 2, "sum")
    f = hip.alloc_from_slice(H.F32, np.zeros(4, np.float32))
    with pytest.raises(H.TensorError):                                           # not a reduction op code
        lib_status = __import__("rtensors_amd._ffi", fromlist=["lib"]).lib.rt_reduce_flat(hip._ctx, H.F32, 11, f.ptr, 4, f.ptr, 4, 0, 4)
        H._check(lib_status)


def test_bad_descriptors_are_refused_not_launched(hip):
    from rtensors_amd import hip as H
    g = hip.alloc_from_slice(H.F32, np.zeros(100, np.float32))
    for meta in [(0, [101], [1]), (50, [51], [1]), (0, [10, 11], [10, 1]), (5, [3], [-3]), (0, [2 ** 40, 2 ** 40], [1, 1])]:
        with pytest.raises(H.TensorError) as e:
            hip.unary_nd("relu", g, *meta)
        assert e.value.kind in ("IdxOutOfBounds", "InvalidArgument"), meta
    with pytest.raises(H.TensorError):
        hip.fill_nd(g, 1.0, 0, [4, 4], [0, 1])                                   # overlapping writes
    with pytest.raises(H.TensorError):
        hip.broadcast((g, (0, [200], [1])), (g, (0, [200], [0])), (g, (0, [200], [1])), "add")
    hip.unary_nd("relu", g, 100, [0], [1])                                       # empty view at the end: fine
    hip.sync()
    assert not hip.dump(g).any()


def test_device_from_environment(hip, monkeypatch):
    """device -1 asks rt_ctx_create to take the device index from RT_HIP_DEVICE (0 when unset)."""
    from rtensors_amd import hip as H
    monkeypatch.delenv("RT_HIP_DEVICE", raising=False)
    H.Hip(-1).close()
    monkeypatch.setenv("RT_HIP_DEVICE", "0")
    h = H.Hip(-1)
    b = h.alloc_from_slice(H.I32, np.arange(5, dtype=np.int32))
    assert h.dump(b).tolist() == [0, 1, 2, 3, 4]
    del b
    h.close()
    for bad in ("banana", "-2", "3x", "4096"):
        monkeypatch.setenv("RT_HIP_DEVICE", bad)
        with pytest.raises(H.TensorError) as e:
            H.Hip(-1)
        assert e.value.kind == "InvalidArgument", bad


def test_overlapping_source_and_destination_are_refused(hip):
    """An output may be the very same view as an input (the in-place operators); any other overlap of the address ranges would
    let block order decide the result and is refused before a launch.  The trait's `&mut dst` / `&src` pairs
    (backend/mod.rs:228, 303-309) cannot express such calls in the reference either."""
    from rtensors_amd import hip as H
    base = np.arange(64, dtype=np.float32)
    g = hip.alloc_from_slice(H.F32, base)
    other = hip.alloc_from_slice(H.F32, np.ones(64, np.float32))
    row = (0, [32], [1])
    # the same view on both sides: in place, fine -- for the left and for the right operand
    hip.broadcast((g, row), (other, row), (g, row), "add")
    hip.broadcast((other, row), (g, row), (g, row), "mul")
    assert np.array_equal(hip.dump(g)[:32], base[:32] + 1) and np.array_equal(hip.dump(g)[32:], base[32:])
    for bad in [(1, [32], [1]), (31, [32], [-1]), (0, [16], [2])]:
        shape = bad[1]
        dst = (0, shape, [1])
        for left, right in (((g, bad), (other, dst)), ((other, dst), (g, bad))):
            with pytest.raises(H.TensorError) as e:
                hip.broadcast(left, right, (g, dst), "add")
            assert e.value.kind == "InvalidArgument" and "overlaps" in str(e.value), bad
    # disjoint halves of one buffer are fine
    hip.broadcast((g, (32, [32], [1])), (other, row), (g, row), "add")
    assert np.array_equal(hip.dump(g)[:32], base[32:] + 1)
    # copy_range_within: onto itself is a no-op, a shifted overlap is refused, disjoint ranges are copied
    hip.copy_range_within(g, g, 4, 4, 20)
    with pytest.raises(H.TensorError) as e:
        hip.copy_range_within(g, g, 4, 0, 20)
    assert e.value.kind == "InvalidArgument"
    hip.copy_range_within(g, g, 0, 40, 8)
    assert np.array_equal(hip.dump(g)[:8], base[40:48])
    # out-of-place unary / scalar, gather and convert into a range of their own source
    def window(byte_offset, length, dtype):           # a range inside g, not owned: backend None keeps it from being freed
        return H.HipBuf(None, g.ptr + byte_offset, length, dtype)
    sub = window(32, 32, H.F32)
    with pytest.raises(H.TensorError):
        hip.unary_to("relu", g, 0, 16, sub)
    with pytest.raises(H.TensorError):
        hip.scalar_to("add", g, 1.0, 0, 16, sub)
    with pytest.raises(H.TensorError):
        hip.gather(g, (0, [4, 4], [1, 4]), sub)
    with pytest.raises(H.TensorError):
        hip.convert(window(0, 32, H.F32), window(64, 32, H.I32))
    hip.unary_to("relu", g, 0, 8, sub)                # source elements 0..8, destination elements 8..16: disjoint
    assert np.array_equal(hip.dump(g)[8:16], hip.dump(g)[:8])


def test_gather_views(hip):
    rng = np.random.default_rng(6)
    for dtype in ("f32", "u8", "i64", "i16"):
        for trial in range(15):
            rank = int(rng.integers(1, 5))
            shape = [int(rng.integers(1, 20)) for _ in range(rank)]
            vals = rand_values(dtype, int(np.prod(shape)), rng)
            o = OTensor.from_buf(dtype, vals, shape); g = G(hip, dtype, vals, shape)
            ov = random_view(o, rng); gv = replay(ov, g)
            assert gv.to_numpy().tobytes() == ov.to_numpy().tobytes(), (dtype, ov.meta)


@pytest.mark.parametrize("dtype", ["f32", "u8", "i16", "f64"])
def test_gather_transposed_views(hip, dtype):
    """Row-major copy (`owned()` / `contiguous()`) of permuted, reversed and stepped views large enough for the
    LDS-transpose copy kernel, with ragged tile edges."""
    rng = np.random.default_rng(17)
    for shape in [(64, 257), (3, 40, 70), (2, 5, 33, 130), (4, 17, 1030), (100, 36), (2, 3, 16, 16), (7, 300, 9), (48, 2100), (2, 32, 1040), (160, 520),
                  (512, 64), (2, 768, 32), (1024, 256),                      # whole numbers of tiles once transposed
                  (6, 300, 64), (3, 5, 272, 48)]:                            # for the rotations below
        r = len(shape)
        vals = rand_values(dtype, int(np.prod(shape)), rng)
        o, g = OTensor.from_buf(dtype, vals, list(shape)), G(hip, dtype, vals, list(shape))
        perms = [list(range(r - 2)) + [r - 1, r - 2]]
        if r >= 3:
            perms.append([r - 1] + list(range(1, r - 1)) + [0])
            perms.append([r - 1] + list(range(r - 1)))                       # the unit-stride dim becomes the outermost
        if r >= 4:
            perms.append([0, r - 1] + list(range(1, r - 1)))                 # ... or lands between the outer dims
        for perm in perms:
            for variant in range(3):
                ov, gv = o.permute(perm), g.permute(perm)
                if variant == 1:
                    ov, gv = ov.slice(r - 2, Slice(None, None, -1)), gv.slice(r - 2, Slice(None, None, -1))
                if variant == 2:
                    ov, gv = ov.slice(r - 1, Slice(1, None, 2)), gv.slice(r - 1, Slice(1, None, 2))
                assert gv.contiguous().dump().tobytes() == ov.to_numpy().tobytes(), (dtype, shape, perm, variant)


@pytest.mark.parametrize("dtype", ["f32", "u8", "i16", "f64", "i64"])
def test_gather_views_with_short_contiguous_pieces(hip, dtype):
    """Row-major copy of views whose contiguous pieces are short in src, in dst or in both (the N-d tile copy through LDS): permuted
    parents with dims of 2 .. 7 elements next to long ones, dst rows of a few elements, one dim reversed, stepped or cut so that the
    edge tiles are ragged along several dims at once, vector and single-element loads and stores.  Against numpy's own copy of the
    same view, bit for bit."""
    rng = np.random.default_rng(41)
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    dims = (2, 3, 7, 16, 33, 42, 64, 100, 129, 256)
    fixed = [((42, 96, 2, 3, 64), (4, 2, 3, 1, 0)),          # dst rows of 42, src unit-stride along a dim of 64 elsewhere
             ((130, 33, 100, 7), (3, 2, 1, 0)),              # unit-stride dim of 7
             ((2995, 16, 7, 2), (3, 1, 2, 0)),               # the fastest 224 elements of src permuted among themselves
             ((20971, 16, 2), (1, 0, 2)),                    # rows of 2 regrouped
             ((64, 4096, 16), (0, 2, 1)), ((300, 300), (1, 0)), ((1000, 7), (1, 0)), ((7, 1000), (1, 0)), ((33, 5, 16, 9), (2, 0, 3, 1))]
    cases = [(shape, perm, 0) for shape, perm in fixed]
    for trial in range(40):
        rank = int(rng.choice((3, 3, 4, 4, 5)))
        while True:
            shape = tuple(int(rng.choice(dims)) for _ in range(rank))
            if 20000 <= int(np.prod(shape)) <= 400000:
                break
        perm = list(range(rank))
        while perm == sorted(perm):
            rng.shuffle(perm)
        cases.append((shape, tuple(int(x) for x in perm), int(rng.integers(0, 4))))
    for shape, perm, variant in cases:
        vals = rand_values(dtype, int(np.prod(shape)), rng)
        g = G(hip, dtype, vals, list(shape)).permute(list(perm))
        want = vals.reshape(shape).transpose(perm)
        ax = int(rng.integers(0, len(shape)))
        if variant == 1:                                     # one dim reversed
            g, want = g.slice(ax, Slice(None, None, -1)), np.flip(want, ax)
        elif variant == 2:                                   # every second or third index of one dim
            k = int(rng.choice((2, 3)))
            g, want = g.slice(ax, Slice(None, None, k)), want[(slice(None),) * ax + (slice(None, None, k),)]
        elif variant == 3 and want.shape[ax] > 3:            # a corner of the parent
            g, want = g.slice(ax, Slice(1, want.shape[ax] - 2, 1)), want[(slice(None),) * ax + (slice(1, want.shape[ax] - 2),)]
        got = g.contiguous().dump()
        assert got.dtype == npd and got.tobytes() == np.ascontiguousarray(want).tobytes(), (dtype, shape, perm, variant, ax)


@pytest.mark.parametrize("dtype", ["f32", "u8", "i16", "f64"])
def test_gather_interleaved_to_planar(hip, dtype):
    """(.., M, C) -> (.., C, M) with a short C (pixels to planes): the LDS-staged planar copy, with odd plane lengths, a batch
    dim, an offset start, and C at both ends of its range; C = 65 and a strided channel dim go to the general kernels."""
    rng = np.random.default_rng(23)
    for (batch, M, C) in [(1, 1000, 3), (2, 4099, 4), (3, 257, 2), (1, 300, 64), (1, 700, 65), (2, 1 << 15, 3), (1, 5000, 17)]:
        vals = rand_values(dtype, batch * M * C + 5, rng)
        o, g = OTensor.from_buf(dtype, vals, [batch * M * C + 5]), G(hip, dtype, vals, [batch * M * C + 5])
        for start in (0, 5):
            ov = o.slice(0, Slice(start, start + batch * M * C, 1)); gv = g.slice(0, Slice(start, start + batch * M * C, 1))
            ov = OTensor(ov.dtype, ov.buf, MetaTensor([batch, M, C], [M * C, C, 1], start), is_view=True).permute([0, 2, 1])
            gv = type(g)(g.backend, g.buf, MetaTensor([batch, M, C], [M * C, C, 1], start), is_view=True).permute([0, 2, 1])
            assert gv.contiguous().dump().tobytes() == ov.to_numpy().tobytes(), (dtype, batch, M, C, start)
            ov2, gv2 = ov.slice(1, Slice(0, None, 2)), gv.slice(1, Slice(0, None, 2))          # every second channel: not this kernel
            assert gv2.contiguous().dump().tobytes() == ov2.to_numpy().tobytes(), (dtype, batch, M, C, start, "strided")


def test_convert(hip):
    from rtensors_amd import hip as H
    rng = np.random.default_rng(8)
    f = np.array([0.4, 0.5, 1.5, 2.5, -0.5, -1.5, 300.7, -300.2, 1e20, -1e20, np.nan, 127.5, -128.5, 65535.5], dtype=np.float32)
    src = hip.alloc_from_slice(H.F32, f)
    def rust_round_cast(x, info):
        out = []
        for v in x.astype(np.float64):
            if np.isnan(v): out.append(0); continue
            r = np.sign(v) * np.floor(np.abs(v) + 0.5)
            out.append(int(min(max(r, info.min), info.max)))
        return out
    for name in ("u8", "i8", "i16", "u16", "i32", "u32", "i64", "u64"):
        dst = hip.alloc(H.DTYPE_BY_NAME[name], f.size)
        hip.convert(src, dst)
        info = np.iinfo(H.NP_DTYPE[H.DTYPE_BY_NAME[name]])
        assert [int(v) for v in hip.dump(dst)] == rust_round_cast(f, info), name
    i = rng.integers(-70000, 70000, size=1000).astype(np.int32)
    isrc = hip.alloc_from_slice(H.I32, i)
    for name in ("u8", "i8", "i16", "u16", "u32", "i64", "u64", "f32", "f64"):
        dst = hip.alloc(H.DTYPE_BY_NAME[name], i.size)
        hip.convert(isrc, dst)
        with np.errstate(all="ignore"):
            assert hip.dump(dst).tobytes() == i.astype(H.NP_DTYPE[H.DTYPE_BY_NAME[name]]).tobytes(), name   # Rust `as` == C cast
    b = hip.alloc(H.BOOL, i.size); hip.convert(isrc, b)
    assert np.array_equal(hip.dump(b), i != 0)
    with pytest.raises(H.TensorError) as e:
        hip.convert(isrc, hip.alloc(H.F32, 3))
    assert e.value.kind == "SizeMismatch"


def test_convert_128bit_integers(hip):
    """`T::convert::<N>` with u128 / i128 on either side (core/value.rs:255-462): Rust `as` between integers (truncate / extend), round half
    away from zero + saturating cast from floats, correctly rounded casts to floats; checked against Python's exact integers."""
    import struct
    from rtensors_amd import hip as H
    rng = np.random.default_rng(1280)
    M = 1 << 128

    def wrap(v, code):                                                   # Rust `as` to a 128-bit type from any integer
        v %= M
        return v - M if code == cpu.I128 and v >= M >> 1 else v
    ints = [0, 1, -1, 2 ** 63, -2 ** 63, 2 ** 64, 2 ** 64 - 1, 2 ** 127 - 1, -2 ** 127, 2 ** 127, 2 ** 128 - 1, 255, 256, -129, 2 ** 100 + 2 ** 76, 2 ** 100 + 2 ** 76 + 1,
            2 ** 100 + 3 * 2 ** 76, 2 ** 128 - 2 ** 103, 2 ** 128 - 2 ** 103 - 1, 2 ** 120 + 2 ** 66, 2 ** 120 + 2 ** 66 + 1]
    ints += [int(rng.integers(0, 2 ** 63)) * int(rng.integers(0, 2 ** 63)) * int(rng.choice([1, -1])) * int(rng.integers(1, 8)) for _ in range(300)]
    for code in (cpu.U128, cpu.I128):
        vals = [wrap(v, code) for v in ints]
        src = hip.alloc_from_slice(code, cpu.from_ints(code, vals))
        # to the narrower integers and bool: truncation
        for name in ("u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64"):
            dcode = cpu.DTYPE_BY_NAME[name]
            dst = hip.alloc(dcode, len(vals)); hip.convert(src, dst)
            bits = cpu.NP_DTYPE[dcode].itemsize * 8
            want = [(v % (1 << bits)) - ((1 << bits) if name[0] == "i" and (v % (1 << bits)) >= 1 << (bits - 1) else 0) for v in vals]
            assert [int(x) for x in hip.dump(dst)] == want, (code, name)
        dst = hip.alloc(cpu.BOOL, len(vals)); hip.convert(src, dst)
        assert hip.dump(dst).tolist() == [v != 0 for v in vals]
        other = cpu.I128 if code == cpu.U128 else cpu.U128
        dst = hip.alloc(other, len(vals)); hip.convert(src, dst)
        assert cpu.to_ints(other, hip.dump(dst)) == [wrap(v, other) for v in vals]
        # to f64: Python's int -> float is correctly rounded; to f32: nearest of the two neighbours, ties to even, by exact integer arithmetic
        dst = hip.alloc(cpu.F64, len(vals)); hip.convert(src, dst)
        assert hip.dump(dst).tolist() == [float(v) for v in vals], code

        def to_f32(v):
            if v == 0: return 0.0
            sgn, a = (-1 if v < 0 else 1), abs(v)
            e = a.bit_length() - 24
            if e <= 0: return float(v)
            q, r = a >> e, a & ((1 << e) - 1)
            half = 1 << (e - 1)
            if r > half or (r == half and q & 1): q += 1
            f = q << e
            return sgn * (float("inf") if f >= (1 << 128) - (1 << 103) and f.bit_length() > 128 or f >= 1 << 128 else float(f))
        dst = hip.alloc(cpu.F32, len(vals)); hip.convert(src, dst)
        got = hip.dump(dst).astype(np.float64).tolist()
        assert got == [to_f32(v) for v in vals], [(v, g, to_f32(v)) for v, g in zip(vals, got) if g != to_f32(v)][:3]
    # from the other types
    for name in ("u8", "i8", "i16", "u32", "i64", "u64", "bool"):
        scode = cpu.DTYPE_BY_NAME[name]
        x = rand_values(name, 500, rng, -2 ** 62, 2 ** 62)
        if name not in ("bool",):
            info = np.iinfo(x.dtype); x[:2] = [info.min, info.max]
        src = hip.alloc_from_slice(scode, x)
        for code in (cpu.U128, cpu.I128):
            dst = hip.alloc(code, x.size); hip.convert(src, dst)
            assert cpu.to_ints(code, hip.dump(dst)) == [wrap(int(v), code) for v in x], (name, code)
    for fname, npd in (("f32", np.float32), ("f64", np.float64)):
        f = np.concatenate([rng.standard_normal(200) * 10.0 ** rng.integers(0, 39, size=200),
                            [0.0, -0.0, 0.5, -0.5, 1.5, 2.5, -2.5, np.nan, np.inf, -np.inf, 2.0 ** 64, 2.0 ** 64 - 2 ** 12, 2.0 ** 127, -2.0 ** 127, 2.0 ** 126,
                             3.4e38, -3.4e38, 1e30, -1e30, 2.0 ** 63, 2.0 ** 100]]).astype(npd)
        src = hip.alloc_from_slice(cpu.DTYPE_BY_NAME[fname], f)

        def rust_cast(v, code):
            v = float(v)
            if v != v: return 0
            if v in (float("inf"), float("-inf")):
                r = v
            else:
                r = int(np.sign(v)) * int(np.floor(abs(v) + 0.5)) if abs(v) < 2 ** 60 else int(v)     # round half away from zero; large values are integers
            lo, hi = (0, M - 1) if code == cpu.U128 else (-(M >> 1), (M >> 1) - 1)
            if r == float("inf"): return hi
            if r == float("-inf"): return lo
            return min(max(r, lo), hi)
        for code in (cpu.U128, cpu.I128):
            dst = hip.alloc(code, f.size); hip.convert(src, dst)
            got = cpu.to_ints(code, hip.dump(dst))
            want = [rust_cast(v, code) for v in f]
            assert got == want, [(float(v), g, w) for v, g, w in zip(f, got, want) if g != w][:3]


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i16"])
def test_broadcast_with_transposed_operand(hip, dtype):
    """One input is a permuted (and possibly reversed / strided) view whose unit-stride dim is not the output's inner dim:
    the LDS-transpose tile kernel.  Ragged tile edges, both operand positions, broadcast and in-place forms."""
    rng = np.random.default_rng(zlib.crc32(dtype.encode()))
    # the last two shapes are whole numbers of tiles for every element size (the kernel's form without edge tests)
    shapes = [(3, 40, 70), (2, 5, 33, 130), (64, 257), (1, 100, 36), (4, 17, 1030), (2, 3, 16, 16), (48, 2100), (2, 32, 1040), (160, 520),
              (64, 512), (2, 3, 32, 768)]
    for shape in shapes:
        r = len(shape)
        perm = list(range(r)); perm[-1], perm[-2] = perm[-2], perm[-1]
        base_shape = [shape[p] for p in perm]                 # base laid out so that permuting it gives `shape`
        vx = rand_values(dtype, int(np.prod(shape)), rng)
        ox, gx = OTensor.from_buf(dtype, vx, base_shape), G(hip, dtype, vx, base_shape)
        for variant in range(4):
            oxv, gxv = ox.permute(perm), gx.permute(perm)
            if variant & 1:                                    # reverse the dim that is unit-stride in memory
                oxv, gxv = oxv.slice(r - 2, Slice(None, None, -1)), gxv.slice(r - 2, Slice(None, None, -1))
            if variant & 2 and r >= 3:                         # the other operand broadcasts along dim 0
                sy = [1] + list(oxv.meta.shape[1:])
            else:
                sy = list(oxv.meta.shape)
            vy = rand_values(dtype, int(np.prod(sy)), rng)
            oy, gy = OTensor.from_buf(dtype, vy, sy), G(hip, dtype, vy, sy)
            for op in ("add", "sub", "mul"):
                f = {"add": "__add__", "sub": "__sub__", "mul": "__mul__"}[op]
                with np.errstate(all="ignore"):
                    w1, w2 = getattr(oxv, f)(oy), getattr(oy, f)(oxv)
                g1, g2 = getattr(gxv, f)(gy), getattr(gy, f)(gxv)
                assert g1.dump().tobytes() == w1.buf.tobytes(), (dtype, shape, variant, op, "x op y")
                assert g2.dump().tobytes() == w2.buf.tobytes(), (dtype, shape, variant, op, "y op x")
            if variant < 2:                                    # both operands transposed alike (a.transpose() - b.transpose()), and unlike
                vz = rand_values(dtype, int(np.prod(shape)), rng)
                oz, gz = OTensor.from_buf(dtype, vz, base_shape).permute(perm), G(hip, dtype, vz, base_shape).permute(perm)
                ozr, gzr = oz.slice(r - 2, Slice(None, None, -1)), gz.slice(r - 2, Slice(None, None, -1))
                for (o2, g2, what) in ((oz, gz, "forward"), (ozr, gzr, "reversed")):
                    with np.errstate(all="ignore"):
                        w4, w5 = oxv - o2, o2 * oxv
                    assert (gxv - g2).dump().tobytes() == w4.buf.tobytes(), (dtype, shape, variant, "both transposed, second " + what)
                    assert (g2 * gxv).dump().tobytes() == w5.buf.tobytes(), (dtype, shape, variant, "both transposed, second " + what)
            if r <= 3 and variant < 2:                         # the transposed operand itself repeats along a new leading dim
                s3 = [9] + list(oxv.meta.shape)
                v3 = rand_values(dtype, int(np.prod(s3)), rng)
                o3, g3 = OTensor.from_buf(dtype, v3, s3), G(hip, dtype, v3, s3)
                with np.errstate(all="ignore"):
                    w3 = o3 - oxv
                assert (g3 - gxv).dump().tobytes() == w3.buf.tobytes(), (dtype, shape, variant, "repeated transposed operand")
            if sy == list(oxv.meta.shape):                     # in place: y (contiguous) += transposed x
                oy += oxv; gy += gxv
                assert gy.dump().tobytes() == oy.buf.tobytes(), (dtype, shape, variant, "inplace")


def test_128bit_integers(hip):
    """u128 / i128: fill, + - * / (tensor and scalar), relu / abs / neg, leaky_relu, gather, equality (division in depth: test_gpu_int128.py)."""
    from rtensors_amd import hip as H
    rng = np.random.default_rng(128)
    vals_a = [int(rng.integers(-2 ** 62, 2 ** 62)) * int(rng.integers(1, 2 ** 62)) for _ in range(600)]
    vals_b = [int(rng.integers(-2 ** 62, 2 ** 62)) * int(rng.integers(1, 2 ** 40)) for _ in range(600)]
    vals_a[:4] = [2 ** 127 - 1, -2 ** 127, 0, -1]
    for name, code in (("i128", cpu.I128), ("u128", cpu.U128)):
        a, b = cpu.from_ints(code, vals_a), cpu.from_ints(code, vals_b)
        oa, ob = OTensor.from_buf(name, a, [20, 30]), OTensor.from_buf(name, b, [20, 30])
        ga, gb = G(hip, name, a, [20, 30]), G(hip, name, b, [20, 30])
        gv = ga.transpose().slice(0, Slice(None, None, -1)); ov = oa.transpose().slice(0, Slice(None, None, -1))
        for op in ("__add__", "__sub__", "__mul__"):
            assert getattr(ga, op)(gb).dump().tobytes() == getattr(oa, op)(ob).buf.tobytes(), (name, op)
            assert getattr(gv, op)(gb.transpose()).dump().tobytes() == getattr(ov, op)(ob.transpose()).buf.tobytes(), (name, op, "view")
        row = OTensor.from_buf(name, b[:30], [30]); grow = G(hip, name, b[:30], [30])
        assert (ga + grow).dump().tobytes() == (oa + row).buf.tobytes()
        assert gv.to_numpy().tobytes() == ov.to_numpy().tobytes()
        for uop in (("relu", "abs", "neg") if name == "i128" else ("relu", "abs")):
            assert ga.unary(uop).dump().tobytes() == oa.unary(uop).buf.tobytes(), (name, uop)
        o2, g2 = oa.owned(), ga.owned()
        o2 += 12345678901234567890123; g2 += 12345678901234567890123
        o2 *= 3; g2 *= 3
        o2.scalar_op_inplace("leaky_relu", 7); g2.scalar_op_inplace("leaky_relu", 7)
        o2.slice(1, Slice(None, None, 2)).fill(5); g2.slice(1, Slice(None, None, 2)).fill(5)
        assert g2.dump().tobytes() == o2.buf.tobytes()
        assert g2.buf == hip.copy(g2.buf) and not (g2.buf == ga.buf)
        ones = cpu.from_ints(code, [v or 1 for v in vals_b])
        assert (ga / G(hip, name, ones, [20, 30])).dump().tobytes() == (oa / OTensor.from_buf(name, ones, [20, 30])).buf.tobytes()


def test_allocation_failure_is_an_error_not_an_abort(hip):
    from rtensors_amd import hip as H
    with pytest.raises(H.TensorError) as e:
        hip.alloc_uninit(H.F32, 1 << 46)            # 256 TiB
    assert e.value.kind == "HipError"
    b = hip.alloc(H.F32, 16)                        # the context keeps working afterwards
    assert not hip.dump(b).any()


def test_one_context_from_several_threads(hip):
    import threading
    from rtensors_amd import hip as H
    errors = []

    def worker(seed):
        try:
            rng = np.random.default_rng(seed)
            for _ in range(30):
                n = int(rng.integers(1000, 200000))
                x = rng.standard_normal(n).astype(np.float32)
                b = hip.alloc_from_slice(H.F32, x)
                hip.scalar_contiguous("mul", b, 2.0, 0, n)
                hip.unary_contiguous("relu", b, 0, n)
                out = hip.alloc(H.F32, 1)
                hip.apply_reduce_contiguous_flat(b, out, 0, n, "max")
                want = np.maximum(x * np.float32(2.0), 0)
                if hip.dump(b).tobytes() != want.tobytes() or hip.dump(out)[0] != max(want.max(), np.finfo(np.float32).min):
                    errors.append(seed)
        except Exception as ex:          # noqa: BLE001
            errors.append(repr(ex))

    ts = [threading.Thread(target=worker, args=(s,)) for s in range(6)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errors, errors


def test_rank_limits(hip):
    from rtensors_amd import hip as H
    # 12 dims that collapse to one contiguous run: fine
    shape = [2] * 12
    strides = [1 << (11 - i) for i in range(12)]
    x = np.arange(4096, dtype=np.float32) - 2000
    g = hip.alloc_from_slice(H.F32, x)
    hip.unary_nd("relu", g, 0, shape, strides)
    assert np.array_equal(hip.dump(g), np.maximum(x, 0))
    # 10 dims of a (3^10)-buffer, every dim sliced with step 2 (some of them backwards): nothing merges, more than 8 dims remain
    # after collapsing; the reference takes any rank up to 128 (core/primitives.rs:377-383, backend/cpu.rs:292-352)
    rng = np.random.default_rng(77)
    n = 3
    for dtype in ("f32", "i32", "u8", "f64"):
        vals = rand_values(dtype, n ** 10, rng)
        o = OTensor.from_buf(dtype, vals.copy(), [n] * 10)
        g = G(hip, dtype, vals, [n] * 10)
        ov, gv = o.view(), g.view()
        for d in range(10):
            sl = Slice(None, None, -2) if d in (2, 7) else Slice(None, None, 2)
            ov, gv = ov.slice(d, sl), gv.slice(d, sl)
        assert ov.meta.shape == [2] * 10
        # in-place unary, scalar, fill through the view
        ov.unary_inplace("relu"); gv.unary_inplace("relu")
        assert g.dump().tobytes() == o.buf.tobytes(), dtype
        ov += 3; gv += 3
        assert g.dump().tobytes() == o.buf.tobytes(), dtype
        # broadcast against a (2, 1, 2) operand and an owned() gather
        vb = rand_values(dtype, 4, rng)
        ob, gb = OTensor.from_buf(dtype, vb, [2, 1, 2]), G(hip, dtype, vb, [2, 1, 2])
        with np.errstate(all="ignore"):
            want, got = ov + ob, gv + gb
        assert got.meta.shape == want.meta.shape
        assert got.dump().tobytes() == want.buf.tobytes(), dtype
        with np.errstate(all="ignore"):
            ov *= ob; gv *= gb
        assert g.dump().tobytes() == o.buf.tobytes(), dtype
        assert gv.owned().dump().tobytes() == ov.owned().buf.tobytes(), dtype
        ov.fill(7); gv.fill(7)
        assert g.dump().tobytes() == o.buf.tobytes(), dtype
    # rank 0 and empty views
    one = hip.alloc_from_slice(H.F32, np.array([-3.0], np.float32))
    hip.unary_nd("neg", one, 0, [], [])
    assert hip.dump(one)[0] == 3.0
    hip.broadcast((one, (0, [], [])), (one, (0, [], [])), (one, (0, [], [])), "mul")
    assert hip.dump(one)[0] == 9.0
    hip.unary_nd("neg", one, 0, [0, 5], [5, 1])
    hip.broadcast((one, (0, [4, 0], [0, 0])), (one, (0, [4, 0], [0, 0])), (one, (0, [4, 0], [0, 1])), "add")
    out = hip.alloc(H.F32, 1)
    hip.apply_reduce_contiguous_flat(one, out, 0, 0, "sum")           # empty reduction: the accumulator's initial value
    assert hip.dump(out)[0] == 0.0
    hip.apply_reduce_contiguous_flat(one, out, 0, 0, "max")
    assert hip.dump(out)[0] == np.finfo(np.float32).min


def test_more_than_2_31_elements(hip):
    """Views and broadcasts with 2^31 + 2^20 elements take the 64-bit index kernels; u8 keeps the buffers at 2-4 GiB."""
    from rtensors_amd import hip as H
    n = (1 << 31) + (1 << 20)
    a = hip.alloc(H.U8, 2 * n)                    # viewed with stride 2
    hip.fill_contiguous(a, 3, 0, 2 * n)
    hip.fill_1d_strided(a, 7, 1, 2, n)            # odd positions = 7 (1-D strided kernel, > 2^31 elements)
    b = hip.alloc(H.U8, n)
    hip.fill_contiguous(b, 10, 0, n)
    hip.fill_nd(b, 20, 0, [n // 2, 1], [2, 1])    # even positions = 20
    d = hip.alloc(H.U8, n)
    # d[i] = a[2i + 1] + b[i]: left operand strided -> generic 64-bit kernel
    hip.broadcast((a, (1, [n], [2])), (b, (0, [n], [1])), (d, (0, [n], [1])), "add")
    host = hip.dump(d)
    want = np.full(n, 17, dtype=np.uint8); want[0::2] = 27
    assert np.array_equal(host, want)
    del host, want
    # N-d view over 2^31+ elements that is not one run: rows of 2^20 with a gap after each
    rows, cols = n // (1 << 20), 1 << 20
    hip.unary_nd("relu", a, 0, [rows, cols - 1], [cols, 1])
    # contiguous path, 2-D in-place binary over everything, then a device-side reduction as checksum
    hip.broadcast((d, (0, [n], [1])), (b, (0, [n], [1])), (d, (0, [n], [1])), "sub")
    out = hip.alloc(H.U8, 1)
    hip.apply_reduce_contiguous_flat(d, out, 0, n, "max")
    assert hip.dump(out)[0] == 7
    hip.apply_reduce_contiguous_flat(d, out, 0, n, "min")
    assert hip.dump(out)[0] == 7
    # positions beyond 2^31 come back whole from the index reductions
    p_max, p_min = (1 << 31) + 12345, (1 << 31) + 77
    hip.write(d, p_max, 9); hip.write(d, p_max + 5, 9); hip.write(d, p_min, 2)
    idx = hip.alloc(H.U64, rows)
    hip.apply_argmax_contiguous_flat(d, idx, 0, n, "argmax")
    assert int(hip.dump(idx)[0]) == p_max
    hip.apply_argmax_contiguous_flat(d, idx, 0, n, "argmin")
    assert int(hip.dump(idx)[0]) == p_min
    hip.apply_argmax_contiguous_nd((d, (0, [rows, cols], [cols, 1])), idx, 1, "argmax")
    got = hip.dump(idx)
    assert int(got[p_max // cols]) == p_max % cols and int(got.sum()) == p_max % cols
    # an N-d broadcast and an N-d in-place op over 2^31+ elements: issued as slices along the outer dim (2047 rows, then 2), each
    # through the 32-bit kernels; rows on both sides of the cut and at both ends are held to numpy
    del a, idx
    yv = (np.arange(cols) % 5).astype(np.uint8)
    y = hip.alloc_from_slice(H.U8, yv)
    z = hip.alloc_uninit(H.U8, n)
    full = (0, [rows, cols], [cols, 1])
    hip.broadcast((d, full), (y, (0, [rows, cols], [0, 1])), (z, full), "add")
    hip.scalar_nd("add", z, 1, 0, [rows, cols - 1], [cols, 1])          # every row but its last column
    row_x, row_z = hip.alloc_uninit(H.U8, cols), hip.alloc_uninit(H.U8, cols)
    for r in (0, 1, 2046, 2047, 2048, rows - 1, p_max // cols):
        hip.copy_range_within(row_x, d, 0, r * cols, cols)
        hip.copy_range_within(row_z, z, 0, r * cols, cols)
        want = hip.dump(row_x) + yv
        want[:-1] += 1
        assert np.array_equal(hip.dump(row_z), want), r
    hip.sync()


def _check_reduce(hip, dtype, outer, R, inner, rng, offset=0):
    """All five ops over (outer, R, inner) along the middle axis, against the oracle (which folds in index order)."""
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    n = outer * R * inner
    x = rand_values(dtype, n + offset, rng, -50, 50)
    if dtype[0] == "f" and n >= 8:
        x[offset:offset + 4] = [0.0, -0.0, np.nan, -0.0]
        x[offset + n - 2:offset + n] = [-0.0, 0.0]
    src = hip.alloc_from_slice(code, x)
    shape = [outer, R, inner]
    m = MetaTensor(shape, [R * inner, inner, 1], offset)
    ops = ("sum", "max", "min", "mean", "prod") if dtype[0] == "f" else ("sum", "max", "min")
    for op in ops:
        with np.errstate(all="ignore"):
            want = cpu.reduce_nd(code, op, x, m, 1, honour_offset=True)
        dst = hip.alloc(code, outer * inner)
        hip.apply_reduce_contiguous_nd((src, (offset, shape, [R * inner, inner, 1])), dst, 1, op)
        got = hip.dump(dst)
        if dtype[0] != "f" or op in ("max", "min"):
            assert got.tobytes() == want.tobytes(), (dtype, op, outer, R, inner, offset)
        elif op == "prod":
            ok = np.isclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-4 if dtype == "f32" else 1e-10, atol=0, equal_nan=True)
            assert ok.all() or R > 64, (dtype, op, outer, R, inner)
        else:
            rel = 1e-5 if dtype == "f32" else 1e-12
            v = np.nan_to_num(np.abs(x[offset:offset + n].astype(np.float64))).reshape(outer, R, inner).sum(axis=1).reshape(-1)
            scale = v / (R if op == "mean" else 1)
            fin = np.isfinite(want.astype(np.float64))
            assert (np.isnan(got) == np.isnan(want)).all(), (dtype, op, outer, R, inner)
            assert (np.abs(got.astype(np.float64) - want.astype(np.float64))[fin] <= rel * scale[fin] + 1e-300).all(), (dtype, op, outer, R, inner)


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i64"])
def test_reduction_shapes_short_rows_narrow_columns_short_axis(hip, dtype):
    """The shapes that have kernels of their own: rows of 1..1025 elements (LDS-tiled), narrow inner dims (streamed with the
    lanes pinned to columns), reduced axes of at most 32 elements (a lane per output); odd counts, unaligned offsets, and the
    hand-over points to the general kernels."""
    rng = np.random.default_rng(zlib.crc32(dtype.encode()))
    for R in (1, 2, 3, 7, 8, 31, 32, 33, 63, 64, 65, 100, 255, 256, 1000, 1023, 1024, 1025):
        for rows in (1, 77, 1000):
            _check_reduce(hip, dtype, rows, R, 1, rng, offset=int(rng.integers(0, 5)))
    # many short rows of a power-of-two number of 16-byte vectors: the kernel without staging (aligned and unaligned starts)
    for R in (2, 4, 8, 16, 32, 64, 128, 256, 512, 1024):
        for offset in (0, 4, 16, 3):
            _check_reduce(hip, dtype, 70000 if R <= 64 else 5000, R, 1, rng, offset=offset)
    for inner in (2, 3, 4, 5, 17, 64, 100, 127, 128):
        for R, outer in ((64, 3), (1000, 1), (5003, 2), (70001, 1)):
            _check_reduce(hip, dtype, outer, R, inner, rng, offset=int(rng.integers(0, 5)))
    for R in (1, 2, 4, 5, 16, 31, 32, 33):
        for inner, outer in ((2, 1000), (3, 1), (64, 50), (100, 7), (1024, 3), (1028, 2), (5, 9), (7, 3), (257, 4), (1001, 2), (19, 40)):
            _check_reduce(hip, dtype, outer, R, inner, rng, offset=int(rng.integers(0, 5)))
    # wide rows whose length is not a multiple of the 16-byte vector (and starts that are not aligned): every lane still loads
    # whole vectors, the last one overlapping its neighbour
    for outer, R, inner in ((2, 300, 257), (1, 5003, 1001), (3, 100, 129), (1, 2000, 1030), (1, 70, 4099), (2, 40, 131)):
        for offset in (0, 1, 3):
            _check_reduce(hip, dtype, outer, R, inner, rng, offset=offset)
    # many small slabs with a few columns (staged through LDS, a group of lanes per column); a short axis over ragged rows
    for outer, R, inner in ((3000, 33, 2), (5000, 17, 5), (2000, 100, 3), (1500, 8, 32), (1100, 33, 60), (4000, 2, 2), (1024, 300, 2), (1030, 1000, 2), (1200, 5, 17),
                            (500, 3, 257), (100, 1, 4097), (50, 2, 4097), (700, 17, 257), (40, 3, 30001)):
        _check_reduce(hip, dtype, outer, R, inner, rng, offset=int(rng.integers(0, 5)))


@pytest.mark.parametrize("dtype", ["f32", "i32", "u8", "f64"])
def test_broadcast_short_rows_under_short_loop_dims(hip, dtype):
    """Outputs whose rows are a few elements long, with operands that repeat along different dims: the shapes on which a block of
    the row kernel would be left with a couple of short rows, and which the flat kernel takes instead (dst one aligned run, inputs
    gathered by index).  Against numpy's broadcasting, bit for bit, for add, mul and sub in either operand order."""
    from rtensors_amd import hip as H
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    rng = np.random.default_rng(zlib.crc32(b"short-rows" + dtype.encode()))
    pairs = [((50, 1, 2, 17), (1, 7, 1, 17)), ((300, 5, 3, 3), (300, 1, 3, 3)), ((40, 100, 1, 17), (40, 100, 3, 1)), ((200, 2, 1, 17), (200, 1, 1, 17)),
             ((9, 257, 1, 17), (9, 1, 1, 17)), ((33, 17, 17, 2), (33, 1, 17, 2)), ((60, 3, 100, 1), (1, 1, 1, 17)), ((700, 1, 1, 17), (700, 1, 17, 1)),
             ((1000, 3, 2, 5), (1000, 1, 2, 5)), ((5, 1, 257, 3), (1, 11, 1, 3)), ((123, 1, 5, 31), (1, 4, 1, 31)), ((64, 2, 2, 8), (64, 1, 2, 1))]
    for sa, sb in pairs:
        a = rand_values(dtype, int(np.prod(sa)), rng, -50, 50).reshape(sa)
        b = rand_values(dtype, int(np.prod(sb)), rng, -50, 50).reshape(sb)
        out_shape = [max(x, y) for x, y in zip(sa, sb)]
        n = int(np.prod(out_shape))

        def strides(shape):
            st, acc = [], 1
            for d, od in zip(reversed(shape), reversed(out_shape)):
                st.append(0 if d == 1 and od != 1 else acc)
                acc *= d
            return list(reversed(st))
        ga, gb, gd = hip.alloc_from_slice(code, a.reshape(-1)), hip.alloc_from_slice(code, b.reshape(-1)), hip.alloc(code, n)
        dst_meta = (0, out_shape, strides(out_shape))
        for op, fn in (("add", np.add), ("mul", np.multiply), ("sub", np.subtract)):
            for (x, gx, sx), (y, gy, sy) in (((a, ga, sa), (b, gb, sb)), ((b, gb, sb), (a, ga, sa))):
                hip.broadcast((gx, (0, out_shape, strides(sx))), (gy, (0, out_shape, strides(sy))), (gd, dst_meta), op)
                with np.errstate(all="ignore"):
                    want = fn(x, y).astype(npd)
                assert hip.dump(gd).tobytes() == np.ascontiguousarray(want).tobytes(), (dtype, op, sx, sy)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_float_max_min_keep_the_first_zero_in_every_kernel_shape(hip, dtype):
    """max over values <= 0 and min over values >= 0 whose zeros come in both signs, in either order, or in one sign only: the
    result is the first zero of the fiber in index order, as in the sequential loop, whichever kernel folds it (a block, a wave
    or a group of lanes per row, rows of whole vectors, split rows and the flat form; lanes along wide, narrow and regrouped
    columns, a lane per output for a short axis).  NaN never wins."""
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = np.dtype(cpu.NP_DTYPE[code]).type
    rng = np.random.default_rng(zlib.crc32(b"zero-sign" + dtype.encode()))
    shapes = [(4, 100000, 1), (3000, 5000, 1), (1, 1 << 21, 1), (5000, 600, 1), (3000, 2000, 1), (20000, 100, 1), (20000, 10, 1), (40000, 64, 1),
              (8192, 256, 1), (70, 33, 1), (1, 5000, 512), (8, 300, 1024), (1, 4096, 4096), (2, 3000, 1001), (1, 100000, 3), (4, 5000, 100),
              (5000, 16, 64), (100, 8, 1000), (1, 70001, 17), (300, 200, 8), (1, 70000, 128), (1, 65536, 256), (1, 30000, 1000), (1, 70001, 128),
              (3000, 33, 2), (5000, 17, 5), (2000, 100, 3), (1100, 33, 60), (1024, 300, 2), (500, 3, 257), (50, 2, 4097)]
    for outer, R, inner in shapes:
        n = outer * R * inner
        mag = np.abs(rng.normal(size=n)).astype(npd) + npd(0.5)
        # per fiber: 0 = no zero, 1 = +0.0 only, 2 = -0.0 only, 3 = both signs; zeros at random places along the fiber
        kind = rng.integers(0, 4, size=(outer, 1, inner))
        u = rng.random(size=(outer, R, inner))
        zero = (u < min(0.5, 3.0 / R)) & (kind > 0)
        neg = np.where(kind == 3, rng.random(size=(outer, R, inner)) < 0.5, kind == 2)
        zeros = np.where(neg, npd(-0.0), npd(0.0)).astype(npd)
        nan = rng.random(size=(outer, R, inner)) < 0.01
        for op, sign in (("max", -1), ("min", 1)):
            x = np.where(zero, zeros, (sign * mag).reshape(outer, R, inner)).astype(npd)
            x[nan & ~zero] = np.nan
            x = np.ascontiguousarray(x).reshape(-1)
            m = MetaTensor([outer, R, inner], [R * inner, inner, 1], 0)
            want = cpu.reduce_nd(code, op, x, m, 1, honour_offset=True)
            src = hip.alloc_from_slice(code, x)
            dst = hip.alloc(code, outer * inner)
            hip.apply_reduce_contiguous_nd((src, (0, [outer, R, inner], [R * inner, inner, 1])), dst, 1, op)
            got = hip.dump(dst)
            assert got.tobytes() == want.tobytes(), (dtype, op, outer, R, inner, int(np.flatnonzero(got.view(np.uint8) != want.view(np.uint8))[0]))
            if outer * inner >= 64:
                assert np.signbit(want[want == 0]).any() and (~np.signbit(want[want == 0])).any(), "the case is meant to hold zero results of both signs"
            if inner == 1 and outer == 1:
                one = hip.alloc(code, 1)
                hip.apply_reduce_contiguous_flat(src, one, 0, n, op)
                assert hip.dump(one).tobytes() == want.tobytes(), (dtype, op, "flat", n)


def _check_stat(hip, dtype, outer, R, inner, rng, offset=0):
    """Variance / stdev / logsumexp / norms along the middle axis of (outer, R, inner).  The GPU folds in tree order, the oracle in
    index order, so the comparison is by tolerance: within 1e-5 (f32) / 1e-12 (f64), relative, of the oracle run in float64 on the
    same values (for f64 that is the oracle itself)."""
    code = cpu.DTYPE_BY_NAME[dtype]
    n = outer * R * inner
    x = (rng.normal(size=n + offset) * 3 + 10).astype(cpu.NP_DTYPE[code])
    src = hip.alloc_from_slice(code, x)
    shape, strides = [outer, R, inner], [R * inner, inner, 1]
    m = MetaTensor(shape, strides, offset)
    x64 = x.astype(np.float64)
    rel = 1e-5 if dtype == "f32" else 1e-12
    for op in cpu.STAT_OPS:
        with np.errstate(all="ignore"):
            want = cpu.reduce_stat(cpu.F64, op, x64, m, 1)
        dst = hip.alloc(code, outer * inner)
        hip.apply_reduce_contiguous_nd((src, (offset, shape, strides)), dst, 1, op)
        got = hip.dump(dst).astype(np.float64)
        assert (np.isnan(got) == np.isnan(want)).all(), (dtype, op, outer, R, inner)
        fin = np.isfinite(want)
        tol = rel * np.abs(want)
        if op in ("var", "pop_var", "std", "pop_std"):
            # a variance is conditioned by kappa = sqrt(1 + mean^2 / var): two samples 1e-3 apart around 10 lose four digits in any
            # arithmetic, the oracle's included
            xs = x64[offset:offset + n].reshape(outer, R, inner)
            with np.errstate(all="ignore"):
                kappa = np.sqrt(1 + xs.mean(axis=1) ** 2 / xs.var(axis=1)).reshape(-1)
            tol = tol * np.where(np.isfinite(kappa), kappa, 1.0)
        assert (np.abs(got - want)[fin] <= tol[fin] + 1e-300).all(), (dtype, op, outer, R, inner, offset, got[:4], want[:4])


def _check_arg(hip, dtype, outer, R, inner, rng, offset=0):
    """argmax / argmin: exact.  Values from a small set so that ties are everywhere; floats also carry NaN."""
    code = cpu.DTYPE_BY_NAME[dtype]
    n = outer * R * inner
    if dtype[0] == "f":
        x = np.round(rng.normal(size=n + offset) * 2).astype(cpu.NP_DTYPE[code])
        x[rng.integers(0, n + offset, size=max(1, (n + offset) // 50))] = np.nan
    else:
        lo = 0 if dtype[0] == "u" else -5
        x = rng.integers(lo, lo + 11, size=n + offset).astype(cpu.NP_DTYPE[code])
    src = hip.alloc_from_slice(code, x)
    shape, strides = [outer, R, inner], [R * inner, inner, 1]
    m = MetaTensor(shape, strides, offset)
    for op in cpu.ARG_OPS:
        want = cpu.argmax(code, op, x, m, 1)
        dst = hip.alloc(cpu.U64, outer * inner)
        hip.apply_argmax_contiguous_nd((src, (offset, shape, strides)), dst, 1, op)
        got = hip.dump(dst)
        assert got.tolist() == want.tolist(), (dtype, op, outer, R, inner, offset)


STAT_SHAPES = ([(rows, R, 1) for R in (1, 2, 3, 7, 8, 31, 32, 33, 64, 65, 100, 255, 256, 1000, 1024, 1025, 2000, 4095) for rows in (1, 77, 1500)]
               + [(3, 70001, 1), (1, 300000, 1), (1100, 4100, 1)]
               + [(30000, R, 1) for R in (1, 2, 4, 8, 16, 32, 64)]
               + [(outer, R, inner) for inner in (2, 3, 5, 17, 63, 64, 100, 128) for R, outer in ((64, 3), (1000, 1), (5003, 2), (70001, 1))]
               + [(outer, R, inner) for R in (1, 2, 5, 16, 33) for inner, outer in ((2, 1000), (3, 1), (64, 50), (1028, 2))]
               + [(1, 65536, 256), (1, 30000, 1000), (1, 8192, 2048)]                  # rows regrouped before the column kernel reads them
               # many small slabs with a few columns (staged through LDS); a short axis over ragged rows (vectors that overlap at a row's end)
               + [(3000, 33, 2), (5000, 17, 5), (2000, 100, 3), (1500, 8, 32), (1100, 33, 60), (4000, 2, 2), (1024, 300, 2), (1030, 1000, 2), (1200, 5, 17)]
               + [(500, 3, 257), (100, 1, 4097), (50, 2, 4097), (700, 17, 257), (40, 3, 30001)]
               + [(1, 300, 5000), (2, 4000, 260), (1, 70, 2052), (2, 300, 257), (1, 5003, 1001), (3, 100, 129), (1, 2000, 1030), (1, 70, 4099), (2, 40, 131)])


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_statistic_reductions_shapes(hip, dtype):
    rng = np.random.default_rng(zlib.crc32(dtype.encode()))
    for outer, R, inner in STAT_SHAPES:
        _check_stat(hip, dtype, outer, R, inner, rng, offset=int(rng.integers(0, 5)))
    for R in (2, 4, 8, 16):                                       # aligned starts reach the kernel without staging
        _check_stat(hip, dtype, 30000, R, 1, rng, offset=0)
        _check_stat(hip, dtype, 30000, R, 1, rng, offset=8)
    # unsplit rows of 80 ... 256 KiB: eight loads in flight per lane for the variance and norm states
    es = 4 if dtype == "f32" else 8
    _check_stat(hip, dtype, 2100, 81920 // es + 3, 1, rng, offset=3)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_logsumexp_results_near_zero(hip, dtype):
    """Runs whose logsumexp is close to 0 (R values around -ln R, and mixed-sign pairs): the result is the sum of two terms of
    opposite sign, max + log(sum exp(x - max)), so its error is relative to the larger of |result| and |largest element|, not to
    |result| -- the bound the C header states.  (f32 uses the hardware exponential: |error| is about 5e-8 here, which a bound
    relative to a result of 1e-4 would not admit.)"""
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 11)
    rel = 1e-5 if dtype == "f32" else 1e-12
    for outer, R, inner in [(20000, 2, 1), (20000, 3, 1), (4000, 10, 1), (300, 1000, 1), (1, 2, 5000), (7, 64, 33), (1, 5000, 3)]:
        n = outer * R * inner
        for centre in (-np.log(R), 0.0):
            x = (centre + rng.normal(size=n) * (1e-3 if centre else 1.0)).astype(npd)
            if centre == 0.0:
                x[::2] = -np.abs(x[::2])                                   # mixed signs
            src = hip.alloc_from_slice(code, x)
            dst = hip.alloc(code, outer * inner)
            shape, strides = [outer, R, inner], [R * inner, inner, 1]
            hip.apply_reduce_contiguous_nd((src, (0, shape, strides)), dst, 1, "logsumexp")
            got = hip.dump(dst).astype(np.float64)
            xs = x.astype(np.float64).reshape(outer, R, inner)
            want = np.logaddexp.reduce(xs, axis=1).reshape(-1)
            scale = np.maximum(np.abs(want), np.abs(xs).max(axis=1).reshape(-1))
            assert (np.abs(got - want) <= rel * scale).all(), (dtype, outer, R, inner, centre, np.abs(got - want).max())
            if centre:
                assert np.abs(want).max() < 0.05                          # these results really are near zero


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i64", "i16"])
def test_argmax_argmin_shapes(hip, dtype):
    rng = np.random.default_rng(zlib.crc32(dtype.encode()))
    for outer, R, inner in STAT_SHAPES:
        _check_arg(hip, dtype, outer, R, inner, rng, offset=int(rng.integers(0, 5)))
    for R in (2, 4, 8, 16, 32, 64):
        _check_arg(hip, dtype, 30000, R, 1, rng, offset=0)
        _check_arg(hip, dtype, 30000, R, 1, rng, offset=16)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_logsumexp_special_values_in_every_kernel_shape(hip, dtype):
    """Fibers that hold NaN, +inf, -inf, nothing but -inf, or values 800 apart (terms that underflow), through every work shape: a NaN
    anywhere gives NaN, else a +inf gives +inf, a fiber of -inf gives -inf, and the rest agree with the float64 formula."""
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = np.dtype(cpu.NP_DTYPE[code]).type
    rng = np.random.default_rng(zlib.crc32(b"lse-special" + dtype.encode()))
    shapes = [(4, 100000, 1), (3000, 5000, 1), (1, 1 << 20, 1), (5000, 600, 1), (20000, 100, 1), (20000, 10, 1), (40000, 64, 1), (8192, 256, 1),
              (40000, 4, 1), (70, 33, 1), (1, 5000, 512), (8, 300, 1024), (1, 4096, 2048), (1, 100000, 3), (4, 5000, 100), (5000, 16, 64), (300, 200, 8),
              (3000, 33, 2), (5000, 17, 5), (2000, 100, 3), (1100, 33, 60), (1024, 300, 2), (500, 3, 257), (50, 2, 4097)]
    for outer, R, inner in shapes:
        x = (rng.normal(size=(outer, R, inner)) * 3).astype(npd)
        x[rng.random(size=x.shape) < 0.02] -= npd(800.0)
        kind = rng.integers(0, 6, size=(outer, 1, inner))          # 0, 1: plain; 2: NaN; 3: +inf; 4: -inf among the values; 5: nothing but -inf
        hit = rng.random(size=x.shape) < min(0.5, 2.0 / R)
        hit[:, :1, :] |= rng.random(size=(outer, 1, inner)) < 0.5   # often in the first element, where a state starts
        hit[:, -1:, :] |= rng.random(size=(outer, 1, inner)) < 0.5
        x = np.where(hit & (kind == 2), npd(np.nan), x)
        x = np.where(hit & (kind == 3), npd(np.inf), x)
        x = np.where(hit & (kind == 4), npd(-np.inf), x)
        x = np.where(np.broadcast_to(kind == 5, x.shape), npd(-np.inf), x).astype(npd)
        x64 = x.astype(np.float64)
        with np.errstate(all="ignore"):
            top = np.nanmax(np.where(np.isnan(x64), -np.inf, x64), axis=1, keepdims=True)
            safe = np.where(np.isfinite(top), top, 0.0)
            want = (safe + np.log(np.exp(x64 - safe).sum(axis=1, keepdims=True))).reshape(-1)
        has_nan = np.isnan(x64).any(axis=1).reshape(-1)
        has_pinf = (x64 == np.inf).any(axis=1).reshape(-1)
        all_ninf = (x64 == -np.inf).all(axis=1).reshape(-1)
        src = hip.alloc_from_slice(code, np.ascontiguousarray(x).reshape(-1))
        dst = hip.alloc(code, outer * inner)
        hip.apply_reduce_contiguous_nd((src, (0, [outer, R, inner], [R * inner, inner, 1])), dst, 1, "logsumexp")
        got = hip.dump(dst).astype(np.float64)
        case = (dtype, outer, R, inner)
        assert (np.isnan(got) == has_nan).all(), (case, "NaN", int(np.flatnonzero(np.isnan(got) != has_nan)[0]))
        assert (got[has_pinf & ~has_nan] == np.inf).all(), (case, "+inf")
        assert (got[all_ninf] == -np.inf).all(), (case, "-inf")
        plain = ~has_nan & ~has_pinf & ~all_ninf
        assert np.isfinite(got[plain]).all(), case
        tol = (1e-5 if dtype == "f32" else 1e-12) * np.maximum(np.abs(want[plain]), 1.0)
        assert (np.abs(got[plain] - want[plain]) <= tol).all(), (case, float(np.abs(got[plain] - want[plain]).max()))
        if inner == 1 and outer == 1:
            one = hip.alloc(code, 1)
            hip.apply_reduce_contiguous_flat(src, one, 0, R, "logsumexp")
            g1 = float(hip.dump(one)[0])
            assert (np.isnan(g1) and has_nan[0]) or g1 == got[0] or abs(g1 - want[0]) <= 1e-5 * max(abs(want[0]), 1.0), (case, "flat", g1)


def test_statistic_reductions_known_answers_and_edges(hip):
    """The reference's Cuda known answers through the C ABI, the flat entry points, and the edge cases the oracle tests pin."""
    import json
    from rtensors_amd import hip as H
    cases = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_reduce_stat_vectors.json")))["cases"]
    for c in cases:
        code = cpu.DTYPE_BY_NAME[c["dtype"]]
        x = np.array(c["data"], dtype=cpu.NP_DTYPE[code])
        src = hip.alloc_from_slice(code, x)
        shape = c["shape"]
        strides = [shape[1], 1]
        arg = c["op"] in cpu.ARG_OPS
        nout = 1 if c["dim"] is None else int(np.prod(shape)) // shape[c["dim"]]
        dst = hip.alloc(cpu.U64 if arg else code, nout)
        if c["dim"] is None:
            (hip.apply_argmax_contiguous_flat if arg else hip.apply_reduce_contiguous_flat)(src, dst, 0, x.size, c["op"])
        else:
            (hip.apply_argmax_contiguous_nd if arg else hip.apply_reduce_contiguous_nd)((src, (0, shape, strides)), dst, c["dim"], c["op"])
        got = hip.dump(dst)
        if arg:
            assert got.tolist() == c["want"], c
        else:
            assert np.allclose(got.astype(np.float64), c["want"], rtol=1e-6 if c["dtype"] == "f32" else 1e-14, atol=0), (c, got)
    nan, inf = float("nan"), float("inf")

    def flat(dtype, op, values, start=0, length=None):
        code = cpu.DTYPE_BY_NAME[dtype]
        x = np.array(values, dtype=cpu.NP_DTYPE[code])
        src = hip.alloc_from_slice(code, x) if x.size else hip.alloc(code, 1)
        arg = op in cpu.ARG_OPS
        dst = hip.alloc(cpu.U64 if arg else code, 1)
        (hip.apply_argmax_contiguous_flat if arg else hip.apply_reduce_contiguous_flat)(src, dst, start, x.size - start if length is None else length, op)
        return hip.dump(dst)[0]
    assert flat("f64", "argmax", [1, 5, 5, 2]) == 1 and flat("f64", "argmin", [3, 1, 1, 2]) == 1
    assert flat("f64", "argmax", [nan, 2, nan, 7, 7]) == 3 and flat("f64", "argmax", [nan, nan]) == 0 and flat("f64", "argmax", [-inf, -inf]) == 0
    assert flat("f32", "argmin", [inf, 4, -inf, -inf]) == 2
    assert flat("f64", "argmax", [9, 1, 5, 5, 2], start=1) == 1                 # positions count from `start`
    assert flat("i32", "argmax", [3, -7, 9, 9, 0]) == 2 and flat("u8", "argmin", [3, 0, 9, 0]) == 1
    assert flat("f64", "logsumexp", [-inf, -inf]) == -inf and flat("f64", "logsumexp", [1.0, inf, 2.0]) == inf
    assert np.isnan(flat("f64", "logsumexp", [1.0, nan]))
    assert flat("f64", "logsumexp", [], length=0) == -inf and flat("f64", "argmax", [], length=0) == 0 and flat("f64", "l2_norm", [], length=0) == 0
    assert np.isclose(flat("f64", "logsumexp", [1000.0, 1000.0]), 1000.0 + np.log(2.0), rtol=1e-15)
    assert np.isclose(flat("f32", "logsumexp", [-1000.0, -1001.0]), -1000.0 + np.log1p(np.exp(-1.0)), rtol=1e-6)
    assert flat("f64", "pop_var", [4.0]) == 0.0 and np.isnan(flat("f64", "var", [4.0]))
    assert np.isclose(flat("f64", "var", [1e9, 1e9 + 1, 1e9 + 2]), 1.0, rtol=1e-12)
    big = 1e9 + np.arange(100001, dtype=np.float64) % 3                            # a large common offset must not cancel
    assert np.isclose(flat("f64", "pop_var", big), big.var(), rtol=1e-11)
    # what the entry points refuse
    f = hip.alloc_from_slice(H.F32, np.arange(8, dtype=np.float32))
    i = hip.alloc_from_slice(H.I32, np.arange(8, dtype=np.int32))
    o32, o64 = hip.alloc(H.F32, 8), hip.alloc(H.U64, 8)
    with pytest.raises(H.TensorError) as e:
        hip.apply_reduce_contiguous_flat(f, o32, 0, 8, "argmax")                   # kinds are not swapped between entry points
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(H.TensorError) as e:
        hip.apply_argmax_contiguous_flat(f, o64, 0, 8, "sum")
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(H.TensorError) as e:
        hip.apply_reduce_contiguous_flat(i, hip.alloc(H.I32, 1), 0, 8, "var")       # WeightValue kinds on an integer
    assert e.value.kind == "UnsupportedOperation"
    lib = __import__("rtensors_amd._ffi", fromlist=["lib"]).lib
    for bad in (8, 8 | 0x300, 7 | 0x100, 6 | 0x400, 11, 0):
        with pytest.raises(H.TensorError):
            H._check(lib.rt_reduce_flat(hip._ctx, H.F32, bad, f.ptr, 8, o32.ptr, 8, 0, 8))
    with pytest.raises(H.TensorError) as e:
        hip.apply_argmax_contiguous_nd((f, (0, [2, 4], [1, 2])), o64, 0, "argmax")
    assert e.value.kind == "WrongDims"
    with pytest.raises(H.TensorError) as e:
        hip.apply_argmax_contiguous_nd((f, (0, [2, 4], [4, 1])), hip.alloc(H.U64, 3), 0, "argmax")
    assert e.value.kind == "IdxOutOfBounds"
    hip.sync()


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i64"])
def test_out_of_place_unary_and_scalar(hip, dtype):
    """rt_unary_to / rt_scalar_to: one pass from a contiguous run into a fresh buffer must equal clone + in-place op
    (ops/unary/mod.rs:114-126, ops/scalar/add.rs:93-97), leave the source untouched, and refuse what the in-place forms refuse."""
    from rtensors_amd import hip as H
    rng = np.random.default_rng(31)
    code = cpu.DTYPE_BY_NAME[dtype]
    n = 70_001
    x = rand_values(dtype, n, rng)
    src = hip.alloc_from_slice(code, x)
    unary_ops = ["relu", "abs", "neg", "square", "sign", "step", "sigmoid"] if dtype[0] == "f" else (["relu", "abs", "step"] + (["neg"] if dtype[0] == "i" else []))
    scalar_ops = {"add": 3, "sub": 7, "mul": 3, "div": 3, "leaky_relu": 2, "leaky_grad": 2}
    for start, length in ((0, n), (4, n - 9), (5, 1000), (n - 3, 3), (16, 0)):
        m = MetaTensor([length], [1], start)
        for op in unary_ops:
            if op in ("step",):
                with np.errstate(invalid="ignore"):
                    want = np.where(x[start:start + length] > 0, 1, 0).astype(x.dtype)
            else:
                full = x.copy()
                with np.errstate(all="ignore"):
                    cpu.unary(code, op, full, m)
                want = full[start:start + length]
            dst = hip.alloc(code, max(length, 1) + 2)
            hip.unary_to(op, src, start, length, dst)
            got = hip.dump(dst)
            if op == "sigmoid":
                assert np.allclose(got[:length], want, rtol=1e-5, atol=1e-5)
            else:
                assert got[:length].tobytes() == want.tobytes(), (op, start, length)
            assert not got[length:].any()                                    # nothing written past the run
        for op, v in scalar_ops.items():
            full = x.copy()
            with np.errstate(all="ignore"):
                cpu.scalar(code, op, full, v, m)
            dst = hip.alloc(code, max(length, 1))
            hip.scalar_to(op, src, v, start, length, dst)
            assert hip.dump(dst)[:length].tobytes() == full[start:start + length].tobytes(), (op, start, length)
    assert hip.dump(src).tobytes() == x.tobytes()                            # the source is only read
    small = hip.alloc(code, 10)
    for bad in (lambda: hip.unary_to("relu", src, 0, 11, small), lambda: hip.unary_to("relu", src, n - 5, 6, small),
                lambda: hip.unary_to("relu", src, 0, n, src), lambda: hip.scalar_to("add", src, 1, 0, 11, small)):
        with pytest.raises(H.TensorError):
            bad()
    if dtype[0] != "f":
        with pytest.raises(H.TensorError):
            hip.unary_to("sigmoid", src, 0, 10, small)                        # bounded on f32/f64 in the reference
        with pytest.raises(H.TensorError):
            hip.scalar_to("div", src, 0, 0, 10, small)                       # integer / 0 scalar


# ---- matmul (BackendMatMul::matmul, backend/mod.rs:474-485) --------------------------------------------------------------------------
MM_SHAPES = [(1, 1, 1, 1), (1, 5, 7, 3), (3, 64, 64, 64), (2, 70, 33, 129), (1, 130, 16, 65), (4, 1, 40, 1), (1, 2, 1, 200)]


def _mm_operand(make, dtype, rng, b, rows, cols, layout, lo=-1000, hi=1000):
    """An operand of logical shape (b, rows, cols) [or (rows, cols) when b == 1 and layout is even] in one of four layouts:
    0 row-major contiguous, 1 row-major rows of a wider matrix at an offset, 2 column-major (transposed base),
    3 column-major with a padded leading dim.  Returns what `make(values, shape)` gives, viewed accordingly."""
    if layout == 0:
        return make(rand_values(dtype, b * rows * cols, rng, lo, hi), [b, rows, cols])
    if layout == 1:
        t = make(rand_values(dtype, b * (rows + 2) * (cols + 5), rng, lo, hi), [b, rows + 2, cols + 5])
        return t.slice(1, Slice(1, rows + 1, 1)).slice(2, Slice(3, cols + 3, 1))
    if layout == 2:
        return make(rand_values(dtype, b * rows * cols, rng, lo, hi), [b, cols, rows]).permute([0, 2, 1])
    t = make(rand_values(dtype, b * (cols + 1) * (rows + 3), rng, lo, hi), [b, cols + 1, rows + 3])
    return t.slice(1, Slice(0, cols, 1)).slice(2, Slice(2, rows + 2, 1)).permute([0, 2, 1])


@pytest.mark.parametrize("dtype", ["i32", "u8", "i64", "i16", "u32", "bool"])
def test_matmul_integers_bit_exact(hip, dtype):
    """The tiled kernel against the Cpu backend's triple loop (backend/cpu.rs:857-939): wrapping sums, every pairing of
    row-/column-major operands (the reference itself has mixed pairings for f32/f64 only), padded leading dims, offsets,
    batches, ragged tiles."""
    seed = zlib.crc32(dtype.encode())
    lo, hi = (-2 ** 31, 2 ** 31 - 1) if dtype in ("i64", "u32", "i32") else (-1000, 1000)      # products overflow and wrap
    for (b, m, k, n) in MM_SHAPES:
        for ll in range(4):
            for rl in range(4):
                r1, r2 = np.random.default_rng(seed), np.random.default_rng(seed)
                ol = _mm_operand(lambda v, s: OTensor.from_buf(dtype, v, s), dtype, r1, b, m, k, ll, lo, hi)
                orr = _mm_operand(lambda v, s: OTensor.from_buf(dtype, v, s), dtype, r1, b, k, n, rl, lo, hi)
                gl = _mm_operand(lambda v, s: G(hip, dtype, v, s), dtype, r2, b, m, k, ll, lo, hi)
                gr = _mm_operand(lambda v, s: G(hip, dtype, v, s), dtype, r2, b, k, n, rl, lo, hi)
                with np.errstate(all="ignore"):
                    want = ol.matmul(orr)
                got = gl.matmul(gr)
                assert list(got.meta.shape) == list(want.meta.shape) == [b, m, n]
                assert got.dump().tobytes() == want.buf.tobytes(), (dtype, (b, m, k, n), ll, rl)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_matmul_floats_within_tolerance(hip, dtype):
    """rocBLAS gemm against the textbook dot product in ascending k.  The reference's own f32/f64 path is OpenBLAS, whose
    summation order is not specified, so bit parity is unpinned; the bound is rel * sum_k |a_ik * b_kj| with rel = 1e-5 (f32)
    / 1e-12 (f64), and the result is cross-checked against numpy in f64."""
    rel = 1e-5 if dtype == "f32" else 1e-12
    seed = 99
    for (b, m, k, n) in MM_SHAPES + [(2, 300, 517, 260)]:
        for ll in range(4):
            for rl in range(4):
                if (b, m, k, n) == (2, 300, 517, 260) and (ll, rl) not in ((0, 0), (1, 3), (2, 1), (3, 2)):
                    continue
                r1, r2 = np.random.default_rng(seed), np.random.default_rng(seed)
                ol = _mm_operand(lambda v, s: OTensor.from_buf(dtype, v, s), dtype, r1, b, m, k, ll)
                orr = _mm_operand(lambda v, s: OTensor.from_buf(dtype, v, s), dtype, r1, b, k, n, rl)
                gl = _mm_operand(lambda v, s: G(hip, dtype, v, s), dtype, r2, b, m, k, ll)
                gr = _mm_operand(lambda v, s: G(hip, dtype, v, s), dtype, r2, b, k, n, rl)
                want = ol.matmul(orr).buf.reshape(b, m, n).astype(np.float64)
                got = gl.matmul(gr).dump().reshape(b, m, n).astype(np.float64)
                A, B = ol.to_numpy().astype(np.float64), orr.to_numpy().astype(np.float64)
                bound = rel * (np.abs(A) @ np.abs(B)) + 1e-300
                assert (np.abs(got - want) <= bound).all(), (dtype, (b, m, k, n), ll, rl, np.abs(got - want).max())
                assert (np.abs(got - A @ B) <= bound).all(), (dtype, (b, m, k, n), ll, rl)


def test_matmul_128_bit_and_rank2(hip):
    vals_a, vals_b = [2 ** 100 + 7, 3, 5, 2 ** 64 + 1, 11, 13], [1, 2 ** 90, 3, 4, 2 ** 127 - 1, 6]
    for name in ("u128", "i128"):
        oa, ob = OTensor.from_buf(name, vals_a, [2, 3]), OTensor.from_buf(name, vals_b, [3, 2])
        ga, gb = G(hip, name, cpu.from_ints(cpu.DTYPE_BY_NAME[name], vals_a), [2, 3]), G(hip, name, cpu.from_ints(cpu.DTYPE_BY_NAME[name], vals_b), [3, 2])
        assert ga.matmul(gb).dump().tobytes() == oa.matmul(ob).buf.tobytes()
        assert ga.matmul(ga.transpose()).dump().tobytes() == oa.matmul(oa.transpose()).buf.tobytes()
    x, y = np.arange(1, 6, dtype=np.float32), np.arange(2, 7, dtype=np.float32)
    gx, gy = G(hip, "f32", x, [5]), G(hip, "f32", y, [5])
    assert gx.dot(gy).dump().tolist() == [float(x @ y)] and gx.dot(gy).meta.shape == []
    assert gx.outer(gy).dump().tobytes() == np.outer(x, y).astype(np.float32).tobytes()


def test_matmul_descriptor_checks(hip):
    """backend/remote/server.rs:299-334, 605-636: a bad operand is an error code, never a launch."""
    from rtensors_amd import hip as H
    a = hip.alloc_from_slice(H.F32, np.arange(12, dtype=np.float32))
    b = hip.alloc_from_slice(H.F32, np.arange(12, dtype=np.float32))
    d = hip.alloc(H.F32, 16)
    ok_l, ok_r = (a, (0, [3, 4], [4, 1]), "row_major"), (b, (0, [4, 3], [3, 1]), "row_major")
    hip.matmul(ok_l, ok_r, d, 1, 3, 4, 3)
    want = (np.arange(12, dtype=np.float32).reshape(3, 4) @ np.arange(12, dtype=np.float32).reshape(4, 3)).reshape(-1)
    assert hip.dump(d)[:9].tolist() == want.tolist()
    bad = [
        ((a, (0, [3, 4], [4, 1]), "row_major"), (b, (0, [4, 3], [3, 1]), "row_major"), a, (1, 3, 4, 3), "alias"),
        ((a, (0, [3, 4], [4, 1]), "column_major"), ok_r, d, (1, 3, 4, 3), "layout code does not match strides"),
        ((a, (0, [3, 4], [4, 1]), "none"), ok_r, d, (1, 3, 4, 3), "layout none"),
        ((a, (11, [3, 4], [-4, 1]), "row_major"), ok_r, d, (1, 3, 4, 3), "negative stride"),
        ((a, (1, [3, 4], [4, 1]), "row_major"), ok_r, d, (1, 3, 4, 3), "extent past the end"),
        ((a, (0, [3, 4], [4, 1]), "row_major"), ok_r, d, (1, 3, 4, 4), "shape does not match m, k, n"),
        ((a, (0, [1, 3, 4], [12, 4, 1]), "row_major"), ok_r, d, (1, 3, 4, 3), "rank mismatch"),
        ((a, (0, [3, 4], [4, 1]), "row_major"), ok_r, hip.alloc(H.F32, 8), (1, 3, 4, 3), "dst too small"),
        ((a, (0, [2, 1, 3, 2], [6, 3, 2, 1]), "row_major"), (b, (0, [2, 1, 2, 3], [3, 6, 3, 1]), "row_major"), d, (2, 3, 2, 3), "batch dims not collapsible"),
    ]
    for l, r, dst, (bb, m, k, n), why in bad:
        with pytest.raises(H.TensorError):
            hip.matmul(l, r, dst, bb, m, k, n)
    # k == 0: empty sums
    hip.fill_contiguous(d, 7.0, 0, 16)
    hip.matmul((a, (0, [3, 0], [0, 1]), "row_major"), (b, (0, [0, 3], [3, 1]), "row_major"), d, 1, 3, 0, 3)
    assert hip.dump(d).tolist() == [0.0] * 9 + [7.0] * 7


@pytest.mark.parametrize("dtype", ["f32", "f64", "i16", "u8", "i32", "i64", "u32"])
def test_broadcast_with_a_permuted_operand_of_short_pieces(hip, dtype):
    """`a op b.permute(..)` where the permuted operand's contiguous pieces are short (a unit-stride dim of a few elements, or dst rows of
    a few elements) and large enough for the two-pass form: the operand is copied into a row-major temporary by the N-d tile copy and
    the op runs on the temporary.  Either operand order, in place, with a reversed dim, into a dst that is itself a view; add, sub, mul
    and (integers) a division with the fault for a zero divisor.  Against numpy on the same view, bit for bit."""
    code = cpu.DTYPE_BY_NAME[dtype]
    npd = cpu.NP_DTYPE[code]
    rng = np.random.default_rng(zlib.crc32(b"permuted-operand" + dtype.encode()))
    cases = [((42, 96, 2, 3, 64), (4, 2, 3, 1, 0)), ((130, 33, 100, 7), (3, 2, 1, 0)), ((2995, 16, 7, 2), (3, 1, 2, 0)), ((20971, 16, 2), (1, 0, 2)),
             ((33, 50, 16, 9, 4), (2, 0, 4, 3, 1)), ((1000, 7, 100), (1, 2, 0))]
    es = np.dtype(npd).itemsize
    for shape, perm in cases:
        n = int(np.prod(shape))
        assert n * es >= 256 << 10
        parent = rand_values(dtype, n, rng, 1, 60).reshape(shape)           # no zeros: the divisions below are defined
        view = parent.transpose(perm)
        out_shape = list(view.shape)
        vst = [int(x) // es for x in view.strides]
        other = rand_values(dtype, n, rng, 1, 60).reshape(out_shape)
        row_major = [int(x) // es for x in other.strides]
        gp, go, gd = hip.alloc_from_slice(code, parent.reshape(-1)), hip.alloc_from_slice(code, other.reshape(-1)), hip.alloc(code, n)
        ops = [("add", np.add), ("sub", np.subtract), ("mul", np.multiply)]
        if npd.kind in "iu":
            ops.append(("div", lambda x, y: (np.trunc(x.astype(np.float64) / y.astype(np.float64))).astype(npd)))
        else:
            ops.append(("div", np.divide))
        for op, fn in ops:
            for view_is_left in (True, False):
                l = (gp, (0, out_shape, vst)) if view_is_left else (go, (0, out_shape, row_major))
                r = (go, (0, out_shape, row_major)) if view_is_left else (gp, (0, out_shape, vst))
                hip.broadcast(l, r, (gd, (0, out_shape, row_major)), op)
                with np.errstate(all="ignore"):
                    want = fn(view, other) if view_is_left else fn(other, view)
                assert hip.dump(gd).tobytes() == np.ascontiguousarray(want.astype(npd)).tobytes(), (dtype, shape, perm, op, view_is_left)
        # in place: other op= view, then with the view's last dim reversed
        hip.broadcast((go, (0, out_shape, row_major)), (gp, (0, out_shape, vst)), (go, (0, out_shape, row_major)), "add")
        with np.errstate(all="ignore"):
            acc = np.add(other, view).astype(npd)
        assert hip.dump(go).tobytes() == np.ascontiguousarray(acc).tobytes(), (dtype, shape, perm, "in place")
        rst = list(vst); rst[-1] = -rst[-1]
        hip.broadcast((go, (0, out_shape, row_major)), (gp, ((out_shape[-1] - 1) * vst[-1], out_shape, rst)), (go, (0, out_shape, row_major)), "sub")
        with np.errstate(all="ignore"):
            acc = np.subtract(acc, np.flip(view, -1)).astype(npd)
        assert hip.dump(go).tobytes() == np.ascontiguousarray(acc).tobytes(), (dtype, shape, perm, "in place, reversed")
    if npd.kind in "iu":
        # a zero divisor inside the permuted operand: the fault the reference panics with, reported by the next call that waits
        shape, perm = cases[0]
        n = int(np.prod(shape))
        parent = rand_values(dtype, n, rng, 1, 60).reshape(shape)
        parent.reshape(-1)[n // 3] = 0
        view = parent.transpose(perm)
        out_shape = list(view.shape)
        vst = [int(x) // es for x in view.strides]
        other = rand_values(dtype, n, rng, 1, 60).reshape(out_shape)
        row_major = [int(x) // es for x in other.strides]
        gp, go, gd = hip.alloc_from_slice(code, parent.reshape(-1)), hip.alloc_from_slice(code, other.reshape(-1)), hip.alloc(code, n)
        hip.broadcast((go, (0, out_shape, row_major)), (gp, (0, out_shape, vst)), (gd, (0, out_shape, row_major)), "div")
        from rtensors_amd import hip as H
        with pytest.raises(H.TensorError) as e:
            hip.sync()
        assert e.value.kind == "ArithmeticError"
        hip.sync()                                                         # reported once, then clear
