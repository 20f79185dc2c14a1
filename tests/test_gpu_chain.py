"""rt_fused_chain (a program of elementwise steps in one pass) against the sequence of separate backend calls it replaces: the
oracle's in-place loops step by step (backend/cpu.rs:485-724, ops/base.rs:27-37), bit for bit for every exact op and every integer
type; exp / sigmoid / silu / tanh bit for bit against the device's own separate kernels and within the reference's 1e-5 of the
oracle.  Random programs over random operand phases and lengths, in place and out of place, the error paths, and the config-2
expression `c = relu(a * 3 + b); c -= 1` at full size."""
import zlib

import numpy as np
import pytest

from oracle import cpu
from oracle.meta import MetaTensor

pytestmark = pytest.mark.gpu

FLOATS = ("f32", "f64")
UNARY_ALL = ["relu", "abs", "step"]
UNARY_SIGNED = ["neg", "abs_grad"]
UNARY_FLOAT_EXACT = ["sqrt", "floor", "ceil", "round", "trunc", "rsqrt", "reciprocal", "square", "cube", "sign"]
UNARY_FLOAT_TOL = ["exp", "sigmoid", "silu", "tanh"]
SCALAR_ALL = ["add", "sub", "mul", "leaky_relu", "leaky_grad"]
BINARY_ALL = ["add", "sub", "mul"]


@pytest.fixture(scope="module")
def hip():
    from rtensors_amd import hip as H
    b = H.Hip.new(0)
    yield b
    b.sync()


def rand_values(dtype, n, rng):
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    if npd.kind == "f":
        x = (rng.standard_normal(n) * 1.5).astype(npd)
        if n >= 8:
            x[:8] = [0.0, -0.0, np.nan, np.inf, -np.inf, np.finfo(npd).tiny / 4, -1.0, 2.5]
        return x
    info = np.iinfo(npd)
    x = rng.integers(max(info.min, -1000), min(info.max, 1000) + 1, size=n, dtype=np.int64).astype(npd)
    if n >= 4:
        x[:4] = [info.min, info.max, 0, 1]
    return x


def same_bits(got, want):
    """Bit for bit, except that a NaN only has to be a NaN: the sign and payload of a NaN that an operation creates (inf - inf,
    0 * inf, sqrt(-1)) differ between the host's and the device's arithmetic units and carry no meaning in the reference either."""
    if got.dtype.kind != "f":
        return got.tobytes() == want.tobytes()
    nan = np.isnan(got) & np.isnan(want)
    bits = got.view(np.uint32 if got.dtype == np.float32 else np.uint64) == want.view(np.uint32 if want.dtype == np.float32 else np.uint64)
    return bool(np.all(nan | bits))


def oracle_step(code, acc, step, inputs):
    """One step of the program on the host, through the oracle's own loops."""
    n = acc.size
    m = MetaTensor([n], [1], 0)
    kind = step[0]
    with np.errstate(all="ignore"):
        if kind == "unary":
            if step[1] in ("step", "abs_grad"):                              # the two gradient maps have no loop in the Cpu backend
                one, lo = acc.dtype.type(1), acc.dtype.type(0 if step[1] == "step" else -1)
                acc[:] = np.where(acc > 0, one, lo)
            else:
                cpu.unary(code, step[1], acc, m)
        elif kind == "scalar":
            cpu.scalar(code, step[1], acc, step[2], m)
        else:
            other = inputs[step[2]].copy()
            out = np.zeros(n, dtype=acc.dtype)
            l, r = (acc, other) if kind == "binary" else (other, acc)
            cpu.broadcast(code, step[1], l.copy(), m, r, m, out, m)
            acc[:] = out
    return acc


def device_sequence(hip, code, acc_buf, step, input_bufs, n):
    """The same step as one separate backend call on the device (in place on acc_buf)."""
    kind = step[0]
    m = (0, [n], [1])
    if kind == "unary":
        hip.unary_contiguous(step[1], acc_buf, 0, n)
    elif kind == "scalar":
        hip.scalar_contiguous(step[1], acc_buf, step[2], 0, n)
    elif kind == "binary":
        hip.broadcast((acc_buf, m), (input_bufs[step[2]], m), (acc_buf, m), step[1])
    else:
        out = hip.alloc_uninit(code, n)
        hip.broadcast((input_bufs[step[2]], m), (acc_buf, m), (out, m), step[1])
        hip.copy_range_within(acc_buf, out, 0, 0, n)


def random_program(dtype, rng, n_inputs):
    npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
    flt, signed = npd.kind == "f", npd.kind in "fi"
    unary = UNARY_ALL + (UNARY_SIGNED if signed else []) + (UNARY_FLOAT_EXACT if flt else [])
    scalar = SCALAR_ALL + (["div"] if flt else [])
    binary = BINARY_ALL + (["div"] if flt else [])
    steps = []
    for _ in range(int(rng.integers(1, 9))):
        k = rng.random()
        if k < 0.35:
            steps.append(("unary", str(rng.choice(unary))))
        elif k < 0.7:
            v = float(rng.choice([3.0, -0.5, 1.0, 0.1, 2.0])) if flt else int(rng.choice([3, 1, 2, 7] + ([-3] if signed else [])))
            steps.append(("scalar", str(rng.choice(scalar)), v))
        else:
            steps.append((str(rng.choice(["binary", "binary_rev"])), str(rng.choice(binary)), int(rng.integers(0, n_inputs))))
    return steps


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i8", "i16", "u16", "u32", "i64", "u64"])
def test_random_chains_match_the_separate_ops(hip, dtype):
    code = cpu.DTYPE_BY_NAME[dtype]
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 17)
    for trial in range(40):
        n_inputs = int(rng.integers(1, 5))
        n = int(rng.choice([1, 2, 3, 15, 17, 100, 255, 1000, 4099, 70_001]))
        pad = 40
        hosts = [rand_values(dtype, n + pad, rng) for _ in range(n_inputs)]
        starts = [int(rng.integers(0, pad)) for _ in range(n_inputs)]
        steps = random_program(dtype, rng, n_inputs)
        ins = [h[s:s + n].copy() for h, s in zip(hosts, starts)]
        want = ins[0].copy()
        for st in steps:
            want = oracle_step(code, want, st, ins)
        bufs = [hip.alloc_from_slice(code, h) for h in hosts]
        in_place = trial % 3 == 0
        if in_place:
            k = int(rng.integers(0, n_inputs))
            hip.fused_chain(list(zip(bufs, starts)), steps, bufs[k], n, starts[k])
            got_all = hip.dump(bufs[k])
            expect_all = hosts[k].copy(); expect_all[starts[k]:starts[k] + n] = want
        else:
            dst_host = rand_values(dtype, n + pad, rng)
            dst = hip.alloc_from_slice(code, dst_host)
            ds = int(rng.integers(0, pad))
            hip.fused_chain(list(zip(bufs, starts)), steps, dst, n, ds)
            got_all = hip.dump(dst)
            expect_all = dst_host.copy(); expect_all[ds:ds + n] = want
            for b, h in zip(bufs, hosts):
                assert hip.dump(b).tobytes() == h.tobytes()                      # inputs are only read
        assert same_bits(got_all, expect_all), (dtype, trial, n, starts, steps)


@pytest.mark.parametrize("dtype", FLOATS)
def test_chain_transcendental_steps(hip, dtype):
    """exp / sigmoid / silu / tanh inside a chain: the same device routine as the separate kernel (bit for bit), and within the
    reference's own 1e-5 of the oracle."""
    code = cpu.DTYPE_BY_NAME[dtype]
    rng = np.random.default_rng(5)
    n = 50_003
    a, b = rand_values(dtype, n, rng), rand_values(dtype, n, rng)
    for op in UNARY_FLOAT_TOL:
        steps = [("scalar", "mul", 0.5), ("binary", "add", 1), ("unary", op), ("scalar", "sub", 1.0)]
        ga, gb = hip.alloc_from_slice(code, a), hip.alloc_from_slice(code, b)
        out = hip.alloc(code, n)
        hip.fused_chain([(ga, 0), (gb, 0)], steps, out, n)
        seq = hip.copy(ga)
        want = a.copy()
        for st in steps:
            device_sequence(hip, code, seq, st, [ga, gb], n)
            want = oracle_step(code, want, st, [a, b])
        got = hip.dump(out)
        assert got.tobytes() == hip.dump(seq).tobytes(), op
        ok = np.isclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-5, atol=1e-5, equal_nan=True)
        assert ok.all(), (op, got[~ok][:4], want[~ok][:4])


def test_chain_refusals(hip):
    from rtensors_amd import hip as H
    a = hip.alloc(H.I32, 100); b = hip.alloc(H.I32, 100); f = hip.alloc(H.F32, 100); bo = hip.alloc(H.BOOL, 100)
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 0), (b, 0)], [("binary", "div", 1)], a, 100)              # integer division reports faults per launch
    assert e.value.kind == "UnsupportedOperation"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 0)], [("unary", "sqrt")], a, 100)                         # float-only op
    assert e.value.kind == "UnsupportedOperation"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(f, 0)], [("unary", "ln")], f, 100)                           # ALU-bound op: not in a chain
    assert e.value.kind == "UnsupportedOperation"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(bo, 0)], [("unary", "relu")], bo, 100)
    assert e.value.kind == "UnsupportedOperation"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 0), (b, 0)], [("binary", "add", 2)], a, 100)              # names an input that is not there
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 0), (b, 0)], [("binary", "add", 1)], a, 90, 5)            # dst overlaps input 0 at another start
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 20), (b, 0)], [("binary", "add", 1)], b, 90, 0)           # input 0 runs past its buffer
    assert e.value.kind == "IdxOutOfBounds"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 0)], [("unary", "relu")] * 9, b, 100)
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(H.TensorError) as e:
        hip.fused_chain([(a, 0)] * 5, [("unary", "relu")], b, 100)
    assert e.value.kind == "InvalidArgument"
    hip.fused_chain([(a, 0)], [("unary", "relu")], b, 0)                               # nothing to do is fine
    hip.sync()


def test_config2_expression_in_one_pass_full_size(hip):
    """c = relu(a * 3 + b) - 1 at 2^28 f32 (2^27 f64, 2^28 i32) as one chain: every element equals the four separate kernels'
    result (compared on the device), and sampled windows equal numpy's step-by-step arithmetic."""
    from rtensors_amd import datagen, hip as H
    for dtype, n in (("f32", 1 << 28), ("f64", 1 << 27), ("i32", 1 << 28)):
        npd = cpu.NP_DTYPE[cpu.DTYPE_BY_NAME[dtype]]
        code = H.DTYPE_BY_NAME[dtype]
        da, db = hip.alloc_uninit(code, n), hip.alloc_uninit(code, n)
        if dtype == "i32":
            datagen.fill_device(da, "int", 1, 0, -(1 << 20), 1 << 20); datagen.fill_device(db, "int", 1, 1, -(1 << 20), 1 << 20)
        else:
            datagen.fill_device(da, "normal", 1, 0); datagen.fill_device(db, "normal", 1, 1)
        three, one = (3, 1) if dtype == "i32" else (3.0, 1.0)
        steps = [("scalar", "mul", three), ("binary", "add", 1), ("unary", "relu"), ("scalar", "sub", one)]
        c = hip.alloc_uninit(code, n)
        hip.fused_chain([(da, 0), (db, 0)], steps, c, n)
        # the same expression as the four kernels of the trait
        t = hip.alloc_uninit(code, n)
        hip.scalar_to("mul", da, three, 0, n, t)
        m = (0, [n], [1])
        hip.broadcast((t, m), (db, m), (t, m), "add")
        hip.unary_contiguous("relu", t, 0, n)
        hip.scalar_contiguous("sub", t, one, 0, n)
        assert hip.equal(c, t), dtype
        chunk = 1 << 20
        for start in (0, 12345 * 4, n - chunk):
            tmp = hip.alloc_uninit(code, chunk)
            hip.copy_range_within(tmp, c, 0, start, chunk)
            got = hip.dump(tmp)
            if dtype == "i32":
                ha, hb = datagen.integers(chunk, 1, 0, -(1 << 20), 1 << 20, start), datagen.integers(chunk, 1, 1, -(1 << 20), 1 << 20, start)
            else:
                ha, hb = datagen.normal(npd, chunk, 1, 0, 1.0, start), datagen.normal(npd, chunk, 1, 1, 1.0, start)
            want = (np.maximum((ha * npd.type(three)).astype(npd) + hb, 0).astype(npd) - npd.type(one)).astype(npd)
            assert got.tobytes() == want.tobytes(), (dtype, start)
        del da, db, c, t
        hip.sync()
