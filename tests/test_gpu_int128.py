"""GPU parity of u128 / i128 division (ops/base.rs:27-37 instantiated at the 128-bit types, core/value.rs:567-581): the device divides
with a hand-written long division.  Quotients are held bit for bit to the oracle's `__int128` division and, independently, to Python's
exact integers; zero divisors and MIN / -1 must come back as the reference's panic does (RT_E_ARITH from the next call that waits for
the stream), for every kernel shape of the broadcast family and for the scalar form."""
import random
import zlib

import numpy as np
import pytest

from oracle import cpu
from oracle.meta import Slice, TensorError as OErr
from oracle.tensor import OTensor
from test_gpu_parity import G, random_view, replay

pytestmark = pytest.mark.gpu

M128 = (1 << 128) - 1
MIN128 = -(1 << 127)


@pytest.fixture(scope="module")
def hip():
    from rtensors_amd import hip as H
    b = H.Hip.new(0)
    yield b
    b.sync()


def wrap(dtype, v):
    """A python integer as a value of `dtype` (two's complement for i128)."""
    v &= M128
    return v - (1 << 128) if dtype == "i128" and v >> 127 else v


def rand_ints(dtype, n, rng: random.Random, small=False):
    """Values of every bit length: both halves used, below 2^64, below 2^32, single bits and their neighbours."""
    out = []
    for _ in range(n):
        bits = rng.randrange(1, 12 if small else 129)
        k = rng.random()
        if k < 0.7:
            v = rng.getrandbits(bits)
        elif k < 0.85:
            v = (1 << (bits - 1)) + rng.choice([-1, 0, 1])
        else:
            v = (1 << bits) - 1
        if dtype == "i128":
            v = min(v, (1 << 127) - 1)
            if rng.random() < 0.5:
                v = -v
        out.append(wrap(dtype, v))
    return out


def trunc_div(a, b):
    q = abs(a) // abs(b)
    return -q if (a < 0) != (b < 0) else q


@pytest.mark.parametrize("dtype", ["u128", "i128"])
def test_128bit_quotients_against_exact_integers(hip, dtype):
    """Contiguous, row-broadcast, strided (element kernel) and scalar forms against Python integers: operand pairs of every size
    pairing, dividends at and next to multiples of the divisor."""
    code = cpu.DTYPE_BY_NAME[dtype]
    rng = random.Random(zlib.crc32(dtype.encode()))
    n = 60_000
    a = rand_ints(dtype, n, rng)
    b = [v or 1 for v in rand_ints(dtype, n, rng)]
    for i in range(0, n, 3):                                   # every third pair: k * d + (-1, 0, 1)
        d = b[i]
        room = 127 - abs(d).bit_length() if dtype == "i128" else 128 - abs(d).bit_length()
        k = rng.getrandbits(max(room, 0)) if room > 0 else 0
        x = k * d + rng.choice([-1, 0, 1])
        lo, hi = (MIN128, (1 << 127) - 1) if dtype == "i128" else (0, M128)
        if lo <= x <= hi:
            a[i] = x
    if dtype == "i128":
        for i in range(n):
            if a[i] == MIN128 and b[i] == -1:
                b[i] = 1
    want = [wrap(dtype, trunc_div(x, y)) for x, y in zip(a, b)]
    va, vb = cpu.from_ints(code, a), cpu.from_ints(code, b)
    ga, gb = hip.alloc_from_slice(code, va), hip.alloc_from_slice(code, vb)
    out = hip.alloc(code, n)
    hip.broadcast((ga, (0, [n], [1])), (gb, (0, [n], [1])), (out, (0, [n], [1])), "div")
    assert cpu.to_ints(code, hip.dump(out)) == want
    # strided: every second pair through the element kernel
    out2 = hip.alloc(code, n)
    hip.broadcast((ga, (0, [n // 2], [2])), (gb, (0, [n // 2], [2])), (out2, (0, [n // 2], [2])), "div")
    assert cpu.to_ints(code, hip.dump(out2))[::2] == want[::2]
    # one row of divisors under 200 rows of dividends
    rows, L = 200, 300
    out3 = hip.alloc(code, rows * L)
    hip.broadcast((ga, (0, [rows, L], [L, 1])), (gb, (7, [rows, L], [0, 1])), (out3, (0, [rows, L], [L, 1])), "div")
    got = cpu.to_ints(code, hip.dump(out3))
    for r in (0, 1, 57, 199):
        assert got[r * L:(r + 1) * L] == [wrap(dtype, trunc_div(a[r * L + c], b[7 + c])) for c in range(L)], r
    hip.sync()
    # tensor / scalar, in place, a reversed view included
    for d in [3, 10, (1 << 64) - 1, (1 << 64) + 1, (1 << 100) + 12345, (1 << 127) - 1] + ([-7, -(1 << 70), MIN128] if dtype == "i128" else [M128]):
        vals = [x for x in a[:5000] if not (dtype == "i128" and x == MIN128 and d == -1)]
        g = G(hip, dtype, cpu.from_ints(code, vals), [len(vals)])
        g /= d
        assert cpu.to_ints(code, g.dump()) == [wrap(dtype, trunc_div(x, d)) for x in vals], d
        g = G(hip, dtype, cpu.from_ints(code, vals), [len(vals)])
        v = g.slice(0, Slice(None, None, -2))
        v /= d
        expect = list(vals)
        for i in range(len(vals) - 1, -1, -2):
            expect[i] = wrap(dtype, trunc_div(vals[i], d))
        assert cpu.to_ints(code, g.dump()) == expect, d
    hip.sync()


@pytest.mark.parametrize("dtype", ["u128", "i128"])
def test_128bit_division_random_views_vs_oracle(hip, dtype):
    from rtensors_amd import hip as H
    code = cpu.DTYPE_BY_NAME[dtype]
    rng = np.random.default_rng(zlib.crc32((dtype + "div").encode()))
    prng = random.Random(int(rng.integers(0, 1 << 30)))
    for trial in range(30):
        rank = int(rng.integers(1, 6))
        full = [int(rng.integers(1, 7)) for _ in range(rank)]
        if trial % 5 == 0:
            full[-1] = int(rng.choice([64, 100, 257, 1024]))
        sa = [d if rng.random() < 0.7 else 1 for d in full]
        sb = [d if rng.random() < 0.7 else 1 for d in full]
        if rng.random() < 0.3:
            sb = sb[int(rng.integers(0, rank)):]
        a = rand_ints(dtype, int(np.prod(sa)), prng)
        b = rand_ints(dtype, int(np.prod(sb)), prng, small=trial % 2 == 0)
        if trial % 3 != 0:
            b = [v or 1 for v in b]                                         # every third trial keeps its zero divisors
        if dtype == "i128" and trial % 6 == 3 and a and b:
            a[prng.randrange(len(a))] = MIN128                              # MIN / -1 overflows
            b[prng.randrange(len(b))] = -1
        va, vb = cpu.from_ints(code, a), cpu.from_ints(code, b)
        oa, ob = OTensor.from_buf(dtype, va, sa), OTensor.from_buf(dtype, vb, sb)
        ga, gb = G(hip, dtype, va, sa), G(hip, dtype, vb, sb)
        ova, ovb = random_view(oa, rng), random_view(ob, rng)
        fault = False
        try:
            want = ova / ovb
        except OErr as e:
            if e.kind == "BroadcastError":
                continue
            assert e.kind == "ArithmeticPanic", e.kind
            fault = True
        got = replay(ova, ga) / replay(ovb, gb)
        if fault:
            with pytest.raises(H.TensorError) as e:
                got.dump()
            assert e.value.kind == "ArithmeticError", (trial, dtype, ova.meta, ovb.meta)
            hip.sync()
            continue
        assert got.meta.shape == want.meta.shape
        assert got.dump().tobytes() == want.buf.tobytes(), (trial, dtype, ova.meta, ovb.meta)
    hip.sync()


@pytest.mark.parametrize("dtype", ["u128", "i128"])
def test_128bit_division_faults(hip, dtype):
    """A zero divisor or MIN / -1 inside a tensor is RT_E_ARITH at the next synchronising call, once, for every kernel shape of the
    broadcast family; without a fault nothing is reported and the quotients equal the oracle's."""
    from rtensors_amd import hip as H
    code = cpu.DTYPE_BY_NAME[dtype]
    rng = np.random.default_rng(zlib.crc32(dtype.encode()) + 99)
    signed = dtype == "i128"
    layouts = [([4096], [4096], None), ([64, 256], [256], None), ([64, 256], [64, 1], None), ([8, 16, 1024], [16, 1], None),
               ([128, 256], [256, 128], "T"), ([33, 70], [33, 70], "step2"), ([3, 5, 7], [1], None)]
    for sa, sb, how in layouts:
        for kind in ("zero", "min_neg1", "clean"):
            if kind == "min_neg1" and not signed:
                continue
            a = [int(v) << 70 | int(v) for v in rng.integers(1, 1 << 40, size=int(np.prod(sa)))]
            b = [int(v) for v in rng.integers(1, 1 << 20, size=int(np.prod(sb)))]
            ib = int(rng.integers(0, len(b)))
            if kind == "zero":
                b[ib] = 0
            elif kind == "min_neg1":
                a = [MIN128] * len(a)
                b[ib] = -1
            va, vb = cpu.from_ints(code, a), cpu.from_ints(code, b)
            oa, ob = OTensor.from_buf(dtype, va, sa), OTensor.from_buf(dtype, vb, sb)
            ga, gb = G(hip, dtype, va, sa), G(hip, dtype, vb, sb)
            if how == "T":
                ob, gb = ob.transpose(), gb.transpose()
            elif how == "step2":
                oa, ga = oa.slice(1, Slice(None, None, 2)), ga.slice(1, Slice(None, None, 2))
                ob, gb = ob.slice(1, Slice(None, None, 2)), gb.slice(1, Slice(None, None, 2))
                if kind != "clean" and (ib % 70) % 2 == 1:
                    continue
            try:
                want = oa / ob
                faulted = False
            except OErr as e:
                assert e.kind == "ArithmeticPanic"
                faulted = True
            assert faulted == (kind != "clean"), (dtype, sa, sb, how, kind)
            got = ga / gb
            if faulted:
                with pytest.raises(H.TensorError) as e:
                    hip.sync()
                assert e.value.kind == "ArithmeticError" and e.value.status == 7
                hip.sync()
                out = cpu.to_ints(code, got.dump())
                if kind == "zero" and how is None and sa == sb:
                    assert out == [0 if y == 0 else wrap(dtype, trunc_div(x, y)) for x, y in zip(a, b)]
            else:
                hip.sync()
                assert got.dump().tobytes() == want.buf.tobytes(), (dtype, sa, sb, how)
    vals = [int(v) for v in rng.integers(1, 1 << 60, size=1000)]
    g = G(hip, dtype, cpu.from_ints(code, vals), [1000])
    with pytest.raises(H.TensorError) as e:
        g /= 0
    assert e.value.kind == "ArithmeticError"
    if signed:
        g /= -1
        hip.sync()
        assert cpu.to_ints(code, g.dump()) == [-v for v in vals]
        vals[17] = MIN128
        g = G(hip, dtype, cpu.from_ints(code, vals), [1000])
        g /= -1
        with pytest.raises(H.TensorError) as e:
            g.dump()
        assert e.value.kind == "ArithmeticError"
        hip.sync()
        assert cpu.to_ints(code, g.dump())[17] == MIN128
