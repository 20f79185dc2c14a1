"""The hand-written 128-bit division of the device code (rtensors_amd/csrc/rt_div128.h), built for the host with g++ and held to
Python's exact integers: truncating quotient for every operand size pairing, the edge values of each branch (divisor below / above
2^64, estimates that need the correction step, MIN / -1 wrapping to MIN)."""
import ctypes as C
import os
import random
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
M128 = (1 << 128) - 1


@pytest.fixture(scope="module")
def lib(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("div128") / "libdiv128.so")
    subprocess.check_call(["g++", "-O2", "-shared", "-fPIC", "-fsanitize=undefined", "-fno-sanitize-recover=undefined", "-o", out,
                           os.path.join(HERE, "support", "div128_host.cpp")])
    L = C.CDLL(out)
    L.div128_many.argtypes = [C.c_int, C.c_size_t, C.c_char_p, C.c_char_p, C.c_char_p]
    L.div_128_by_64.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
    L.div_128_by_64.restype = C.c_uint64
    return L


def _signed(v):
    return v - (1 << 128) if v >> 127 else v


def _trunc_div(a, b):
    q = abs(a) // abs(b)
    return -q if (a < 0) != (b < 0) else q


def _interesting(rng, count):
    """Unsigned 128-bit values of every bit length: random bits, all ones, a single bit, a bit +- 1, halves equal to 0 / 2^64 - 1."""
    out = [0, 1, 2, 3, M128, M128 - 1, 1 << 127, (1 << 127) - 1, (1 << 127) + 1, 1 << 64, (1 << 64) - 1, (1 << 64) + 1, (1 << 63), (1 << 32),
           (1 << 32) - 1, ((1 << 64) - 1) << 64, 0xFFFFFFFF00000000FFFFFFFF00000000, 0x00000000FFFFFFFF00000000FFFFFFFF]
    for bits in range(1, 129):
        top = 1 << (bits - 1)
        out += [top, (top - 1) | (top >> 1), (top << 1) - 1 if bits < 128 else M128]
        for _ in range(count):
            out.append(top | rng.getrandbits(bits - 1) if bits > 1 else 1)
    return out


def _run(lib, is_signed, pairs):
    a = b"".join((x & M128).to_bytes(16, "little") for x, _ in pairs)
    b = b"".join((y & M128).to_bytes(16, "little") for _, y in pairs)
    q = C.create_string_buffer(16 * len(pairs))
    lib.div128_many(1 if is_signed else 0, len(pairs), a, b, q)
    raw = q.raw
    return [int.from_bytes(raw[16 * i:16 * i + 16], "little") for i in range(len(pairs))]


def test_unsigned_quotients(lib):
    rng = random.Random(1)
    vals = _interesting(rng, 3)
    pairs = [(rng.choice(vals), rng.choice(vals)) for _ in range(150_000)]
    pairs += [(x, y) for x in vals[:18] for y in vals[:18]]
    # dividends just below, at and just above multiples of the divisor: the estimate-and-correct steps
    for _ in range(60_000):
        d = rng.choice(vals)
        if d == 0:
            continue
        k = rng.getrandbits(rng.randrange(0, 129 - d.bit_length() + 1)) if d.bit_length() <= 128 else 0
        for delta in (-1, 0, 1):
            x = k * d + delta
            if 0 <= x <= M128:
                pairs.append((x, d))
    pairs = [(x, y) for x, y in pairs if y != 0]
    got = _run(lib, False, pairs)
    for (x, y), q in zip(pairs, got):
        assert q == x // y, (hex(x), hex(y), hex(q), hex(x // y))


def test_signed_quotients(lib):
    rng = random.Random(2)
    vals = _interesting(rng, 2)
    pairs = []
    for _ in range(150_000):
        x, y = _signed(rng.choice(vals)), _signed(rng.choice(vals))
        if rng.random() < 0.3:
            x = -x if -(1 << 127) <= -x < (1 << 127) else x
        if y:
            pairs.append((x, y))
    mn = -(1 << 127)
    pairs += [(mn, 1), (mn, -1), (mn, 2), (mn, mn), (mn + 1, -1), ((1 << 127) - 1, -1), (-1, mn), (7, -2), (-7, 2), (-7, -2)]
    got = _run(lib, True, pairs)
    for (x, y), q in zip(pairs, got):
        want = _trunc_div(x, y)
        if x == mn and y == -1:
            want = mn                                                   # wraps; the caller raises the fault
        assert _signed(q) == want, (x, y, _signed(q), want)


def test_128_by_64_step(lib):
    rng = random.Random(3)
    for _ in range(200_000):
        v = rng.getrandbits(rng.randrange(1, 65)) or 1
        u1 = rng.randrange(0, v)
        u0 = rng.choice([0, (1 << 64) - 1, rng.getrandbits(64), rng.getrandbits(32)])
        assert lib.div_128_by_64(u1, u0, v) == ((u1 << 64) | u0) // v, (u1, u0, v)
    top = (1 << 64) - 1
    for v in (1 << 63, top, (1 << 63) + 1, (1 << 32) + 1, (1 << 32), 3):
        for u1 in (0, v - 1, v // 2):
            for u0 in (0, top, 1 << 63):
                assert lib.div_128_by_64(u1, u0, v) == ((u1 << 64) | u0) // v
