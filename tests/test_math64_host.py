"""The hand-written f64 logarithm of the device code (rtensors_amd/csrc/rt_math64.h), built for the host with g++ and measured against
numpy's 80-bit long double logarithm: error in units of the last place over the whole range (every binade sampled, the neighbourhood of
1 where the result cancels, denormals), and the special values of IEEE / Rust's f64::ln and f64::ln_1p."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def lib(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("math64") / "libmath64.so")
    subprocess.check_call(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-o", out, os.path.join(HERE, "support", "math64_host.cpp")])
    L = C.CDLL(out)
    for f in (L.log_many, L.log1p_many):
        f.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p]
    return L


def call(fn, x):
    x = np.ascontiguousarray(x, dtype=np.float64)
    y = np.empty_like(x)
    fn(x.size, x.ctypes.data, y.ctypes.data)
    return y


def ulp_error(got, exact_ld):
    """|got - exact| in units of the last place of the exact value (rounded to f64)."""
    ref = exact_ld.astype(np.float64)
    ulp = np.spacing(np.abs(ref)).astype(np.longdouble)
    return np.abs(got.astype(np.longdouble) - exact_ld) / ulp


def samples(rng):
    mant = 1.0 + rng.random(400_000)
    expo = rng.integers(-1022, 1024, size=mant.size)
    x = np.ldexp(mant, expo)
    near1 = 1.0 + np.concatenate([rng.standard_normal(100_000) * 10.0 ** rng.integers(-16, 0, size=100_000)])
    near1 = near1[near1 > 0]
    den = np.ldexp(rng.random(20_000), rng.integers(-1074, -1021, size=20_000))
    den = den[den > 0]
    edges = np.array([np.sqrt(2) / 2, np.sqrt(2), np.nextafter(np.sqrt(2) / 2, 0), np.nextafter(np.sqrt(2), 2), np.nextafter(1.0, 0), np.nextafter(1.0, 2),
                      np.finfo(np.float64).max, np.finfo(np.float64).tiny, 5e-324, 2.0, 0.5, np.e, 10.0])
    return np.concatenate([x, near1, den, edges])


def test_log_within_one_ulp(lib):
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("no 80-bit long double on this machine")
    x = samples(np.random.default_rng(1))
    got = call(lib.log_many, x)
    err = ulp_error(got, np.log(x.astype(np.longdouble)))
    assert err.max() < 1.0, (float(err.max()), float(x[err.argmax()]))


def test_log1p_within_one_ulp(lib):
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("no 80-bit long double on this machine")
    rng = np.random.default_rng(2)
    mag = 10.0 ** rng.uniform(-300, 300, size=300_000)
    # all magnitudes; the whole domain below 1; next to -1; either side of the two points where the routine changes from x itself to the
    # mantissa of 1 + x (1 + x = sqrt(2) / 2 and sqrt(2)); arguments around half an ulp of 1, where 1 + x rounds to 1
    x = np.concatenate([mag, -mag[mag < 1], rng.uniform(-1, 1, size=200_000), -1 + 10.0 ** rng.uniform(-16, 0, size=50_000),
                        rng.uniform(0.40, 0.43, size=100_000), rng.uniform(-0.30, -0.28, size=100_000),
                        10.0 ** rng.uniform(-17, -14, size=100_000), -(10.0 ** rng.uniform(-17, -14, size=100_000)),
                        np.array([1e-16, -1e-16, 2.0 ** -53, 2.0 ** -52, 1.0, np.finfo(np.float64).max, 5e-324, -5e-324])])
    x = x[x > -1]
    got = call(lib.log1p_many, x)
    err = ulp_error(got, np.log1p(x.astype(np.longdouble)))
    assert err.max() < 1.0, (float(err.max()), float(x[err.argmax()]))


def test_special_values(lib):
    inf, nan = np.inf, np.nan
    with np.errstate(all="ignore"):
        got = call(lib.log_many, np.array([0.0, -0.0, -1.0, -inf, inf, nan, 1.0, -5e-324]))
    assert got[0] == -inf and got[1] == -inf and np.isnan(got[2]) and np.isnan(got[3]) and got[4] == inf and np.isnan(got[5])
    assert got[6] == 0.0 and not np.signbit(got[6]) and np.isnan(got[7])
    with np.errstate(all="ignore"):
        got = call(lib.log1p_many, np.array([0.0, -0.0, -1.0, -2.0, inf, -inf, nan, 1e-300]))
    assert got[0] == 0.0 and not np.signbit(got[0]) and got[1] == 0.0 and np.signbit(got[1])
    assert got[2] == -inf and np.isnan(got[3]) and got[4] == inf and np.isnan(got[5]) and np.isnan(got[6]) and got[7] == 1e-300
