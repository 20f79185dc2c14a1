"""The hand-written f64 routines of the device code (rtensors_amd/csrc/rt_math64.h: logarithm, arcsine / arccosine, sine / cosine /
tangent, the exponential of non-positive arguments, and the reciprocal, quotient and square-root helpers under them), built for the host with g++ and measured against numpy's
80-bit long double functions: error in units of the last place over the whole range each routine is used on, and the special values of
IEEE / Rust's f64 methods.  The host build replaces the hardware's reciprocal and reciprocal-square-root estimates by cruder ones
(20 bits), so the bounds hold for the device a fortiori; tests/test_gpu_math.py asserts them there as well."""
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
    for f in (L.log_many, L.log1p_many, L.asin_many, L.acos_many, L.tan_many, L.sqrt_ge1_many, L.rcp_many, L.exp_nonpos_many):
        f.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p]
    L.quot_many.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]
    L.sincos_kernel_many.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]
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


def need_long_double():
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("no 80-bit long double on this machine")


def test_asin_acos_within_two_ulp(lib):
    need_long_double()
    rng = np.random.default_rng(3)
    # the whole domain; next to +-1, where the square-root form ends; every magnitude down to the denormals; either side of |x| = 0.5, where
    # the two forms meet
    x = np.concatenate([rng.uniform(-1, 1, 1_000_000), 1 - 10.0 ** rng.uniform(-16, 0, 100_000), -1 + 10.0 ** rng.uniform(-16, 0, 100_000),
                        10.0 ** rng.uniform(-300, 0, 100_000), -(10.0 ** rng.uniform(-300, 0, 100_000)), rng.uniform(0.49, 0.51, 100_000),
                        rng.uniform(-0.51, -0.49, 100_000), np.array([0.5, -0.5, 1.0, -1.0, 0.975, 5e-324])])
    x = x[np.abs(x) <= 1]
    xl = x.astype(np.longdouble)
    err = ulp_error(call(lib.asin_many, x), np.arcsin(xl))
    assert err.max() < 2.0, ("asin", float(err.max()), float(x[err.argmax()]))
    err = ulp_error(call(lib.acos_many, x[x < 1]), np.arccos(xl[x < 1]))                # acos(1) = 0 exactly, checked below
    assert err.max() < 1.5, ("acos", float(err.max()), float(x[err.argmax()]))
    sp = np.array([0.0, -0.0, 1.0, -1.0, 1.5, -1.5, np.nan, np.inf, -np.inf, 5e-324, -5e-324, np.nextafter(1.0, 2)])
    with np.errstate(all="ignore"):
        a, b = call(lib.asin_many, sp), call(lib.acos_many, sp)
        assert np.array_equal(a, np.arcsin(sp), equal_nan=True) and np.signbit(a[1]) and not np.signbit(a[0])
        assert np.array_equal(b, np.arccos(sp), equal_nan=True)


def trig_arguments(rng):
    k = rng.integers(-2 ** 20, 2 ** 20, 200_000)
    near = (k * (np.pi / 2)) * (1 + rng.standard_normal(k.size) * 10.0 ** rng.integers(-16, -3, k.size))      # next to multiples of pi/2
    x = np.concatenate([rng.uniform(-10, 10, 600_000), rng.uniform(-1e6, 1e6, 300_000), 10.0 ** rng.uniform(-300, 9, 200_000),
                        -(10.0 ** rng.uniform(-300, 9, 200_000)), near, rng.uniform(-2.0 ** 30, 2.0 ** 30, 200_000), rng.uniform(-0.8, 0.8, 200_000),
                        np.array([np.pi / 4, -np.pi / 4, np.pi / 2, np.pi, 3 * np.pi / 4, 2.0 ** 30 - 1, 5e-324])])
    return x[np.abs(x) < 2.0 ** 30]


def test_tan_below_2_30(lib):
    need_long_double()
    x = trig_arguments(np.random.default_rng(7))
    xl = x.astype(np.longdouble)
    err = ulp_error(call(lib.tan_many, x), np.tan(xl))
    assert err.max() < 3.0, ("tan", float(err.max()), float(x[err.argmax()]))
    sp = np.array([0.0, -0.0, 5e-324, -5e-324, 1e-300, np.pi / 2, np.pi, -np.pi / 4])
    got = call(lib.tan_many, sp)
    assert np.array_equal(got, np.tan(sp)) and np.signbit(got[1]) and not np.signbit(got[0])
    # the two kernels under it, on arguments within a quarter turn of 0 (no quadrant): sine and cosine within 1.5 ulp
    y = np.ascontiguousarray(np.concatenate([np.random.default_rng(8).uniform(-np.pi / 4, np.pi / 4, 500_000), 10.0 ** np.random.default_rng(9).uniform(-300, -1, 100_000)]))
    s_out, c_out = np.empty_like(y), np.empty_like(y)
    lib.sincos_kernel_many(y.size, y.ctypes.data, s_out.ctypes.data, c_out.ctypes.data)
    yl = y.astype(np.longdouble)
    assert ulp_error(s_out, np.sin(yl)).max() < 1.5 and ulp_error(c_out, np.cos(yl)).max() < 1.5


def test_reciprocal_quotient_and_square_root_helpers(lib):
    need_long_double()
    rng = np.random.default_rng(5)
    a = np.concatenate([1 + rng.random(300_000) * 3, 10.0 ** rng.uniform(0, 307, 300_000), 1 + 10.0 ** rng.uniform(-16, 0, 100_000)])
    err = ulp_error(call(lib.sqrt_ge1_many, a), np.sqrt(a.astype(np.longdouble)))
    assert err.max() <= 1.0, float(err.max())
    got = call(lib.sqrt_ge1_many, np.array([1.0, np.inf, np.nan, 4.0]))
    assert got[0] == 1.0 and got[1] == np.inf and np.isnan(got[2]) and got[3] == 2.0
    d = np.concatenate([1 + 10.0 ** rng.uniform(-16, 300, 300_000), rng.uniform(1, 2, 300_000), rng.uniform(-500, 500, 100_000)])
    err = ulp_error(call(lib.rcp_many, d), 1 / d.astype(np.longdouble))
    assert err.max() <= 1.0, float(err.max())
    n, d = rng.uniform(-2, 2, 500_000), rng.uniform(2.0 ** -53, 2, 500_000)
    n[:1000], d[:1000] = 2.0 - 2.0 ** -52, 2.0 ** -53 * (1 + rng.random(1000))               # the largest quotients atanh forms
    x = np.ascontiguousarray(n); y = np.ascontiguousarray(d); out = np.empty_like(x)
    lib.quot_many(x.size, x.ctypes.data, y.ctypes.data, out.ctypes.data)
    err = ulp_error(out, x.astype(np.longdouble) / y.astype(np.longdouble))
    assert err.max() <= 1.0, float(err.max())


def test_exp_of_non_positive_arguments_within_one_and_a_half_ulp(lib):
    if np.finfo(np.longdouble).nmant < 63:
        pytest.skip("no 80-bit long double on this machine")
    rng = np.random.default_rng(9)
    ln2 = np.log(2.0)
    k = rng.integers(0, 1080, size=200_000)
    # the whole range down to where the result is 0, every magnitude near 0, either side of the points where the nearest multiple of
    # ln 2 changes (|r| largest), results in the denormal range
    x = -np.concatenate([rng.uniform(0, 760, size=400_000), 10.0 ** rng.uniform(-320, 2.9, size=200_000), (k + 0.5) * ln2 + rng.normal(size=k.size) * 1e-9,
                         k * ln2 + rng.normal(size=k.size) * 1e-9, rng.uniform(700, 746, size=100_000), np.array([0.0, 5e-324, 1e-16, 1.0, 708.4, 745.13, 745.14, 750.0, 1e300])])
    x = x[x <= 0]
    got = call(lib.exp_nonpos_many, x)
    exact = np.exp(x.astype(np.longdouble))
    normal = exact >= np.finfo(np.float64).tiny
    err = ulp_error(got[normal], exact[normal])
    assert err.max() < 1.5, (float(err.max()), float(x[normal][err.argmax()]))
    # denormal results: within one unit of the last (denormal) place; and nothing below 2^-1075 comes back non-zero
    sub = np.abs(got[~normal].astype(np.longdouble) - exact[~normal]) / np.longdouble(5e-324)
    assert sub.max() <= 1.0, float(sub.max())
    special = call(lib.exp_nonpos_many, np.array([-np.inf, np.nan, -0.0, -1e308]))
    assert special[0] == 0.0 and special[1] == 0.0 and special[2] == 1.0 and special[3] == 0.0        # NaN is the caller's business
