"""Pins the CPU oracle to the reference: every known-answer vector transcribed from the reference's own tests
(tests/golden/*.json, each case cites its source lines) must come out of the oracle exactly."""
import numpy as np
import pytest

import golden_dsl
from oracle import cpu
from oracle.meta import Slice, TensorError
from oracle.tensor import OTensor

CASES = golden_dsl.load("reference_vectors.json") + golden_dsl.load("reference_scalar_vectors.json") + golden_dsl.load("reference_view_vectors.json") + golden_dsl.load("reference_operand_vectors.json") + golden_dsl.load("reference_matmul_vectors.json")
META_CASES = golden_dsl.load("reference_meta_vectors.json")


def _factory(dtype, values, shape):
    return OTensor.from_buf(dtype, values, shape)


def _meta_of(t):
    return t.meta.shape, t.meta.strides, t.meta.offset, t.meta.is_contiguous()


@pytest.mark.parametrize("case", CASES + META_CASES, ids=lambda c: c["name"])
def test_reference_vector(case, oracle_lib):
    env, err = golden_dsl.run_case(case, _factory, Slice, TensorError)
    golden_dsl.check_case(case, env, err, lambda t: t.to_numpy(), lambda t, idx: t.get(idx), _meta_of)


def test_order_sensitive_sum_is_sequential(oracle_lib):
    # backend/cpu.rs:1167-1172 expects 1.0999999999999999 while the CUDA test on the same data expects 1.1
    # (backend/cuda.rs:2305-2310): only a strict left-to-right f64 accumulation gives the former.
    x = np.array([0.2, 0.3, 0.1, 0.3, 0.3, -0.1, -0.3, 0.3])
    assert cpu.reduce_flat(cpu.F64, "sum", x, 0, 8)[0] == 1.0999999999999999
    assert cpu.reduce_flat(cpu.F64, "sum", x, 0, 8)[0] != 1.1


def test_large_n_spot_checks(oracle_lib):
    # ops/mod.rs:3115-3213 (sizes scaled down 10x; the closed forms are size independent)
    n = 1_000_000
    t = OTensor.from_buf("i32", np.arange(n, dtype=np.int32), [n])
    t += 100
    assert np.array_equal(t.buf, np.arange(n, dtype=np.int32) + 100)
    t = OTensor.from_buf("i32", np.arange(1, n + 1, dtype=np.int32), [n])
    t *= 3
    assert np.array_equal(t.buf, np.arange(1, n + 1, dtype=np.int32) * 3)
    m = OTensor.from_buf("i32", np.arange(1000 * 1000, dtype=np.int32), [1000, 1000])
    col = m.slice(1, Slice.index(500))
    col += 999
    want = np.arange(1000 * 1000, dtype=np.int32).reshape(1000, 1000)
    want[:, 500] += 999
    assert np.array_equal(m.buf.reshape(1000, 1000), want)
    f = OTensor.from_buf("f32", (np.arange(n, dtype=np.float32) * np.float32(0.5)), [n])
    f *= 2.0
    assert np.array_equal(f.buf, np.arange(n, dtype=np.float32))
