"""rt_reduce_nd_static (the entry point that allocates nothing) against rt_reduce_nd, through the C ABI.

Both run the same kernels with the same split, so every result is compared bit for bit (floats included).  Two calls in a row
share the built-in workspace, the second with a smaller input; the context's allocator must see no device allocation."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from rtensors_amd import hip as H
    b = H.Hip.new(0)
    yield b
    b.sync()


def _both(hip, H, src, shape, dim, op, out_dtype=None):
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * shape[i + 1]
    nout = int(np.prod(shape)) // shape[dim]
    a = hip.alloc(out_dtype if out_dtype is not None else src.dtype, nout)
    b = hip.alloc(out_dtype if out_dtype is not None else src.dtype, nout)
    hip.sync()
    before = hip.mem_stats()["device_allocs"]
    hip.apply_reduce_contiguous_nd_static((src, (0, shape, strides)), b, dim, op)
    after = hip.mem_stats()["device_allocs"]
    assert after == before, "the entry point that allocates nothing asked the context's allocator for device memory"
    hip.apply_reduce_contiguous_nd((src, (0, shape, strides)), a, dim, op)
    return hip.dump(a), hip.dump(b)


def test_static_call_leaves_the_scratch_buffer_alone():
    """On a fresh context a split reduction through rt_reduce_nd grows the context's scratch buffer (one device allocation, which the
    allocator's counter sees); the same reduction through rt_reduce_nd_static, issued first, must not."""
    from rtensors_amd import hip as H
    be = H.Hip.new(0)
    n = 1 << 22
    src = be.alloc_from_slice(H.F32, np.ones(n, dtype=np.float32))
    a, b = be.alloc(H.F32, 1), be.alloc(H.F32, 1)
    be.sync()
    before = be.mem_stats()["device_allocs"]
    be.apply_reduce_contiguous_nd_static((src, (0, [n], [1])), b, 0, "sum")
    assert be.mem_stats()["device_allocs"] == before, "the static entry point grew the context's scratch buffer"
    be.apply_reduce_contiguous_nd((src, (0, [n], [1])), a, 0, "sum")
    assert be.mem_stats()["device_allocs"] == before + 1, "the scratch growth of rt_reduce_nd is not counted: the check above proves nothing"
    assert be.dump(a)[0] == be.dump(b)[0] == float(n)
    del src, a, b
    be.close()


@pytest.mark.parametrize("dtype", ["f32", "i32", "f64"])
def test_static_workspace_reduction_matches_rt_reduce_nd(hip, dtype):
    from rtensors_amd import hip as H
    from oracle import cpu
    from oracle.meta import MetaTensor
    rng = np.random.default_rng(7)
    code = H.DTYPE_BY_NAME[dtype]
    npd = H.NP_DTYPE[code]
    # shapes whose reductions split (few outputs, long reduced axis) and therefore use the workspace; the second call of each
    # pair is smaller than the first, so it meets the leftovers of the first in the workspace
    cases = [
        ([1 << 22], 0), ([1 << 18], 0),                      # full reduce of one long row
        ([4096, 2048], 0), ([1024, 512], 0),                 # column reduce, R split over blocks
        ([2, 1 << 20], 1), ([3, 40000], 1),                  # two / three long rows
        ([1, 300000, 3], 1), ([1, 70000, 3], 1),             # narrow columns
    ]
    for shape, dim in cases:
        n = int(np.prod(shape))
        x = (rng.standard_normal(n) * 3).astype(npd) if npd.kind == "f" else rng.integers(-1000, 1001, size=n).astype(npd)
        src = hip.alloc_from_slice(code, x)
        for op in ("sum", "max", "mean", "min", "prod"):
            want, got = _both(hip, H, src, shape, dim, op)
            assert want.tobytes() == got.tobytes(), (dtype, shape, dim, op)
        for op in (("var", "logsumexp", "l2_norm") if npd.kind == "f" else ()):
            # the statistics keep partial states of 8 .. 24 bytes: a split over many columns may not fit the workspace
            try:
                want, got = _both(hip, H, src, shape, dim, op)
            except H.TensorError as e:
                assert e.status == 1 and "workspace" in str(e), str(e)
                continue
            assert want.tobytes() == got.tobytes(), (dtype, shape, dim, op)
        # and against the oracle to the documented bar (integers exact, float sums within rel * sum|x|)
        want, got = _both(hip, H, src, shape, dim, "sum")
        strides = [1] * len(shape)
        for i in range(len(shape) - 2, -1, -1):
            strides[i] = strides[i + 1] * shape[i + 1]
        ref = cpu.reduce_nd(cpu.DTYPE_BY_NAME[dtype], "sum", x, MetaTensor(shape, strides, 0), dim)
        if npd.kind == "f":
            rel = 1e-5 if dtype == "f32" else 1e-12
            sabs = np.abs(x.astype(np.float64)).reshape(shape).sum(axis=dim).reshape(-1)
            assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64).reshape(-1)) <= rel * sabs + 1e-300)
        else:
            assert got.tobytes() == ref.tobytes()


def test_static_workspace_limit_is_an_error_not_a_launch(hip):
    from rtensors_amd import hip as H
    # variance over axis 0 of (256, 65536) f32: the column reduce splits R in two and its partial states (mean, m2, count per
    # column and segment) exceed the 1 MiB workspace; sum / max / min / mean partials of any shape fit
    shape = [256, 1 << 16]
    src = hip.alloc(H.F32, shape[0] * shape[1])
    dst = hip.alloc(H.F32, shape[1])
    hip.fill_contiguous(dst, 5.0, 0, dst.len)
    try:
        hip.apply_reduce_contiguous_nd_static((src, (0, shape, [shape[1], 1])), dst, 0, "var")
        refused = False
    except H.TensorError as e:
        refused = True
        assert e.status == 1 and "workspace" in str(e)
    if refused:
        assert np.all(hip.dump(dst) == 5.0)          # nothing was launched
    else:
        assert np.all(hip.dump(dst) == 0.0)          # the plan did not split: it ran without the workspace, which is fine too
