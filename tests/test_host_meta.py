"""The C++ host layer's metadata arithmetic (no device needed) against the reference's own expectations and against the
oracle's independent Python restatement on random layouts."""
import numpy as np
import pytest

import golden_dsl
from oracle import meta as om


@pytest.fixture(scope="module")
def T():
    from rtensors_amd import tensor
    return tensor


def test_library_exports_every_declared_symbol():
    import re, os
    from rtensors_amd import _ffi
    hdr = open(os.path.join(os.path.dirname(_ffi.HERE), "include", "rt_hip.h")).read()
    declared = set(re.findall(r"^(?:int32_t|const char\*)\s+(rt_[a-z0-9_]+)\s*\(", hdr, flags=re.M))
    assert declared == set(_ffi.SYMBOLS), declared ^ set(_ffi.SYMBOLS)
    for name in declared:
        assert hasattr(_ffi.lib, name)
    assert _ffi.lib.rt_dtype_size(10) == 4 and _ffi.lib.rt_dtype_size(9) == 16 and _ffi.lib.rt_dtype_size(99) == 0
    assert _ffi.lib.rt_status_name(3) == b"RT_E_OUT_OF_BOUNDS"


META_CASES = golden_dsl.load("reference_meta_vectors.json")


class MetaOnly:
    """Runs the golden program format on metadata alone through the C++ layer."""

    def __init__(self, T, shape, strides=None, offset=0):
        self.T, self.shape, self.offset = T, list(shape), offset
        self.strides = list(strides) if strides is not None else om.shape_to_stride(shape)

    def slice(self, dim, sl):
        return MetaOnly(self.T, *self.T.meta_slice(self.shape, self.strides, self.offset, dim, self.T.Slice(sl.start, sl.end, sl.step)))

    def permute(self, dims): return MetaOnly(self.T, *self.T.meta_permute(self.shape, self.strides, self.offset, dims))
    def transpose(self): return self.permute(list(range(len(self.shape) - 1, -1, -1)))
    def unsqueeze_at(self, d): return MetaOnly(self.T, *self.T.meta_unsqueeze(self.shape, self.strides, self.offset, d))
    def squeeze_at(self, d): return MetaOnly(self.T, *self.T.meta_squeeze(self.shape, self.strides, self.offset, d))
    def squeeze(self): return MetaOnly(self.T, *self.T.meta_squeeze(self.shape, self.strides, self.offset, None))


@pytest.mark.parametrize("case", META_CASES, ids=lambda c: c["name"])
def test_reference_meta_vectors(T, case):
    values = {}

    def factory(dtype, vals, shape):
        m = MetaOnly(T, shape)
        values[id(m)] = vals
        m.base = vals
        return m

    def propagate(env):
        for name, t in env.items():
            if not hasattr(t, "base"):
                t.base = next(iter(case["inputs"].values()))["values"]

    env, err = golden_dsl.run_case(case, factory, om.Slice, T.TensorError)
    propagate(env)

    def get(t, idx):
        return t.base[om.logical_to_buffer_idx(idx, t.strides, t.offset)]

    golden_dsl.check_case(case, env, err, lambda t: None, get,
                          lambda t: (t.shape, t.strides, t.offset, T.meta_is_contiguous(t.shape, t.strides)))


def test_random_layouts_match_oracle_meta(T):
    rng = np.random.default_rng(0)
    for trial in range(400):
        rank = int(rng.integers(0, 5))
        shape = [int(rng.integers(1, 7)) for _ in range(rank)]
        o = om.MetaTensor.row_major(shape)
        c = MetaOnly(T, shape)
        for _ in range(int(rng.integers(1, 5))):
            r = len(o.shape)
            k = int(rng.integers(0, 4))
            try:
                if k == 0 and r > 0:
                    d = int(rng.integers(0, r + 1)); n = o.shape[d] if d < r else 1
                    sl = om.Slice(*[None if rng.random() < 0.3 else int(rng.integers(0, n + 2)) for _ in range(2)], int(rng.choice([-3, -2, -1, 0, 1, 2, 3])))
                    want = om.compute_sliced_parameters(o.shape, o.strides, o.offset, d, sl)
                    got = c.slice(d, sl)
                    o = om.MetaTensor(*want)
                elif k == 1:
                    dims = [int(x) for x in rng.permutation(r)] if rng.random() < 0.9 else [0] * (r + 1)
                    want = om.compute_permuted_parameters(o.shape, o.strides, dims)
                    got = c.permute(dims)
                    o = om.MetaTensor(want[0], want[1], o.offset)
                elif k == 2:
                    d = int(rng.integers(0, r + 2))
                    want = om.compute_unsqueezed_parameters(o.shape, o.strides, d)
                    got = c.unsqueeze_at(d)
                    o = om.MetaTensor(want[0], want[1], o.offset)
                else:
                    d = None if rng.random() < 0.5 else int(rng.integers(0, r + 1))
                    want = om.compute_squeezed_parameters(o.shape, o.strides, d)
                    got = c.squeeze() if d is None else c.squeeze_at(d)
                    o = om.MetaTensor(want[0], want[1], o.offset)
            except om.TensorError as e:
                with pytest.raises(T.TensorError) as ge:
                    {0: lambda: c.slice(d, sl), 1: lambda: c.permute(dims), 2: lambda: c.unsqueeze_at(d),
                     3: lambda: (c.squeeze() if d is None else c.squeeze_at(d))}[k]()
                assert ge.value.kind == e.kind, (k, e.kind, ge.value.kind)
                break
            c = got
            assert (c.shape, c.strides, c.offset) == (o.shape, o.strides, o.offset)
            assert T.meta_is_contiguous(c.shape, c.strides) == o.is_contiguous()


def test_broadcast_params_match_oracle(T):
    rng = np.random.default_rng(1)
    for trial in range(300):
        ra, rb = int(rng.integers(0, 5)), int(rng.integers(0, 5))
        full = [int(rng.integers(1, 5)) for _ in range(max(ra, rb))]
        sa = [d if rng.random() < 0.7 else (1 if rng.random() < 0.8 else d + 1) for d in full[len(full) - ra:]]
        sb = [d if rng.random() < 0.7 else (1 if rng.random() < 0.8 else d + 1) for d in full[len(full) - rb:]]
        a, b = om.MetaTensor.row_major(sa), om.MetaTensor.row_major(sb)
        try:
            want = om.compute_broadcasted_params(a, b)
        except om.TensorError:
            with pytest.raises(T.TensorError) as e:
                T.meta_broadcast(a.shape, a.strides, b.shape, b.strides)
            assert e.value.kind == "BroadcastError"
            continue
        assert T.meta_broadcast(a.shape, a.strides, b.shape, b.strides) == tuple(want)
