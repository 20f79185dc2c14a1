"""The permuting tile copy (rtensors_amd/csrc/rt_permute.h) on the host: the plan and the three stages of a block are the same code
the kernel runs; here every lane of every block is walked on the CPU under the address sanitizer, with an LDS tile and position tables
of exactly the planned sizes and a source buffer that ends where the view ends, so an index that leaves any of them aborts the run.
The result must equal the row-major copy of the view (TensorView::owned, core/tensor.rs:299-325)."""
import os
import random
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def exe(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("permute") / "permute_host")
    san = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-gpu-sanitize"]
    cmd = ["hipcc", "--offload-host-only", "-x", "hip", "-O2", "-std=c++17", "-Wno-unused-function"] + san
    cmd += [os.path.join(HERE, "support", "permute_host.cpp"), "-o", out, "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return out


def _view(rng, max_elems):
    """A permuted / reversed / stepped view of a row-major parent, as (shape, strides, offset), collapsed like rt_collapse does not
    need to be: the plan takes any strides."""
    dims = (1, 2, 3, 5, 7, 16, 33, 42, 64, 100, 129, 256, 300)
    rank = rng.choice((2, 3, 3, 4, 4, 5))
    while True:
        shp = [rng.choice(dims) for _ in range(rank)]
        n = 1
        for x in shp:
            n *= x
        if n <= max_elems:
            break
    st, s = [0] * rank, 1
    for i in reversed(range(rank)):
        st[i] = s
        s *= shp[i]
    perm = list(range(rank))
    rng.shuffle(perm)
    shape = [shp[i] for i in perm]
    strides = [st[i] for i in perm]
    kind = rng.random()
    if kind < 0.3:                                   # a step along one dim
        ax = rng.randrange(rank)
        k = rng.choice((2, 3))
        shape[ax] = (shape[ax] + k - 1) // k
        strides[ax] *= k
    if kind > 0.6:                                   # one dim reversed
        ax = rng.randrange(rank)
        strides[ax] = -strides[ax]
    if 0.5 < kind < 0.6:                             # a corner of the parent
        ax = rng.randrange(rank)
        shape[ax] = max(1, shape[ax] - rng.choice((1, 2, 5)))
    offset = -sum((d - 1) * s for d, s in zip(shape, strides) if s < 0)
    return shape, strides, offset


def test_every_element_lands_once(exe):
    rng = random.Random(23)
    cases = []
    fixed = [
        ([64, 3, 2, 96, 42], [1, 6144, 18432, 64, 36864], 0),          # short dst rows, long unit-stride dim elsewhere
        ([7, 100, 33, 29], [1, 231, 7, 23100], 0),                     # unit-stride dim of 7
        ([2, 16, 7, 2995], [1, 14, 2, 224], 0),                        # the fastest 224 elements of src permuted among themselves
        ([16, 20971, 2], [2, 32, 1], 0),                               # planar <- interleaved with a short inner dim
        ([300, 300], [1, 300], 0), ([1000, 7], [1, 1000], 0), ([7, 1000], [1, 7], 0),
        ([5, 1], [1, 5], 0), ([1, 1], [1, 1], 0), ([4097], [1], 0), ([4097], [-1], 4096), ([513, 3], [6, 2], 0),
        ([3, 3, 3, 3, 3, 3, 3, 3], [1, 3, 9, 27, 81, 243, 729, 2187], 0),
        ([40, 50, 60], [0, 60, 1], 0), ([40, 50, 60], [1, 0, 40], 0),  # repeated dims
    ]
    for es in (1, 2, 4, 8):
        for shape, strides, offset in fixed:
            cases.append((es, shape, strides, offset))
        for _ in range(120):
            shape, strides, offset = _view(rng, 150000)
            cases.append((es, shape, strides, offset))
    text = "\n".join(f"{es} {len(sh)} {' '.join(map(str, sh))} {' '.join(map(str, st))} {off}" for es, sh, st, off in cases) + "\n"
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    r = subprocess.run([exe], input=text, capture_output=True, text=True, env=env, timeout=900)
    assert r.returncode == 0 and not r.stderr.strip(), r.stderr[-3000:]
    out = r.stdout.strip().split("\n")
    assert len(out) == len(cases)
    planned = 0
    for c, line in zip(cases, out):
        assert line.startswith("ok") or line == "skip", (c, line)
        planned += line.startswith("ok")
    assert planned >= len(cases) * 9 // 10
