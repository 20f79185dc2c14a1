"""The tiled traversal of the streaming kernels (TileMap in rtensors_amd/csrc/rt_common.h) on the host: for buffers in every phase of
a 4 KiB page and of many lengths, with the block sizes and window shapes the kernels use, every vector must be owned by exactly one
lane of the launch, no lane may point outside the run, and the block-wise form of the index arithmetic must agree with the
lane-by-lane form."""
import os
import random
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def exe(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("tilemap") / "tilemap_host")
    san = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-gpu-sanitize"]
    cmd = ["hipcc", "--offload-host-only", "-x", "hip", "-O2", "-std=c++17", "-Wno-unused-function"] + san
    cmd += [os.path.join(HERE, "support", "tilemap_host.cpp"), "-o", out, "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return out


def test_every_vector_is_owned_once(exe):
    rng = random.Random(11)
    shapes = [(256, 1024, 4, 4096),        # read-modify-write kernels, copies, binary kernels, the chain
              (512, 1024, 16, 65536),      # fill
              (128, 1024, 4, 4096), (256, 512, 4, 4096), (1024, 1024, 16, 65536)]
    cases = []
    for nthreads, piece, rows, stride in shapes:
        window = rows * stride // 16
        lens = [0, 1, 2, 63, 64, 255, 256, 257, 1023, 1024, window - 1, window, window + 1, 2 * window + 77, 3 * window, 5 * window + 255]
        lens += [rng.randrange(1, 6 * window) for _ in range(12)]
        for n in lens:
            for phase in (0, 16, 128, 1024, 4080, 4096 - 128, rng.randrange(0, 256) * 16):
                cases.append((phase, n, nthreads, piece, rows, stride))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    r = subprocess.run([exe], input="\n".join(" ".join(map(str, c)) for c in cases) + "\n", capture_output=True, text=True, env=env, timeout=600)
    assert r.returncode == 0 and not r.stderr.strip(), r.stderr[-3000:]
    out = r.stdout.strip().split("\n")
    assert len(out) == len(cases)
    for c, line in zip(cases, out):
        assert line.startswith("ok"), (c, line)
