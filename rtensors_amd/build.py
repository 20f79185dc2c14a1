"""Builds librt_hip.so (HIP kernels + C ABI) and librt_datagen.so for gfx950 with hipcc, in-tree.

    python -m rtensors_amd.build            # incremental
    python -m rtensors_amd.build --force    # recompile everything

hipcc cross-compiles without a GPU.  Objects go to rtensors_amd/_build/, the shared libraries to rtensors_amd/lib/.
"""
from __future__ import annotations

import os
import subprocess
import sys
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "lib")
ARCH = os.environ.get("RT_HIP_ARCH", "gfx950")



def read_build_flags(path: str = os.path.join(CSRC, "build_flags.txt"), arch: str = ARCH) -> dict:
    """The sections of csrc/build_flags.txt (compile flags, sources, headers, link flags): the one description of the build that
    this builder and the Rust-side build script (integration/rust/build_hip.rs) both read."""
    out, cur = {}, None
    for ln in open(path):
        ln = ln.strip()
        if not ln or ln.startswith("#"):
            continue
        if ln.startswith("[") and ln.endswith("]"):
            cur = ln[1:-1]
            out[cur] = []
        else:
            out[cur].append(ln.replace("{arch}", arch))
    return out


_B = read_build_flags()
FLAGS = _B["compile"]
LINK = _B["link"]
LIBS = {
    "librt_hip.so": _B["sources"],
    "librt_datagen.so": ["rt_datagen.hip"],          # synthetic-data generator of the benchmark and the tests, not part of the backend
}
HEADERS = [os.path.normpath(os.path.join(CSRC, h)) for h in _B["headers"]]


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def _filter(text: str) -> str:
    keep = [ln for ln in text.splitlines() if "is not a recognized feature for this target" not in ln]
    return "\n".join(keep).strip()


def _compile(src: str, force: bool) -> str:
    path = os.path.join(CSRC, src)
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    if force or _stale(obj, [path] + HEADERS):
        t0 = time.time()
        r = subprocess.run(["hipcc"] + FLAGS + ["-c", path, "-o", obj], capture_output=True, text=True)
        msg = _filter(r.stdout + r.stderr)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{msg}")
        if msg:
            print(msg, file=sys.stderr)
        print(f"[build] {src}: {time.time() - t0:.1f}s", file=sys.stderr)
    return obj


def build(force: bool = False, jobs: int = 8) -> None:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB, exist_ok=True)
    srcs = [s for ss in LIBS.values() for s in ss if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = dict(zip(srcs, ex.map(lambda s: _compile(s, force), srcs)))
    for lib, ss in LIBS.items():
        ss = [s for s in ss if s in objs]
        if not ss:
            continue
        out = os.path.join(LIB, lib)
        deps = [objs[s] for s in ss]
        if force or _stale(out, deps):
            r = subprocess.run(["hipcc"] + [f for f in LINK if not f.startswith("-l")] + ["-o", out] + deps + [f for f in LINK if f.startswith("-l")],
                               capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"link of {lib} failed:\n{_filter(r.stdout + r.stderr)}")
            print(f"[build] linked {lib}", file=sys.stderr)


    _build_host(force)


def _build_host(force: bool) -> None:
    """librt_host.so: the C++ host layer.  Built with g++ against include/rt_hip.h only (no HIP headers) and linked to
    librt_hip.so, the way a foreign-language binding would use the C ABI."""
    host = os.path.join(HERE, "host")
    src = os.path.join(host, "rt_host_capi.cpp")
    out = os.path.join(LIB, "librt_host.so")
    deps = [src] + [os.path.join(host, h) for h in ("rt_meta.hpp", "rt_backend.hpp", "rt_tensor.hpp", "rt_expr.hpp", "rt_grad.hpp")] + [h for h in HEADERS if h.endswith('rt_hip.h')]
    if force or _stale(out, deps + [os.path.join(LIB, "librt_hip.so")]):
        cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", out, src, "-L" + LIB, "-lrt_hip", "-Wl,-rpath,$ORIGIN"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"g++ failed on the host layer:\n{r.stdout + r.stderr}")
        if (r.stdout + r.stderr).strip():
            print((r.stdout + r.stderr).strip(), file=sys.stderr)
        print("[build] linked librt_host.so", file=sys.stderr)


if __name__ == "__main__":
    build(force="--force" in sys.argv)
