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

# -ffp-contract=off / no fast-math: float results must be the plain IEEE operations the reference's Cpu backend does.
# -packed-fp32-ops is switched off on purpose (scalar v_add/v_mul/v_fma f32 only).
FLAGS = [
    "-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
    # the device code of each object is stored zstd-compressed and unpacked by the HIP runtime when the library is loaded
    "--offload-compress",
]

LIBS = {
    "librt_hip.so": ["rt_runtime.hip", "rt_layout.hip", "rt_elementwise.hip", "rt_broadcast.hip", "rt_broadcast_tile.hip", "rt_reduce.hip", "rt_reduce_stat.hip", "rt_misc.hip", "rt_matmul.hip", "rt_fused.hip"],
    "librt_datagen.so": ["rt_datagen.hip"],
}
HEADERS = [os.path.join(CSRC, "rt_common.h"), os.path.join(CSRC, "rt_broadcast_common.h"), os.path.join(CSRC, "rt_div128.h"),
           os.path.join(HERE, "..", "include", "rt_hip.h")]


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
            r = subprocess.run(["hipcc", f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", out] + deps + ["-ldl", "-lpthread"], capture_output=True, text=True)
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
    deps = [src] + [os.path.join(host, h) for h in ("rt_meta.hpp", "rt_backend.hpp", "rt_tensor.hpp", "rt_expr.hpp", "rt_grad.hpp")] + HEADERS[3:]
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
