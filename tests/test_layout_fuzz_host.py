"""The library's descriptor checks (rt_check_extent, rt_collapse, the overlap test; rtensors_amd/csrc/rt_layout.hip) on the CPU, built
with AddressSanitizer + UndefinedBehaviorSanitizer and fuzzed.  No GPU is involved: the checks are host code that runs before any
launch, reached through the context-free entry points rt_debug_check_view / rt_debug_check_overlap.

What is held against what:
  * status and element count against `oracle.meta.check_extent` (the reference's remote-server validator, backend/remote/server.rs:
    241-275, in exact integers), for descriptors with values up to 2^64 - 1 and strides down to -2^63;
  * the canonical layout against properties, not against a second copy of the algorithm: it addresses exactly the same set of elements
    as the view (enumerated for small views; lowest / highest address and count for huge ones), its strides are non-negative and sorted,
    no dim has size 1 and no two neighbouring dims could still be merged;
  * the overlap answer against interval arithmetic on the exact bounds."""
import os
import random
import subprocess

import pytest

from oracle.meta import check_extent, view_bounds

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
STATUS = {0: "ok", 1: "invalid", 3: "out_of_bounds", 6: "rank"}
U64 = (1 << 64) - 1


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    d = tmp_path_factory.mktemp("layout_fuzz")
    obj, drv, exe = str(d / "rt_layout.o"), str(d / "driver.o"), str(d / "layout_fuzz")
    san = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-gpu-sanitize"]
    flags = ["--offload-host-only", "-x", "hip", "-O1", "-g", "-std=c++17"] + san
    r = subprocess.run(["hipcc"] + flags + ["-c", os.path.join(ROOT, "rtensors_amd", "csrc", "rt_layout.hip"), "-o", obj], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run(["hipcc"] + flags + ["-c", os.path.join(HERE, "support", "layout_fuzz.cpp"), "-o", drv], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run(["hipcc", "--offload-host-only"] + san + [drv, obj, "-o", exe, "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


def run(driver, lines):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([driver], input="\n".join(lines) + "\n", capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and not r.stderr.strip(), (r.returncode, r.stderr[-4000:])
    out = r.stdout.strip().split("\n")
    assert len(out) == len(lines)
    return [[int(x) for x in ln.split()] for ln in out]


def random_view(rng: random.Random, big: bool):
    rank = rng.choice([0, 1, 1, 2, 2, 3, 4, 5, 8, 9, 12])
    if big:
        pick_dim = lambda: rng.choice([0, 1, 2, 3, 1 << 31, (1 << 32) + 1, 1 << 62, 1 << 63, U64, rng.getrandbits(64)])
        pick_stride = lambda: rng.choice([0, 1, -1, 2, -(1 << 63), (1 << 63) - 1, rng.getrandbits(63), -rng.getrandbits(63), 1 << 40])
        shape = [pick_dim() for _ in range(rank)]
        strides = [pick_stride() for _ in range(rank)]
        offset = rng.choice([0, 1, U64, 1 << 63, rng.getrandbits(64), rng.getrandbits(20)])
        length = rng.choice([0, 1, U64, 1 << 63, rng.getrandbits(64), rng.getrandbits(30)])
        return offset, shape, strides, length
    shape = [rng.choice([1, 1, 2, 3, 4, 5, 7]) if rng.random() > 0.03 else 0 for _ in range(rank)]
    # a mostly valid view: strides of a row-major tensor, stepped / reversed / permuted / repeated, sometimes pushed out of bounds
    full = [d * rng.choice([1, 1, 2, 3]) for d in shape]
    st, acc = [0] * rank, 1
    for i in range(rank - 1, -1, -1):
        st[i] = acc
        acc *= max(full[i], 1)
    order = list(range(rank))
    if rng.random() < 0.4:
        rng.shuffle(order)
    shape = [shape[i] for i in order]
    strides = [st[i] * rng.choice([1, 1, 1, 2, -1, -2, 0]) for i in order]
    lo, hi = view_bounds(0, [max(d, 1) for d in shape], strides)
    offset = -lo + rng.choice([0, 0, 0, 1, 5])
    length = offset + hi + 1 + rng.choice([0, 0, 0, 3, -1, -2])
    if rng.random() < 0.05:
        offset = max(0, offset - rng.choice([1, 2]))
    return offset, shape, strides, max(length, 0)


def elements(offset, shape, strides):
    out = [offset]
    for d, s in zip(shape, strides):
        out = [o + k * s for o in out for k in range(d)]
    return out


def test_extent_check_and_canonical_layout(driver):
    rng = random.Random(20240)
    cases = [random_view(rng, big=i % 3 == 0) for i in range(30_000)]
    cases += [(0, [], [], 1), (0, [], [], 0), (5, [], [], 5), (0, [0], [1], 0), (1, [0], [1], 0), (3, [4], [-1], 4), (2, [4], [-1], 4), (0, [1 << 63, 4, 0], [1, 1, 1], 10),
              (0, [0, 1 << 63, 4], [1, 1, 1], 10), (0, [U64, U64], [0, 0], 1), (0, [3, 3], [0, 0], 1), (0, [1 << 63], [0], 1), (0, [(1 << 63) - 1], [0], 1)]
    lines = [f"V {off} {ln} {len(sh)} " + " ".join(map(str, sh)) + " " + " ".join(map(str, st)) for off, sh, st, ln in cases]
    got = run(driver, lines)
    seen = {"ok": 0, "invalid": 0, "out_of_bounds": 0, "rank": 0}
    for (off, sh, st, ln), g in zip(cases, got):
        status, count, orank, ooff = g[:4]
        want, n = check_extent(off, sh, st, ln)
        if STATUS.get(status) == "rank":
            assert want == "ok" and len([d for d in sh if d != 1]) > 8, (off, sh, st, ln)
            seen["rank"] += 1
            continue
        assert STATUS.get(status) == want, (off, sh, st, ln, status, want)
        seen[want] += 1
        if want != "ok":
            continue
        assert count == n
        if n == 0:
            continue
        cshape, cstr = g[4:4 + orank], g[4 + orank:4 + 2 * orank]
        assert all(d > 1 for d in cshape) and all(s >= 0 for s in cstr) and cstr == sorted(cstr, reverse=True), (sh, st, cshape, cstr)
        for i in range(orank - 1):
            assert cstr[i] != cstr[i + 1] * cshape[i + 1], ("dims left unmerged", sh, st, cshape, cstr)
        m = 1
        for d in cshape:
            m *= d
        assert m == n
        assert (ooff, ooff + sum((d - 1) * s for d, s in zip(cshape, cstr))) == view_bounds(off, sh, st)
        if n <= 4096:
            assert sorted(elements(ooff, cshape, cstr)) == sorted(elements(off, sh, st)), (off, sh, st, ooff, cshape, cstr)
    assert min(seen["ok"], seen["invalid"], seen["out_of_bounds"]) > 500, seen


def test_overlap_answers(driver):
    rng = random.Random(77)
    cases = []
    while len(cases) < 10_000:
        off, sh, st, ln = random_view(rng, big=False)
        if check_extent(off, sh, st, ln)[0] != "ok":
            continue
        k = rng.random()
        if k < 0.25:
            off2, st2 = off, list(st)                                        # the very same view
        elif k < 0.5:
            off2, st2 = off, [s if d > 1 else s + 7 for d, s in zip(sh, st)]  # same but for strides of size-1 dims, which address nothing
        else:
            o2, s2, t2, l2 = random_view(rng, big=False)
            if len(s2) != len(sh):
                continue
            off2, st2 = o2, t2
        if check_extent(off2, sh, st2, ln)[0] != "ok":
            continue
        cases.append((rng.choice([1, 2, 4, 8, 16]), ln, sh, off, st, off2, st2))
    lines = [f"O {es} {ln} {len(sh)} " + " ".join(map(str, sh)) + f" {a} " + " ".join(map(str, sa)) + f" {b} " + " ".join(map(str, sb)) for es, ln, sh, a, sa, b, sb in cases]
    got = run(driver, lines)
    meets = sames = 0
    for (es, ln, sh, a, sa, b, sb), (status, meet, same) in zip(cases, got):
        assert status == 0
        if 0 in sh:
            assert (meet, same) == (0, 0)
            continue
        (alo, ahi), (blo, bhi) = view_bounds(a, sh, sa), view_bounds(b, sh, sb)
        assert meet == int(alo <= bhi and blo <= ahi), (sh, a, sa, b, sb)
        assert same == int(a == b and all(x == y for d, x, y in zip(sh, sa, sb) if d > 1)), (sh, a, sa, b, sb)
        meets += meet
        sames += same
    assert meets > 1000 and sames > 1000 and meets < len(cases)


def test_the_exported_entry_points_agree_with_the_sanitized_build(driver):
    """The same answers from the shipped library (librt_hip.so loads without a GPU; these two entry points need no context)."""
    import ctypes as C
    from rtensors_amd._ffi import lib
    rng = random.Random(5)
    cases = [random_view(rng, big=i % 2 == 0) for i in range(2000)]
    lines = [f"V {off} {ln} {len(sh)} " + " ".join(map(str, sh)) + " " + " ".join(map(str, st)) for off, sh, st, ln in cases]
    got = run(driver, lines)
    for (off, sh, st, ln), g in zip(cases, got):
        r = len(sh)
        shape = (C.c_uint64 * max(r, 1))(*sh)
        strides = (C.c_int64 * max(r, 1))(*st)
        count, orank, ooff = C.c_uint64(0), C.c_int32(0), C.c_int64(0)
        oshape, ostr = (C.c_int64 * 8)(), (C.c_int64 * 8)()
        status = lib.rt_debug_check_view(off, r, shape, strides, ln, C.byref(count), C.byref(orank), oshape, ostr, C.byref(ooff))
        assert status == g[0]
        if status == 0:
            assert (count.value, orank.value) == (g[1], g[2])
            if count.value:
                assert [ooff.value] + list(oshape[:orank.value]) + list(ostr[:orank.value]) == g[3:]
