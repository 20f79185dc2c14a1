#!/usr/bin/env python3
"""Benchmark of the MI355X backend hot path: achieved HBM GB/s (and % of the 8 TB/s peak) per kernel.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--kernel NAME] [--no-cpu] [--no-detail]

One "step" is the headline pair of BASELINE.json's metric at its >= 1 GiB shapes: the strided broadcast add of
config 3 (x (16,1,512,1024) + y (1,64,1,1024) -> 2 GiB f32) followed by the axis sum of config 4 (sum over the last
axis of (8192,32768) f32, 1 GiB).  Inputs are generated on the device and resident in HBM before the timed region.
`value` = algorithmic bytes of one step / time of one step.  Every other kernel of configs 1-5 is timed once more in
`detail`.  `--kernel NAME` runs a single kernel only (used for the rocprofv3 runs whose summaries live in profiles/).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM = 8.0e12   # bytes/s, MI355X HBM3E

# HBM bytes per launch of the config-3 broadcast-add kernel as rocprofv3 counted them (--pmc FETCH_SIZE and --pmc WRITE_SIZE, each scaled
# by what the same counter reads for the 1 GiB copy kernel): read from the committed summary of those runs, not measured by this run.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bin_rows4_kernel_config3_broadcast_add.txt")


def profiled_traffic():
    try:
        for ln in open(TRAFFIC_PROFILE):
            if ln.startswith("traffic_bytes_per_call:"):
                return int(ln.split(":")[1].split()[0])
    except OSError:
        pass
    return None


def profiled_duration_us(path=TRAFFIC_PROFILE, kernel="bin_rows4_kernel"):
    """Average duration of the kernel's timed launches in the committed rocprofv3 kernel trace (the `timed avg us` column of the
    summary): the figure of the machine the profile was taken on, to set beside this run's own."""
    try:
        for ln in open(path):
            if kernel in ln and "blocks" not in ln.split(kernel)[0][-8:] and "FETCH_SIZE" not in ln:
                parts = ln.split()
                try:
                    return float(parts[-1])
                except ValueError:
                    continue
    except OSError:
        pass
    return None


def row_major(shape):
    st = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        st[i] = st[i + 1] * shape[i + 1]
    return st


class Workloads:
    """Builds the device tensors of configs 1-5 lazily and exposes each kernel as a closure `() -> None` plus its
    algorithmic bytes (unique input elements + output elements, times sizeof)."""

    def __init__(self, hip):
        from rtensors_amd import datagen, hip as H
        self.hip, self.H, self.dg = hip, H, datagen
        self._cache = {}

    def _gen(self, name, dtype, n, dist, seed, stream, p0=1.0, p1=0.0):
        key = (name,)
        if key not in self._cache:
            b = self.hip.alloc_uninit(dtype, n)
            self.dg.fill_device(b, dist, seed, stream, p0, p1)
            self._cache[key] = b
        return self._cache[key]

    def _out(self, name, dtype, n):
        key = (name, "out")
        if key not in self._cache:
            self._cache[key] = self.hip.alloc_uninit(dtype, n)
        return self._cache[key]

    def drop(self):
        self._cache.clear()

    # ---- config 3: strided broadcast --------------------------------------------------------------------------------
    def c3a_add(self):
        H = self.H
        x = self._gen("c3x", H.F32, 16 * 512 * 1024, "normal", 2, 0)
        y = self._gen("c3y", H.F32, 64 * 1024, "uniform", 2, 1)
        shape = [16, 64, 512, 1024]
        z = self._out("c3z", H.F32, 16 * 64 * 512 * 1024)
        left = (x, (0, shape, [524288, 0, 1024, 1]))
        right = (y, (0, shape, [0, 1024, 0, 1]))
        dst = (z, (0, shape, row_major(shape)))
        nbytes = (x.len + y.len + z.len) * 4
        return (lambda: self.hip.broadcast(left, right, dst, "add")), nbytes, z.len

    def c3b_add(self):
        # x = contiguous (16,1024,512) .permute([0,2,1]) .slice(1, step -1) .unsqueeze_at(1), broadcast along dim 1:
        # strides (524288, 0, -1, 512), offset 511
        H = self.H
        x = self._gen("c3x", H.F32, 16 * 512 * 1024, "normal", 2, 0)
        y = self._gen("c3y", H.F32, 64 * 1024, "uniform", 2, 1)
        shape = [16, 64, 512, 1024]
        z = self._out("c3z", H.F32, 16 * 64 * 512 * 1024)
        left = (x, (511, shape, [524288, 0, -1, 512]))
        right = (y, (0, shape, [0, 1024, 0, 1]))
        dst = (z, (0, shape, row_major(shape)))
        nbytes = (x.len + y.len + z.len) * 4
        return (lambda: self.hip.broadcast(left, right, dst, "add")), nbytes, z.len

    # ---- config 4: reductions ---------------------------------------------------------------------------------------------
    def _c4(self, dtype_name):
        H = self.H
        if dtype_name == "f32":
            return self._gen("c4t", H.F32, 8192 * 32768, "normal", 3, 0)
        return self._gen("c4i", H.I32, 8192 * 32768, "int", 3, 1, -1000, 1000)

    def _c4_axis(self, dtype_name, op, dim):
        H = self.H
        t = self._c4(dtype_name)
        shape = [8192, 32768]
        nout = shape[1 - dim]
        out = self._out(f"c4o{dim}{dtype_name}", t.dtype, nout)
        src = (t, (0, shape, [32768, 1]))
        return (lambda: self.hip.apply_reduce_contiguous_nd(src, out, dim, op)), (t.len + nout) * 4, t.len

    def c4_sum1(self): return self._c4_axis("f32", "sum", 1)
    def c4_mean1(self): return self._c4_axis("f32", "mean", 1)
    def c4_max1(self): return self._c4_axis("f32", "max", 1)
    def c4_sum0(self): return self._c4_axis("f32", "sum", 0)
    def c4_i32_sum1(self): return self._c4_axis("i32", "sum", 1)
    def c4_i32_max1(self): return self._c4_axis("i32", "max", 1)
    def c4_i32_min0(self): return self._c4_axis("i32", "min", 0)

    # statistics and index reductions on the config-4 tensor (the Cuda backend's other reduction kinds)
    def _c4_stat(self, op, dim):
        H = self.H
        t = self._c4("f32")
        arg = op in ("argmax", "argmin")
        if dim is None:
            out = self._out("c4sall" + ("u64" if arg else ""), H.U64 if arg else t.dtype, 1)
            f = self.hip.apply_argmax_contiguous_flat if arg else self.hip.apply_reduce_contiguous_flat
            return (lambda: f(t, out, 0, t.len, op)), t.len * 4 + (8 if arg else 4), t.len
        shape = [8192, 32768]
        nout = shape[1 - dim]
        out = self._out(f"c4s{dim}" + ("u64" if arg else ""), H.U64 if arg else t.dtype, nout)
        src = (t, (0, shape, [32768, 1]))
        f = self.hip.apply_argmax_contiguous_nd if arg else self.hip.apply_reduce_contiguous_nd
        return (lambda: f(src, out, dim, op)), t.len * 4 + nout * (8 if arg else 4), t.len

    def c4_var1(self): return self._c4_stat("var", 1)
    def c4_std0(self): return self._c4_stat("std", 0)
    def c4_var_all(self): return self._c4_stat("var", None)
    def c4_lse1(self): return self._c4_stat("logsumexp", 1)
    def c4_lse0(self): return self._c4_stat("logsumexp", 0)
    def c4_l2norm1(self): return self._c4_stat("l2_norm", 1)
    def c4_l1norm0(self): return self._c4_stat("l1_norm", 0)
    def c4_argmax1(self): return self._c4_stat("argmax", 1)
    def c4_argmin0(self): return self._c4_stat("argmin", 0)
    def c4_argmax_all(self): return self._c4_stat("argmax", None)

    def _stat_shape(self, op, outer, R, inner):
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        arg = op in ("argmax", "argmin")
        d = self._out("statout" + ("u64" if arg else ""), H.U64 if arg else H.F32, 1 << 26 if not arg else 1 << 25)
        shape, strides = [outer, R, inner], [R * inner, inner, 1]
        f = self.hip.apply_argmax_contiguous_nd if arg else self.hip.apply_reduce_contiguous_nd
        return (lambda: f((a, (0, shape, strides)), d, 1, op)), outer * R * inner * 4 + outer * inner * (8 if arg else 4), outer * R * inner

    def lse_rows10(self): return self._stat_shape("logsumexp", (1 << 28) // 10, 10, 1)       # class scores: rows of 10
    def argmax_rows10(self): return self._stat_shape("argmax", (1 << 28) // 10, 10, 1)
    def lse_rows1000(self): return self._stat_shape("logsumexp", (1 << 28) // 1000, 1000, 1)
    def var_rows256(self): return self._stat_shape("var", 1 << 20, 256, 1)
    def var_inner3(self): return self._stat_shape("var", 1, (1 << 28) // 3, 3)                # per-channel statistics of pixels
    def var_mid64(self): return self._stat_shape("var", 65536, 64, 64)

    # ---- shapes off the configs that have work forms of their own ------------------------------------------------------------
    def _shape(self, op, dtype_name, outer, R, inner):
        """`op` over the middle axis of a (outer, R, inner) view of 1 GiB of normal(0, 1) data."""
        H = self.H
        code, es = (H.F64, 8) if dtype_name == "f64" else (H.F32, 4)
        a = self._gen("gib" + dtype_name, code, (1 << 30) // es, "normal", 1, 0)
        d = self._out("gibout" + dtype_name, code, (1 << 30) // es // 2)
        shape, strides = [outer, R, inner], [R * inner, inner, 1]
        return (lambda: self.hip.apply_reduce_contiguous_nd((a, (0, shape, strides)), d, 1, op)), (outer * R * inner + outer * inner) * es, outer * R * inner

    def lse_f64_rows32768(self): return self._shape("logsumexp", "f64", 4096, 32768, 1)       # f64 logsumexp: the exponential written for it
    def var_rows512(self): return self._shape("var", "f32", 1 << 19, 512, 1)                  # rows of 2 KiB: 16 lanes per row
    def var_f64_rows256(self): return self._shape("var", "f64", 1 << 19, 256, 1)
    def var_mid4(self): return self._shape("var", "f32", 1 << 20, 4, 64)                      # a short middle axis: a lane per output vector
    def sum_slab33x2(self): return self._shape("sum", "f32", (1 << 28) // 66, 33, 2)          # many small slabs with two columns: through LDS
    def lse_slab300x2(self): return self._shape("logsumexp", "f32", (1 << 28) // 600, 300, 2)
    def max_cols128(self): return self._shape("max", "f32", 1, 1 << 21, 128)                  # float max over regrouped rows
    def var_cols50176(self): return self._shape("var", "f32", 1, 5349, 50176)                 # 196 column tiles: the split by rounds of blocks

    def bcast_rows17(self):
        """out (19737, 100, 2, 17) = (19737, 1, 2, 17) + (1, 100, 1, 17): rows of 17 elements under a loop dim of 2 (the flat kernel)."""
        H = self.H
        o = [19737, 100, 2, 17]
        n = o[0] * o[1] * o[2] * o[3]
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        b = self._gen("c2b", H.F32, 1 << 28, "normal", 1, 1)
        d = self._out("c2cf32", H.F32, 1 << 28)
        ls, rs, ds = [2 * 17, 0, 17, 1], [0, 17, 0, 1], [100 * 2 * 17, 2 * 17, 17, 1]
        return (lambda: self.hip.broadcast((a, (0, o, ls)), (b, (0, o, rs)), (d, (0, o, ds)), "add")), (19737 * 34 + 1700 + n) * 4, n

    def c4_sum_all(self):
        t = self._c4("f32")
        out = self._out("c4oall", t.dtype, 1)
        return (lambda: self.hip.apply_reduce_contiguous_flat(t, out, 0, t.len, "sum")), (t.len + 1) * 4, t.len

    # ---- config 2: contiguous elementwise chain ----------------------------------------------------------------------------
    def _c2(self, which, dtype_name="f32"):
        H = self.H
        if dtype_name == "f32":
            dt, n, es = H.F32, 1 << 28, 4
            a = self._gen("c2a", dt, n, "normal", 1, 0); b = self._gen("c2b", dt, n, "normal", 1, 1)
        elif dtype_name == "f64":
            dt, n, es = H.F64, 1 << 27, 8
            a = self._gen("c2a64", dt, n, "normal", 1, 0); b = self._gen("c2b64", dt, n, "normal", 1, 1)
        else:
            dt, n, es = H.I32, 1 << 28, 4
            a = self._gen("c2ai", dt, n, "int", 1, 0, -(1 << 20), 1 << 20); b = self._gen("c2bi", dt, n, "int", 1, 1, -(1 << 20), 1 << 20)
        c = self._out("c2c" + dtype_name, dt, n)
        m = (0, [n], [1])
        three = 3 if dtype_name == "i32" else 3.0
        one = 1 if dtype_name == "i32" else 1.0
        if which == "mul":
            return (lambda: self.hip.scalar_contiguous("mul", a, three, 0, n)), 2 * n * es, n
        if which == "add":
            return (lambda: self.hip.broadcast((a, m), (b, m), (c, m), "add")), 3 * n * es, n
        if which == "relu":
            return (lambda: self.hip.unary_contiguous("relu", c, 0, n)), 2 * n * es, n
        if which == "sub":
            return (lambda: self.hip.scalar_contiguous("sub", c, one, 0, n)), 2 * n * es, n
        if which == "copy":
            return (lambda: self.hip.gather(a, m, c)), 2 * n * es, n
        if which == "fill":
            return (lambda: self.hip.fill_contiguous(c, one, 0, n)), n * es, n
        raise KeyError(which)

    def _c2_fused(self, dtype_name):
        """c = relu(a * 3 + b) - 1 as one rt_fused_chain launch: two reads and one write."""
        H = self.H
        if dtype_name == "f32":
            dt, n, es = H.F32, 1 << 28, 4
            a = self._gen("c2a", dt, n, "normal", 1, 0); b = self._gen("c2b", dt, n, "normal", 1, 1)
        elif dtype_name == "f64":
            dt, n, es = H.F64, 1 << 27, 8
            a = self._gen("c2a64", dt, n, "normal", 1, 0); b = self._gen("c2b64", dt, n, "normal", 1, 1)
        else:
            dt, n, es = H.I32, 1 << 28, 4
            a = self._gen("c2ai", dt, n, "int", 1, 0, -(1 << 20), 1 << 20); b = self._gen("c2bi", dt, n, "int", 1, 1, -(1 << 20), 1 << 20)
        c = self._out("c2c" + dtype_name, dt, n)
        three, one = (3, 1) if dtype_name == "i32" else (3.0, 1.0)
        steps = [("scalar", "mul", three), ("binary", "add", 1), ("unary", "relu"), ("scalar", "sub", one)]
        return (lambda: self.hip.fused_chain([(a, 0), (b, 0)], steps, c, n)), 3 * n * es, n

    def c2_fused(self): return self._c2_fused("f32")
    def c2_fused_f64(self): return self._c2_fused("f64")
    def c2_fused_i32(self): return self._c2_fused("i32")

    def c2_mul(self): return self._c2("mul")
    def c2_add(self): return self._c2("add")
    def c2_relu(self): return self._c2("relu")
    def c2_sub(self): return self._c2("sub")
    def c2_f64_add(self): return self._c2("add", "f64")
    def c2_f64_mul(self): return self._c2("mul", "f64")
    def c2_i32_add(self): return self._c2("add", "i32")
    def c2_i32_mul(self): return self._c2("mul", "i32")
    def copy(self): return self._c2("copy")
    def fill(self): return self._c2("fill")

    def clone(self):
        """Backend::copy of a 1 GiB buffer (what TensorBase::clone / owned() issue), allocation from the cache included."""
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        return (lambda: self.hip.copy(a)), 2 * (1 << 28) * 4, 1 << 28

    def copy_range(self):
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        c = self._out("c2cf32", H.F32, 1 << 28)
        return (lambda: self.hip.copy_range_within(c, a, 0, 0, 1 << 28)), 2 * (1 << 28) * 4, 1 << 28

    def view_relu(self):
        # in-place relu on the left half of a (16384,16384) f32 matrix: a non-contiguous view with unit-stride rows
        H = self.H
        n = 16384
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        return (lambda: self.hip.unary_nd("relu", a, 0, [n, n // 2], [n, 1])), 2 * n * (n // 2) * 4, n * (n // 2)

    def tr_add(self):
        # z = a + b.transpose() on (16384,16384) f32: the right operand's unit-stride dim is the output's row dim
        H = self.H
        n = 16384
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0); b = self._gen("c2b", H.F32, 1 << 28, "normal", 1, 1)
        c = self._out("c2cf32", H.F32, 1 << 28)
        shape = [n, n]
        return (lambda: self.hip.broadcast((a, (0, shape, [n, 1])), (b, (0, shape, [1, n])), (c, (0, shape, [n, 1])), "add")), 3 * n * n * 4, n * n

    # ---- reductions over short rows / narrow columns / a short middle axis (1 GiB f32 each) -------------------------------------------
    def _red(self, outer, R, inner):
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        d = self._out("redout", H.F32, 1 << 26)
        shape, strides = [outer, R, inner], [R * inner, inner, 1]
        return (lambda: self.hip.apply_reduce_contiguous_nd((a, (0, shape, strides)), d, 1, "sum")), (outer * R * inner + outer * inner) * 4, outer * R * inner

    def red_rows32(self): return self._red(1 << 23, 32, 1)
    def red_rows256(self): return self._red(1 << 20, 256, 1)
    def red_inner3(self): return self._red(1, (1 << 28) // 3, 3)
    def red_inner100(self): return self._red(1, (1 << 28) // 100, 100)
    def red_mid64(self): return self._red(65536, 64, 64)
    def red_mid4(self): return self._red(1 << 20, 4, 64)

    # ---- layouts without a unit-stride inner dim (one element per lane kernels) --------------------------------------------------------
    def strided1d_relu(self):
        """In-place relu on every second element of a 2^28 f32 buffer: every cache line is read and written, half of it is used."""
        H = self.H
        c = self._out("c2cf32", H.F32, 1 << 28)
        return (lambda: self.hip.unary_1d_strided("relu", c, 0, 2, 1 << 27)), 2 * (1 << 27) * 4, 1 << 27

    def nd_step2_relu(self):
        """In-place relu on m[:, ::2] of a 16384 x 16384 f32 matrix."""
        H = self.H
        n = 16384
        c = self._out("c2cf32", H.F32, n * n)
        return (lambda: self.hip.unary_nd("relu", c, 0, [n, n // 2], [n, 2])), 2 * (n * n // 2) * 4, n * n // 2

    def generic_step2_add(self):
        """z[:, ::2] = x[:, ::2] + y[:, ::2] on 16384 x 16384 f32 matrices: no operand has a unit-stride inner dim."""
        H = self.H
        n = 16384
        a = self._gen("c2a", H.F32, n * n, "normal", 1, 0); b = self._gen("c2b", H.F32, n * n, "normal", 1, 1)
        c = self._out("c2cf32", H.F32, n * n)
        m = (0, [n, n // 2], [n, 2])
        return (lambda: self.hip.broadcast((a, m), (b, m), (c, m), "add")), 3 * (n * n // 2) * 4, n * n // 2

    # ---- buffer equality and dtype conversion (PartialEq of Backend::Buf, Backend::convert) ------------------------------------------
    def equal_f32(self):
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        b = self._out("c2eq", H.F32, 1 << 28)
        self.hip.copy_range_within(b, a, 0, 0, 1 << 28)
        return (lambda: self.hip.equal(a, b)), 2 * (1 << 28) * 4, 1 << 28

    def convert_f32_f64(self):
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        d = self._out("cvt64", H.F64, 1 << 28)
        return (lambda: self.hip.convert(a, d)), (1 << 28) * 12, 1 << 28

    def convert_f32_i32(self):
        H = self.H
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        d = self._out("cvt32", H.I32, 1 << 28)
        return (lambda: self.hip.convert(a, d)), (1 << 28) * 8, 1 << 28

    # ---- ALU-heavy maps: the f64 logarithm (hand-written) and integer division on the config-3 shapes ---------------------------------------
    def _f64_unary(self, op):
        H = self.H
        n = 1 << 27
        a = self._gen("c2a64", H.F64, n, "uniform", 1, 0)
        z = self._out("c2cf64", H.F64, n)
        return (lambda: self.hip.unary_to(op, a, 0, n, z)), 2 * n * 8, n

    def f64_ln(self): return self._f64_unary("ln")
    def f64_ln1p(self): return self._f64_unary("ln1p")
    def f64_atan(self): return self._f64_unary("atan")

    def __getattr__(self, name):
        """`f64_<op>` for every unary op: the out-of-place map over 1 GiB of f64 (f64_tan, f64_asin, f64_tanh ...); `c3_div_<dtype>` for
        every integer dtype: the division on the config-3 shapes."""
        if name in ("H", "hip", "dg", "_cache"):
            raise AttributeError(name)
        if name.startswith("f64_") and name[4:] in self.H.UNARY:
            return lambda: self._f64_unary(name[4:])
        if name.startswith("c3_div_") and name[7:] in ("u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64"):
            return lambda: self._c3_div(name[7:])
        raise AttributeError(name)

    def _c3_div(self, dtype_name):
        """x / y on the config-3 shapes (x (16,1,512,L) / y (1,64,1,L) -> (16,64,512,L), L = 4 KiB of elements per row), values 1 .. 100."""
        H = self.H
        dt = H.DTYPE_BY_NAME[dtype_name]
        es = H.NP_DTYPE[dt].itemsize
        B, J, K, L = 16, 64, 512, 4096 // es
        def ints(name, n, stream):
            key = (name,)
            if key not in self._cache:
                f = self.hip.alloc_uninit(H.I32, n)
                self.dg.fill_device(f, "int", 2, stream, 1, 100)
                b = self.hip.alloc_uninit(dt, n)
                self.hip.convert(f, b)
                self._cache[key] = b
            return self._cache[key]
        x, y = ints("c3dx" + dtype_name, B * K * L, 0), ints("c3dy" + dtype_name, J * L, 1)
        z = self._out("c3dz" + dtype_name, dt, B * J * K * L)
        shape = [B, J, K, L]
        return (lambda: self.hip.broadcast((x, (0, shape, [K * L, 0, L, 1])), (y, (0, shape, [0, L, 0, 1])), (z, (0, shape, row_major(shape))), "div")), \
            (x.len + y.len + z.len) * es, z.len

    def c3_div_i64(self): return self._c3_div("i64")
    def c3_div_i32(self): return self._c3_div("i32")
    def c3_div_u8(self): return self._c3_div("u8")

    # ---- matmul (behind the same trait; MFMA-bound, not part of the headline) ---------------------------------------------------------
    def _mm(self, dtype_name, n):
        H = self.H
        dt = H.DTYPE_BY_NAME[dtype_name]
        dist = "normal" if dtype_name[0] == "f" else "int"
        a = self._gen(f"mma_{dtype_name}", dt, n * n, dist, 7, 0, -1000, 1000) if dist == "int" else self._gen(f"mma_{dtype_name}", dt, n * n, dist, 7, 0)
        b = self._gen(f"mmb_{dtype_name}", dt, n * n, dist, 7, 1, -1000, 1000) if dist == "int" else self._gen(f"mmb_{dtype_name}", dt, n * n, dist, 7, 1)
        c = self._out(f"mmc_{dtype_name}", dt, n * n)
        meta = (0, [n, n], [n, 1])
        fn = lambda: self.hip.matmul((a, meta, "row_major"), (b, meta, "row_major"), c, 1, n, n, n)
        fn.flops = 2 * n ** 3
        return fn, 3 * n * n * H.NP_DTYPE[dt].itemsize, n * n

    def mm_f32(self): return self._mm("f32", 8192)
    def mm_f64(self): return self._mm("f64", 4096)
    def mm_i32(self): return self._mm("i32", 4096)

    # ---- config 1 -------------------------------------------------------------------------------------------------------------
    def tr_copy(self):
        """Row-major copy of a transposed 16384 x 16384 f32 view (`contiguous()` of `m.transpose()`)."""
        H = self.H
        n = 16384
        a = self._gen("c2a", H.F32, n * n, "normal", 1, 0)
        c = self._out("c2cf32", H.F32, n * n)
        return (lambda: self.hip.gather(a, (0, [n, n], [1, n]), c)), 2 * n * n * 4, n * n

    def gather_rows42(self):
        """Row-major copy of a (64, 3, 2, 4096, 42) f32 view with strides (1, 262144, 786432, 64, 1572864): dst rows of 42 elements,
        src unit-stride along the outermost dim (the N-d tile copy through LDS)."""
        H = self.H
        shape, strides = [64, 3, 2, 4096, 42], [1, 262144, 786432, 64, 1572864]
        n = 64 * 3 * 2 * 4096 * 42
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        c = self._out("c2cf32", H.F32, 1 << 28)
        return (lambda: self.hip.gather(a, (0, shape, strides), c)), 2 * n * 4, n

    def add_perm_rows42(self):
        """c = a + v with v the (64, 3, 2, 4096, 42) view of gather_rows42 and a, c row-major: the add rides on the second stage of the N-d
        tile copy of v.  Algorithmic bytes are the three tensors once."""
        H = self.H
        shape, strides = [64, 3, 2, 4096, 42], [1, 262144, 786432, 64, 1572864]
        n = 64 * 3 * 2 * 4096 * 42
        rm = [3 * 2 * 4096 * 42, 2 * 4096 * 42, 4096 * 42, 42, 1]
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        b = self._gen("c2b", H.F32, 1 << 28, "normal", 1, 1)
        c = self._out("c2cf32", H.F32, 1 << 28)
        return (lambda: self.hip.broadcast((a, (0, shape, rm)), (b, (0, shape, strides)), (c, (0, shape, rm)), "add")), 3 * n * 4, n

    def gather_unit7(self):
        """Row-major copy of a (7, 3300, 2905) f32 view with strides (1, 7, 23100): a (2905, 3300, 7) tensor with its axes reversed,
        whose unit-stride dim has 7 elements."""
        H = self.H
        shape, strides = [7, 3300, 2905], [1, 7, 23100]
        n = 7 * 3300 * 2905
        a = self._gen("c2a", H.F32, 1 << 28, "normal", 1, 0)
        c = self._out("c2cf32", H.F32, 1 << 28)
        return (lambda: self.hip.gather(a, (0, shape, strides), c)), 2 * n * 4, n

    def c1_add(self):
        H = self.H
        a = self._gen("c1a", H.F32, 4096, "uniform", 0, 0); b = self._gen("c1b", H.F32, 4096, "uniform", 0, 1)
        c = self._out("c1c", H.F32, 4096 * 4096)
        shape = [4096, 4096]
        return (lambda: self.hip.broadcast((a, (0, shape, [0, 1])), (b, (0, shape, [1, 0])), (c, (0, shape, [4096, 1])), "add")), \
            (4096 + 4096 + 4096 * 4096) * 4, 4096 * 4096

    def c1_sum1(self):
        H = self.H
        self.c1_add()[0]()
        c = self._out("c1c", H.F32, 4096 * 4096)
        s = self._out("c1s", H.F32, 4096)
        return (lambda: self.hip.apply_reduce_contiguous_nd((c, (0, [4096, 4096], [4096, 1])), s, 1, "sum")), (4096 * 4096 + 4096) * 4, 4096 * 4096

    # ---- config 5: the graded reduction (d(bias) = column sum over the batch dim) and the bias add --------------------------------
    def c5_bias_add(self):
        H = self.H
        x = self._gen("c5x", H.F32, 65536 * 4096, "normal", 4, 0)
        bias = self._gen("c5b", H.F32, 4096, "normal", 4, 1, 0.1)
        y = self._out("c5y", H.F32, 65536 * 4096)
        shape = [65536, 4096]
        return (lambda: self.hip.broadcast((x, (0, shape, [4096, 1])), (bias, (0, shape, [0, 1])), (y, (0, shape, [4096, 1])), "add")), \
            (2 * x.len + 4096) * 4, x.len

    def c5_colsum(self):
        H = self.H
        x = self._gen("c5x", H.F32, 65536 * 4096, "normal", 4, 0)
        g = self._out("c5g", H.F32, 4096)
        return (lambda: self.hip.apply_reduce_contiguous_nd((x, (0, [65536, 4096], [4096, 1])), g, 0, "sum")), (x.len + 4096) * 4, x.len


    # ---- config 5 in three fused passes (rt_fused_*) -----------------------------------------------------------------------------------
    def _c5_fused_bufs(self):
        H = self.H
        n, d = 65536, 4096
        x = self._gen("c5x", H.F32, n * d, "normal", 4, 0)
        t = self._gen("c5t", H.F32, n * d, "uniform", 4, 2)
        bias = self._gen("c5b", H.F32, d, "normal", 4, 1, 0.1)
        y, g = self._out("c5y", H.F32, n * d), self._out("c5gm", H.F32, n * d)
        loss, db = self._out("c5loss", H.F32, 1), self._out("c5g", H.F32, d)
        return n, d, x, t, bias, y, g, loss, db

    def c5_fused_bias_relu(self):
        n, d, x, t, bias, y, g, loss, db = self._c5_fused_bufs()
        return (lambda: self.hip.fused_bias_relu(x, bias, y, n, d)), (2 * n * d + d) * 4, n * d

    def c5_fused_l1_forward(self):
        n, d, x, t, bias, y, g, loss, db = self._c5_fused_bufs()
        self.hip.fused_bias_relu(x, bias, y, n, d)
        return (lambda: self.hip.fused_l1_forward(y, t, g, loss, n * d)), 3 * n * d * 4 + 4, n * d

    def c5_fused_backward(self):
        n, d, x, t, bias, y, g, loss, db = self._c5_fused_bufs()
        self.hip.fused_bias_relu(x, bias, y, n, d)
        self.hip.fused_l1_forward(y, t, g, loss, n * d)
        return (lambda: self.hip.fused_l1_relu_backward(g, y, loss, db, n, d)), (2 * n * d + d) * 4 + 4, n * d

    def c5_fused2_forward(self):
        n, d, x, t, bias, y, g, loss, db = self._c5_fused_bufs()
        return (lambda: self.hip.fused_bias_relu_l1(x, bias, t, y, loss, n, d)), (3 * n * d + d) * 4 + 4, n * d

    def c5_fused2_backward(self):
        n, d, x, t, bias, y, g, loss, db = self._c5_fused_bufs()
        self.hip.fused_bias_relu_l1(x, bias, t, y, loss, n, d)
        return (lambda: self.hip.fused_l1_relu_backward_t(y, t, loss, db, n, d)), (2 * n * d + d) * 4 + 4, n * d


HEADLINE = ["c3a_add", "c4_sum1"]
DETAIL = ["copy", "fill", "c1_add", "c1_sum1", "c2_mul", "c2_add", "c2_relu", "c2_sub", "c2_f64_mul", "c2_f64_add", "c2_i32_mul", "c2_i32_add",
          "c2_fused", "c2_fused_f64", "c2_fused_i32",
          "c3a_add", "c3b_add", "c4_sum1", "c4_mean1", "c4_max1", "c4_sum0", "c4_sum_all", "c4_i32_sum1", "c4_i32_max1", "c4_i32_min0",
          "c4_var1", "c4_std0", "c4_lse1", "c4_argmax1", "c5_bias_add", "c5_colsum", "c5_fused_bias_relu", "c5_fused_l1_forward", "c5_fused_backward", "c5_fused2_forward", "c5_fused2_backward",
          "view_relu", "tr_add", "tr_copy", "gather_rows42", "add_perm_rows42"]
KIND = {"copy": "elementwise", "fill": "elementwise"}


def preheat(hip, fns, seconds):
    """Keeps the device busy for `seconds` of wall time so that the timed region runs at steady clocks."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            for fn in fns:
                fn()
        hip.sync()


def time_kernel(hip, fn, iters, warmup, settle=0.0, block=10):
    """Average duration in ms of one launch of `fn`: (mean over all launches, median and min over blocks of `block` launches),
    HIP events on the backend's own stream.  An event is recorded every `block` launches, not after every launch: an event
    between two launches costs the stream about 5 us (the next kernel waits until the marker has been processed), which a
    caller that just issues kernels never pays and which the rocprofv3 kernel trace of the same launches does not contain.
    `settle`: seconds of the same launch, untimed, before the warm-up.  A kernel with another power profile than its
    predecessor (LDS traffic, more lanes) starts at full speed, is held back for some tens of milliseconds while the board's
    power management finds its level, and then recovers: the staged config-3b add 0.30 ms -> up to 0.42 ms -> 0.305 ms over its
    first hundred launches.  The steady level is what a run of the same kernel sees."""
    if settle > 0:
        preheat(hip, [fn], settle)
    for _ in range(warmup):
        fn()
    block = max(1, min(block, iters))
    nblocks = max(1, iters // block)
    evs = [hip.event() for _ in range(nblocks + 1)]
    hip.record(evs[0])
    for b in range(nblocks):
        for _ in range(block):
            fn()
        hip.record(evs[b + 1])
    hip.sync()
    times = [hip.elapsed_ms(evs[b], evs[b + 1]) / block for b in range(nblocks)]
    return float(np.mean(times)), float(np.median(times)), float(np.min(times))


def api_overhead(hip):
    """Host-side cost of the calls around the kernels, in microseconds per call as seen from this process (the ctypes hop,
    roughly 1-2 us, is included): a cached allocate + free, the asynchronous enqueue of an elementwise, a broadcast and an
    axis-reduce call on tiny operands, and the launch-to-completion round trip of one tiny call."""
    from rtensors_amd import hip as H
    n = 2000
    out = {}
    b = hip.alloc(H.F32, 1 << 18); del b
    hip.sync()
    t0 = time.perf_counter()
    for _ in range(n):
        b = hip.alloc_uninit(H.F32, 1 << 18); del b
    out["alloc_free_cached_1MiB_us"] = round((time.perf_counter() - t0) / n * 1e6, 2)
    a = hip.alloc(H.F32, 64); c = hip.alloc(H.F32, 64 * 64); r = hip.alloc(H.F32, 64)
    shape = [64, 64]
    calls = {
        "enqueue_scalar_contiguous_us": lambda: hip.scalar_contiguous("add", a, 1.0, 0, 64),
        "enqueue_broadcast_rank2_us": lambda: hip.broadcast((a, (0, shape, [0, 1])), (a, (0, shape, [1, 0])), (c, (0, shape, [64, 1])), "add"),
        "enqueue_reduce_axis_us": lambda: hip.apply_reduce_contiguous_nd((c, (0, shape, [64, 1])), r, 1, "sum"),
    }
    for name, fn in calls.items():
        fn(); hip.sync()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        out[name] = round((time.perf_counter() - t0) / n * 1e6, 2)
        hip.sync()
    t0 = time.perf_counter()
    for _ in range(200):
        hip.scalar_contiguous("add", a, 1.0, 0, 64); hip.sync()
    out["round_trip_tiny_call_plus_sync_us"] = round((time.perf_counter() - t0) / 200 * 1e6, 2)
    return out


def host_layer_runs(iters=10):
    """Whole operator sequences issued through the C++ host layer (allocation of every result and temporary included), wall
    clock per iteration: the config-2 chain c = relu(a * 3 + b); c -= 1 and the config-5 training step at full size
    (65536 x 4096).  The reference's operators issue the chain as two clones + four kernels (13 x 1 GiB of traffic); the host
    layer's operators run `a * 3` and `relu(u)` as one out-of-place pass each, so its four kernels move 2 + 3 + 2 + 2 = 9 x 1 GiB
    (`c2_chain_4_kernels_ms`); recorded as an expression (`lazy(a) * 3 + b ...`) it is one fused launch over 3 x 1 GiB (`c2_chain_ms`)."""
    from rtensors_amd import tensor as T
    be = T.Backend(0)
    rng = np.random.default_rng(0)
    out = {}
    n = 1 << 28
    a = T.Tensor.from_buf(be, "f32", rng.standard_normal(n, dtype=np.float32), [n])
    b = T.Tensor.from_buf(be, "f32", rng.standard_normal(n, dtype=np.float32), [n])

    def chain():
        c = ((a * 3.0) + b).relu()
        c -= 1.0
        return c
    for _ in range(3):
        chain()
    be.sync()
    t0 = time.perf_counter()
    for _ in range(iters):
        chain()
    be.sync()
    ms = (time.perf_counter() - t0) / iters * 1e3
    out["c2_chain_4_kernels_ms"] = round(ms, 4)                                # the operators one by one: 9 x 1 GiB of traffic
    out["c2_chain_4_kernels_GBps"] = round(9 * n * 4 / (ms * 1e-3) / 1e9, 1)

    def fused():
        return (((T.lazy(a) * 3.0) + b).relu() - 1.0).eval()                   # the same expression recorded, then one rt_fused_chain launch
    for _ in range(3):
        fused()
    be.sync()
    t0 = time.perf_counter()
    for _ in range(iters):
        fused()
    be.sync()
    ms = (time.perf_counter() - t0) / iters * 1e3
    out["c2_chain_ms"] = round(ms, 4)
    out["c2_chain_GBps"] = round(3 * n * 4 / (ms * 1e-3) / 1e9, 1)             # two reads and one write
    out["c2_chain_bytes"] = 3 * n * 4
    del a, b
    rows, cols = 65536, 4096
    x = T.Tensor.from_buf(be, "f32", rng.standard_normal(rows * cols, dtype=np.float32), [rows, cols])
    target = T.Tensor.from_buf(be, "f32", rng.random(rows * cols, dtype=np.float32) * 2 - 1, [rows, cols])
    bias = T.Tensor.from_buf(be, "f32", rng.standard_normal(cols, dtype=np.float32) * 0.1, [cols])
    # the step in two fused passes (rt_fused_bias_relu_l1 + rt_fused_l1_relu_backward_t: 5 x 1 GiB of traffic), in three (the gradient map
    # stored: 7 x) and on the tape, one backend call per arithmetic step (about 22 x)
    # c5_train_step_ms is the step as the reference's engine can reach it through the trait (the tape); the fused forms need an
    # engine-side change to be used and have keys of their own
    for name, fn in (("c5_train_step_fused2_ms", lambda: T.train_step_fused(x, bias, target, 0.01)),
                     ("c5_train_step_fused3_ms", lambda: T.train_step_fused(x, bias, target, 0.01, True, 3)),
                     ("c5_train_step_ms", lambda: T.train_step(x, bias, target, 0.01))):
        for _ in range(2):
            fn()
        be.sync()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        be.sync()
        out[name] = round((time.perf_counter() - t0) / iters * 1e3, 4)
    out["c5_train_step_fused2_bytes"] = 5 * rows * cols * 4
    out["c5_train_step_fused2_GBps"] = round(out["c5_train_step_fused2_bytes"] / (out["c5_train_step_fused2_ms"] * 1e-3) / 1e9, 1)
    return out


def cpu_baseline():
    """The CPU oracle (C++ restatement of the reference's single-threaded Cpu backend) timed on one whole headline step: the
    config-3 broadcast add (2 GiB out) and the config-4 axis sum (1 GiB in), about 5 s of CPU work on one core."""
    from oracle import cpu
    from oracle.meta import MetaTensor
    from rtensors_amd import datagen
    cpu.build()
    x = datagen.normal(np.float32, 16 * 512 * 1024, 2, 0)
    y = datagen.uniform(np.float32, 64 * 1024, 2, 1)
    shape = [16, 64, 512, 1024]
    z = np.zeros(16 * 64 * 512 * 1024, dtype=np.float32)          # zero-filled: its pages are mapped before the clock starts
    t0 = time.perf_counter()
    cpu.broadcast(cpu.F32, "add", x, MetaTensor(shape, [524288, 0, 1024, 1], 0), y, MetaTensor(shape, [0, 1024, 0, 1], 0),
                  z, MetaTensor(shape, row_major(shape), 0))
    t_add = time.perf_counter() - t0
    add_bytes = (x.size + y.size + z.size) * 4
    del z
    rows = 8192
    t = datagen.normal(np.float32, rows * 32768, 3, 0)
    t0 = time.perf_counter()
    cpu.reduce_nd(cpu.F32, "sum", t, MetaTensor([rows, 32768], [32768, 1], 0), 1)
    t_sum = time.perf_counter() - t0
    sum_bytes = (t.size + rows) * 4
    return {
        "value": round((add_bytes + sum_bytes) / (t_add + t_sum) / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"one whole step, nothing extrapolated: config-3 add ({add_bytes / 2**20:.0f} MiB, {t_add:.2f} s, {add_bytes / t_add / 1e9:.3f} GB/s) "
                  f"+ config-4 sum_at(1) ({sum_bytes / 2**20:.0f} MiB, {t_sum:.2f} s, {sum_bytes / t_sum / 1e9:.3f} GB/s); "
                  f"host has {os.cpu_count()} logical cpus, the reference Cpu backend uses 1",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--preheat", type=float, default=1.5,
                    help="seconds of untimed GPU work during set-up, before the warm-up steps: right after process start the "
                         "device runs below its steady clocks (the same kernel measures 0.40 ms cold and 0.31 ms after ~50 ms of work; "
                         "on some machines the axis sum was still 4 %% slower a quarter of a second in than a few seconds later)")
    ap.add_argument("--kernel", type=str, default=None, help="run only this kernel (see DETAIL) --steps times")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-detail", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    from rtensors_amd import hip as H      # raises if librt_hip.so is missing: there is no CPU fallback
    hip = H.Hip.new(0)
    w = Workloads(hip)

    if args.kernel:
        for name in args.kernel.split(","):                    # several names: one after the other in this process
            fn, nbytes, nelem = getattr(w, name)()
            preheat(hip, [fn], args.preheat)
            mean, med, mn = time_kernel(hip, fn, args.steps, args.warmup)
            rec = {"kernel": name, "ms_mean": mean, "ms_median": med, "ms_min": mn, "bytes": nbytes,
                   "GBps": nbytes / (mean * 1e-3) / 1e9, "frac_of_peak": nbytes / (mean * 1e-3) / PEAK_HBM}
            if hasattr(fn, "flops"):
                rec["TFLOPs"] = fn.flops / (mean * 1e-3) / 1e12
            print(json.dumps(rec), flush=True)
        return

    # ---- headline step ---------------------------------------------------------------------------------------------------
    add_fn, add_bytes, add_elems = w.c3a_add()
    sum_fn, sum_bytes, sum_elems = w.c4_sum1()
    preheat(hip, [add_fn, sum_fn], args.preheat)
    for _ in range(args.warmup):
        add_fn(); sum_fn()
    K = args.steps
    # the timed region: K steps issued as a caller would issue them, one event before and one after, barrier on both sides
    e0, e1 = hip.event(), hip.event()
    hip.sync()
    t0 = time.perf_counter()
    hip.record(e0)
    for i in range(K):
        add_fn()
        sum_fn()
    hip.record(e1)
    hip.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / K
    step_ms_events = hip.elapsed_ms(e0, e1) / K
    step_bytes = add_bytes + sum_bytes
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    # the same K steps once more with an event after every kernel, to split the step between its two kernels.  Every event
    # holds the stream up for about 5 us, so these figures are upper bounds of the kernels' durations inside the step.
    evs = [hip.event() for _ in range(2 * K + 1)]
    hip.record(evs[0])
    for i in range(K):
        add_fn()
        hip.record(evs[2 * i + 1])
        sum_fn()
        hip.record(evs[2 * i + 2])
    hip.sync()
    add_all = [hip.elapsed_ms(evs[2 * i], evs[2 * i + 1]) for i in range(K)]
    sum_all = [hip.elapsed_ms(evs[2 * i + 1], evs[2 * i + 2]) for i in range(K)]
    in_step = {"add_ms": round(float(np.mean(add_all)), 4), "add_ms_median": round(float(np.median(add_all)), 4),
               "sum_ms": round(float(np.mean(sum_all)), 4), "sum_ms_median": round(float(np.median(sum_all)), 4),
               "note": "same K steps repeated with an event after every kernel; each event adds about 5 us to the launch before it"}
    # each kernel on its own, launched back to back (what `rocprofv3 --kernel-trace -- python3 bench.py --kernel c3a_add` times)
    add_ms, add_med, _ = time_kernel(hip, add_fn, 100, 10, settle=0.1)
    sum_ms, sum_med, _ = time_kernel(hip, sum_fn, 100, 10, settle=0.1)

    detail = {}
    if not args.no_detail:
        for name in DETAIL:
            fn, nbytes, nelem = getattr(w, name)()
            mean, med, mn = time_kernel(hip, fn, 60, 10, settle=0.0 if nbytes < (1 << 28) else 0.1)
            detail[name] = {"ms": round(mean, 4), "ms_median": round(med, 4), "GBps": round(nbytes / (mean * 1e-3) / 1e9, 1),
                            "frac": round(nbytes / (mean * 1e-3) / PEAK_HBM, 4), "Gelem_s": round(nelem / (mean * 1e-3) / 1e9, 2)}
    w.drop()
    if not args.no_detail:
        detail["api_overhead"] = api_overhead(hip)
        detail["host_layer"] = host_layer_runs()

    out = {
        "metric": "achieved HBM GB/s (% of peak) for broadcast-add + axis-sum, f32, 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 3 strided broadcast add x(16,1,512,1024)+y(1,64,1,1024)->(16,64,512,1024) f32 (2 GiB out), "
                               "then config 4 sum over the last axis of (8192,32768) f32 (1 GiB in)",
                   "bytes_per_step": step_bytes, "pct_of_peak": round(100 * value * 1e9 / PEAK_HBM, 2)},
        "step_ms_by_events": round(step_ms_events, 4),
        # achieved / frac / kernel_ms: the add kernel inside the alternating add / sum steps (mean over K steps, HIP events on the
        # backend stream, one after every kernel; each event holds the stream for about 5 us, so the figure is a lower bound of the
        # kernel's own rate).  standalone: the same kernel launched back to back, outside the steps.  profile: the kernel's average
        # duration in the committed rocprofv3 trace (another machine, another day) and the fraction that duration implies.
        "roofline": {"bound": "hbm", "kernel": "bin_rows4_kernel<float, add, vec, vec> (config 3 broadcast add)",
                     "achieved": round(add_bytes / (in_step["add_ms"] * 1e-3) / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(add_bytes / (in_step["add_ms"] * 1e-3) / PEAK_HBM, 4), "traffic": profiled_traffic(),
                     "traffic_source": "profiles/" + os.path.basename(TRAFFIC_PROFILE) + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured by this run)",
                     "measured": "inside the add / sum steps: K steps with a HIP event after every kernel (each event costs the stream about 5 us)",
                     "kernel_ms": in_step["add_ms"], "kernel_ms_median": in_step["add_ms_median"],
                     "frac_median": round(add_bytes / (in_step["add_ms_median"] * 1e-3) / PEAK_HBM, 4),
                     "in_step": in_step,
                     "standalone": {"kernel_ms": round(add_ms, 4), "kernel_ms_median": round(add_med, 4),
                                    "achieved": round(add_bytes / (add_ms * 1e-3) / 1e9, 1), "frac": round(add_bytes / (add_ms * 1e-3) / PEAK_HBM, 4),
                                    "measured": "100 launches back to back, a HIP event every 10 launches"},
                     "profile": (lambda us: {"timed_avg_us": us, "frac_profile": round(add_bytes / (us * 1e-6) / PEAK_HBM, 4) if us else None,
                                             "source": "profiles/" + os.path.basename(TRAFFIC_PROFILE) + " (rocprofv3 --kernel-trace of `bench.py --kernel c3a_add`, the machine that took the profile)"})(profiled_duration_us()),
                     "axis_sum": {"kernel": "reduce_rows_block_kernel<sum, float>", "achieved": round(sum_bytes / (in_step["sum_ms"] * 1e-3) / 1e9, 1),
                                  "frac": round(sum_bytes / (in_step["sum_ms"] * 1e-3) / PEAK_HBM, 4), "kernel_ms": in_step["sum_ms"],
                                  "kernel_ms_median": in_step["sum_ms_median"],
                                  "standalone": {"kernel_ms": round(sum_ms, 4), "kernel_ms_median": round(sum_med, 4),
                                                 "frac": round(sum_bytes / (sum_ms * 1e-3) / PEAK_HBM, 4)},
                                  "profile": (lambda us: {"timed_avg_us": us, "frac_profile": round(sum_bytes / (us * 1e-6) / PEAK_HBM, 4) if us else None,
                                                          "source": "profiles/reduce_rows_block_kernel_config4_sum_last_axis.txt"})(
                                      profiled_duration_us(os.path.join(ROOT, "profiles", "reduce_rows_block_kernel_config4_sum_last_axis.txt"), "reduce_rows_block_kernel"))}},
        "detail": detail,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
