#!/usr/bin/env python3
"""Benchmark of the axis primitives on one MI355X.

A step is one pass of the scan / long-reduce configuration (BASELINE.json
configs[1]): inclusive cumsum along the last axis of int32 [64, 2^20] and of
fp32 [64, 2^20], then a 1-D fp32 reduce_sum over 2^30 elements, all inputs
resident in HBM before the timed region starts.  `value` is the algorithmic
bytes of the step (every input element read once, every output element written
once) divided by the wall time of the K timed steps.

Per-operation figures for every configuration (Gelem/s, GB/s, fraction of the
8 TB/s HBM peak) are reported in `per_op`; `roofline` describes the kernel that
dominates the step; `cpu_baseline` times the CPU restatement of the reference's
algorithm on this box's host cores on a bounded sample of the same workload.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs all|step|...] [--no-cpu]
Prints ONE JSON line on stdout.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the library's kernels come from the committed profiler summary (two
# rocprofv3 --pmc runs of this script, FETCH_SIZE then WRITE_SIZE, each scaled by what the
# counter reads for a plain 1 GiB device copy): a counter cannot be read from inside the timed
# run, so the figures are those of the kernels as profiled, looked up by kernel name.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_all_configs_hbm_traffic_pmc.txt")


def profiled_traffic():
    """{(configuration, kernel name as the profile prints it): HBM bytes per launch} from the lines
    `traffic_bytes_per_launch <bytes> <configuration> <kernel>` of the committed summary ({} when
    it is absent).  The profile is taken one configuration (C1 ... C5) at a time, so a kernel that
    several configurations launch at different sizes has a figure for each."""
    out = {}
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch "):
                    _, nbytes, config, name = line.rstrip("\n").split(" ", 3)
                    out[(config, name)] = int(nbytes)
    except OSError:
        pass
    return out


def traffic_of(kernels, table, config):
    """Sum over the kernels of one call (name prefixes) as profiled for the operation's
    configuration; None when any is missing from the profile."""
    if not kernels or not table:
        return None
    total = 0
    for k in ([kernels] if isinstance(kernels, str) else kernels):
        hit = [v for (c, name), v in table.items() if c == config[:2] and name.startswith(k)]
        if not hit:
            return None
        total += hit[0]
    return total


FAMILY_OF = (("top_k", "top_k"), ("argsort", "sort"), ("sort", "sort"), ("cumsum", "scan"),
             ("reduce_", "reduce"), ("argmax", "reduce"), ("log_sum_exp", "reduce"))


def family_of(op_name):
    for prefix, family in FAMILY_OF:
        if op_name.startswith(prefix):
            return family
    return None


# outputs whose error exceeds 4 ulp x log2(n) of the fp64 result itself (no allowance for
# cancellation), counted by the fp32 cumsum gates: {operation: count}
STRICT_FAILURES = {}

METRIC = "HBM GB/s (% of ~8 TB/s peak) + Gelem/s per op: reduce, scan, top_k, sort"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Op:
    """One measured operation: a list of prepared calls over rotated input buffers."""

    def __init__(self, config, name, elems, alg_bytes, calls, verify=None, kernel=None):
        self.config, self.name, self.elems, self.alg_bytes = config, name, elems, alg_bytes
        self.calls, self.verify, self.kernel = calls, verify, kernel
        self._i = 0

    def issue(self):
        self.calls[self._i % len(self.calls)]()
        self._i += 1


def make_ops(be, which):
    want = set(which.split(","))
    def on(*names):
        return bool(want & set(names))
    import numpy as np
    import torch
    from dlf_amd import frontend as F
    from dlf_amd import synth
    from dlf_amd.frontend import Tensor, dtype_code, prepare_reduce
    from dlf_amd.shape import Shape

    dev = be.device
    np_of = {torch.float32: np.float32, torch.int32: np.int32, torch.int64: np.int64, torch.float64: np.float64, torch.float16: np.float16}

    def tensor(t):
        return Tensor(be, Shape(list(t.shape)), t.view(-1), np_of[t.dtype])

    def gen(shape, dtype, fn, copies):
        out = []
        for c in range(copies):
            t = torch.empty(shape, dtype=dtype, device=dev)
            synth.fill(t, fn(c))
            out.append(t)
        return out

    def empty(shape, dtype):
        return torch.empty(shape, dtype=dtype, device=dev)

    def reduce_calls(name, xs, axes):
        calls, outs = [], []
        for x in xs:
            X = tensor(x)
            view, out_dims, m, n = prepare_reduce(X.shape, list(axes), False)
            Y = Tensor.empty(be, out_dims, X.dtype)
            calls.append(be.reduce(name, dtype_code(X.dtype), m, n, view, X.storage, Y.shape, Y.storage, defer=True))
            outs.append(Y)
        return calls, outs

    def argmax_calls(xs, axis):
        calls, outs = [], []
        for x in xs:
            X = tensor(x)
            view = X.shape.moveaxis(axis, -1)
            y_dims = [e for i, e in enumerate(X.shape.extents) if i != axis]
            Y = Tensor.empty(be, y_dims, np.int32)
            k = view.extents[-1]
            calls.append(be.arg_reduce("argmax", dtype_code(X.dtype), 2, view.size // k, k, view, X.storage,
                                       Y.shape, Y.storage, defer=True))
            outs.append(Y)
        return calls, outs

    def scan_calls(xs, axis):
        y = empty(xs[0].shape, xs[0].dtype)
        Y = tensor(y)
        calls = []
        for x in xs:
            X = tensor(x)
            n = X.shape.extents[axis]
            calls.append(be.scan("cumsum", dtype_code(X.dtype), X.size // n, n, False,
                                 X.shape.moveaxis(axis, -1), X.storage, Y.shape.moveaxis(axis, -1), Y.storage, defer=True))
        return calls, y

    ops = []

    # ---------------- ceilings: what the memory system gives a plain two-way and a one-way stream
    # at the sizes of C2 and C5 (dlfx_copy of a dense view = one 128-bit non-temporal load and
    # store per thread; the one-way stream is the library's reduce_max over rows of 4096, a workgroup a row)
    if on("all", "ceil", "ceilbig"):
        sizes = []
        if on("all", "ceil"):
            sizes += [("[64,2^20]", (64, 1 << 20), 4), ("[32,512,56,56]", (32, 512, 56, 56), 4)]
        if on("ceilbig"):
            # the same two streams at 1 GiB and 4 GiB: what the memory system gives once a launch is
            # long enough for its ramp-up and tail not to matter
            sizes += [("[2^28]", (1 << 16, 4096), 2), ("[2^30]", (1 << 18, 4096), 1)]
        for label, shape, copies in sizes:
            xs = gen(shape, torch.float32, lambda c: synth.normal(900 + c), copies)
            y = empty(shape, torch.float32)
            count = xs[0].numel()
            dense = [count]
            calls = [be.copy(dtype_code(np.float32), dense, x.view(-1), 0, [1], y.view(-1), 0, [1], defer=True) for x in xs]

            def v_copy(x=xs[0], y=y, call=calls[0]):
                call()
                assert torch.equal(x, y), "copy"
            ops.append(Op("ceil", "copy_f32_" + label, count, 8 * count, calls, v_copy, "copy_dense"))
            rows = [x.view(-1, 4096) for x in xs]
            calls, outs = reduce_calls("reduce_max", rows, [1])

            def v_read(x=rows[0], out=outs[0], call=calls[0]):
                call()
                assert torch.equal(out.storage.view(-1), x.max(dim=1).values), "reduce_max"
            ops.append(Op("ceil", "read_f32_" + label, count, 4 * count + 4 * (count // 4096), calls, v_read, "reduce_rows_block"))

    # ---------------- C2: scans and the long reduce (the step)
    if on("all", "step", "c2"):
        xi = gen((64, 1 << 20), torch.int32, lambda c: synth.randint(2 + 100 * c, 0, 100), 4)
        calls, y = scan_calls(xi, 1)

        def v_c2a(xi=xi, y=y, call=calls[0]):
            call()
            assert torch.equal(y, torch.cumsum(xi[0], 1, dtype=torch.int32)), "C2a cumsum int32 not bit-exact"
        ops.append(Op("C2a", "cumsum_i32_[64,2^20]", 64 << 20, 2 * 4 * (64 << 20), calls, v_c2a, "scan_rows_chained"))

        xf = gen((64, 1 << 20), torch.float32, lambda c: synth.normal(3 + 100 * c), 4)
        calls, yf = scan_calls(xf, 1)

        def v_c2b(xf=xf, y=yf, call=calls[0]):
            call()
            want = torch.cumsum(xf[0].double(), 1)
            mag = torch.cumsum(xf[0].double().abs(), 1)
            err = (y.double() - want).abs()
            tol = 4 * 20 * float(np.finfo(np.float32).eps) * torch.maximum(want.abs(), mag)
            assert bool((err <= tol).all()), "C2b cumsum fp32 out of tolerance"
            # prefixes cross zero, so a bound relative to the prefix alone is ill-posed: counted, not gated
            STRICT_FAILURES["C2b cumsum_f32_[64,2^20]"] = int((err > 4 * 20 * float(np.finfo(np.float32).eps) * want.abs()).sum())
        ops.append(Op("C2b", "cumsum_f32_[64,2^20]", 64 << 20, 2 * 4 * (64 << 20), calls, v_c2b, "scan_rows_chained"))

        xl = gen((1 << 30,), torch.float32, lambda c: synth.unit_interval_exact(4), 1)
        calls, outs = reduce_calls("reduce_sum", xl, [])

        def v_c2c(xl=xl, out=outs[0], call=calls[0]):
            call()
            # every element is a multiple of 2^-23 below 1 in magnitude: the fp64 sum is exact
            want = float(xl[0].double().sum())
            got = float(out.storage[0])
            assert abs(got - want) <= 4 * 30 * float(np.finfo(np.float32).eps) * max(abs(want), 1.0), (got, want)
        ops.append(Op("C2c", "reduce_sum_f32_[2^30]", 1 << 30, 4 * (1 << 30) + 4, calls, v_c2c, "reduce_rows_block"))

    # ---------------- C1: logits head
    if on("all", "c1"):
        x1 = gen((256, 1000), torch.float32, lambda c: synth.normal(1 + 100 * c), 8)
        for name in ("reduce_sum", "reduce_max", "reduce_log_sum_exp"):
            calls, outs = reduce_calls(name, x1, [1])

            def v(name=name, x=x1[0], out=outs[0], call=calls[0]):
                call()
                ref = {"reduce_sum": lambda t: t.double().sum(1), "reduce_max": lambda t: t.double().amax(1),
                       "reduce_log_sum_exp": lambda t: torch.logsumexp(t.double(), 1)}[name](x)
                assert torch.allclose(out.storage[:256].double(), ref, rtol=1e-5, atol=1e-5), name
            ops.append(Op("C1", name + "_f32_[256,1000]", 256000, 1024000 + 1024, calls, v))
        calls, outs = argmax_calls(x1, 1)

        def v_am(x=x1[0], out=outs[0], call=calls[0]):
            call()
            assert torch.equal(out.storage[:256].long(), torch.argmax(x, 1))
        ops.append(Op("C1", "argmax_f32_[256,1000]", 256000, 1024000 + 1024, calls, v_am))
        ops += topk_ops(be, tensor, x1, [5], "C1", "[256,1000]")
        # the same five results from one launch (dlfx_logits_head); reported beside C1, not part of it
        hs, hm, hl = (empty((256,), torch.float32) for _ in range(3))
        ha = torch.empty(256, dtype=torch.int32, device=dev)
        hv = empty((256, 5), torch.float32)
        hi = torch.empty((256, 5), dtype=torch.int32, device=dev)
        calls = [be.logits_head(dtype_code(np.float32), 256, 1000, x.view(-1), 0, 1000, hs, hm, ha, hl, 5, hv, hi, defer=True) for x in x1]

        def v_head(x=x1[0], call=calls[0]):
            call()
            assert torch.allclose(hs.double(), x.double().sum(1), rtol=1e-5, atol=1e-5)
            assert torch.equal(hm, x.amax(1)) and torch.equal(ha.long(), torch.argmax(x, 1))
            assert torch.allclose(hl.double(), torch.logsumexp(x.double(), 1), rtol=1e-5, atol=1e-5)
            top = torch.topk(x, 5, dim=1)
            assert torch.equal(hv, top.values) and torch.equal(torch.gather(x, 1, hi.long()), hv)
        ops.append(Op("C1f", "logits_head(sum,max,argmax,lse,top_k5)_f32_[256,1000]", 256000, 1024000 + 256 * 56, calls, v_head,
                      "logits_head_rows"))

    # ---------------- C3: top_k
    if on("all", "c3"):
        x3 = gen((4096, 32000), torch.float32, lambda c: synth.quantised_normal(5 + 100 * c), 4)
        ops += topk_ops(be, tensor, x3, [1, 5, 50, 256], "C3", "[4096,32000]")

    # ---------------- C4: sort / argsort
    if on("all", "c4"):
        x4a = gen((1024, 65536), torch.float32, lambda c: synth.quantised_uniform(6 + 100 * c), 4)
        ops += sort_ops(be, tensor, x4a, "C4a", "f32_[1024,65536]")
        x4b = gen((256, 1 << 20), torch.int64, lambda c: synth.full_range_i64(7), 1)
        ops += sort_ops(be, tensor, x4b, "C4b", "i64_[256,2^20]")

    # ---------------- beside the baseline's configurations: float rows on both sides of zero
    # (N(0,1) values at the C4a shape, at the row length from which the images of such rows have
    # the gap around zero closed, and doubles); not part of all
    if on("spread"):
        for shape, dtype, text in (((1024, 65536), torch.float32, "f32_normal_[1024,65536]"),
                                   ((2048, 32768), torch.float32, "f32_normal_[2048,32768]"),
                                   ((512, 65536), torch.float64, "f64_normal_[512,65536]")):
            xs = gen(shape, dtype, lambda c: synth.normal(9 + 100 * c), 4)
            ops += sort_ops(be, tensor, xs, "C4n", text)

    # ---------------- beside the baseline's configurations: rows that evenly spaced bins do not cut -
    # one value, ten values, and nine keys in ten inside a window of 1000 values with the rest
    # spread over the whole range (at the C4 shapes and as one long row); not part of all
    if on("repeats"):
        def clustered(seed):
            wide, near, pick = synth.full_range_i64(seed), synth.randint(seed + 1, 0, 1000), synth.randint(seed + 2, 0, 10)
            return lambda idx: torch.where(pick(idx) > 0, near(idx) + 12345, wide(idx))
        for shape, dtype, fn, text in (((1024, 65536), torch.float32, lambda c: synth.randint(40 + 100 * c, 0, 10), "f32_ten_values_[1024,65536]"),
                                       ((256, 1 << 20), torch.int64, lambda c: (lambda idx: torch.full_like(idx, 7)), "i64_one_value_[256,2^20]"),
                                       ((256, 1 << 20), torch.int64, lambda c: synth.randint(41 + 100 * c, 0, 10), "i64_ten_values_[256,2^20]"),
                                       ((256, 1 << 20), torch.int64, lambda c: clustered(42 + 100 * c), "i64_clustered_[256,2^20]"),
                                       ((1, 2500000), torch.int64, lambda c: clustered(43 + 100 * c), "i64_clustered_[1,2500000]"),
                                       ((1, 2500000), torch.int64, lambda c: synth.full_range_i64(44 + 100 * c), "i64_[1,2500000]")):
            xs = gen(shape, dtype, fn, 2)
            ops += [op for op in sort_ops(be, tensor, xs, "C4r", text) if "_asc_" in op.name]

    # ---------------- beside the baseline's configurations: shapes at which a sweep found a step in the
    # time per element (each named with what takes it now); not part of all
    if on("beside"):
        def timed_only(call):
            def v(call=call):
                call()
            return v

        def enough(shape, dtype):
            # copies to rotate through: a working set of 1.3 GB, so that the 256 MB cache in front of HBM holds none of them
            size = int(np.prod(shape)) * torch.empty((), dtype=dtype).element_size()
            return max(2, min(12, -(-1300000000 // size)))
        # scans and reductions along an axis that is not the innermost
        for shape, axis, what in (((262144, 64), 0, "few columns: the axis cut into segments"), ((4194304, 16), 0, "few columns: the axis cut into segments"),
                                  ((16384, 1000), 0, "the axis cut into segments"), ((8, 21, 512, 512), 1, "a short axis: a lane per column"),
                                  ((64, 3, 224, 224), 1, "a short axis: a lane per column")):
            xs = gen(shape, torch.float32, lambda c: synth.normal(50 + 100 * c), enough(shape, torch.float32))
            text = "_f32_[%s]" % ",".join(str(e) for e in shape)
            count = int(np.prod(shape))
            calls, _ = scan_calls(xs, axis)
            ops.append(Op("B1", "cumsum{%d}%s" % (axis, text), count, 8 * count, calls, timed_only(calls[0])))
            calls, _ = argmax_calls(xs, axis)
            ops.append(Op("B1", "argmax{%d}%s" % (axis, text), count, 4 * count, calls, timed_only(calls[0])))
        # statistics per channel: rows made of contiguous runs
        xs = gen((32, 512, 56, 56), torch.float32, lambda c: synth.normal(51 + 100 * c), enough((32, 512, 56, 56), torch.float32))
        calls, _ = reduce_calls("reduce_sum", xs, [0, 2, 3])
        ops.append(Op("B2", "reduce_sum{0,2,3}_f32_[32,512,56,56]", 32 * 512 * 3136, 4 * 32 * 512 * 3136, calls, timed_only(calls[0])))
        # many short rows that are not whole cache lines; rows of a few long runs; rows of 1024 to 8192 elements made of runs
        for shape, axes in (((2867200, 56), [1]), ((4194304, 16), [1]), ((8, 16, 32, 64, 64), [0, 2, 3, 4]), ((16, 64, 128, 128), [1, 3]), ((32, 512, 56, 56), [3])):
            xs = gen(shape, torch.float32, lambda c: synth.normal(56 + 100 * c), enough(shape, torch.float32))
            calls, _ = reduce_calls("reduce_sum", xs, axes)
            ops.append(Op("B2", "reduce_sum{%s}_f32_[%s]" % (",".join(str(a) for a in axes), ",".join(str(e) for e in shape)), int(np.prod(shape)), 4 * int(np.prod(shape)), calls, timed_only(calls[0])))
        # long rows near the end of the bucket route (bins packed bucket by bucket), doubles with the gap closed
        for shape, dtype, text in (((16, 2300000), torch.float32, "f32_normal_[16,2300000]"), ((16, 2400000), torch.float32, "f32_normal_[16,2400000]"),
                                   ((3355, 10000), torch.float64, "f64_normal_[3355,10000]")):
            xs = gen(shape, dtype, lambda c: synth.normal(52 + 100 * c), enough(shape, dtype))
            ops += [op for op in sort_ops(be, tensor, xs, "B3", text) if "_asc_" in op.name]
        # half elements along an axis that is not the innermost: two neighbouring columns a lane
        for shape, axis in (((32, 512, 56, 56), 1), ((64, 1 << 20), 0), ((8, 21, 512, 512), 1)):
            xs = gen(shape, torch.float16, lambda c: synth.normal(54 + 100 * c), enough(shape, torch.float16))
            text = "_f16_[%s]" % ",".join(str(e) for e in shape)
            count = int(np.prod(shape))
            calls, _ = scan_calls(xs, axis)
            ops.append(Op("B5", "cumsum{%d}%s" % (axis, text), count, 4 * count, calls, timed_only(calls[0])))
            calls, _ = reduce_calls("reduce_sum", xs, [axis])
            ops.append(Op("B5", "reduce_sum{%d}%s" % (axis, text), count, 2 * count, calls, timed_only(calls[0])))
            calls, _ = argmax_calls(xs, axis)
            ops.append(Op("B5", "argmax{%d}%s" % (axis, text), count, 2 * count, calls, timed_only(calls[0])))
        # top_k along an axis that is not the innermost (register lists, a lane per column)
        for shape, axis in (((32, 512, 56, 56), 1), ((16, 80, 160, 160), 1)):
            xs = gen(shape, torch.float32, lambda c: synth.normal(55 + 100 * c), enough(shape, torch.float32))
            count = int(np.prod(shape))
            for k in (1, 5):
                out_dims = [k if i == axis else e for i, e in enumerate(shape)]
                Yk = Tensor.empty(be, out_dims, np.float32)
                Ik = Tensor.empty(be, out_dims, np.int32)
                calls = []
                for x in xs:
                    X = tensor(x)
                    calls.append(be.top_k(k, 1, dtype_code(np.float32), 2, X.shape.moveaxis(axis, -1), X.storage, Yk.shape.moveaxis(axis, -1), Yk.storage,
                                          Ik.shape.moveaxis(axis, -1), Ik.storage, defer=True))
                ops.append(Op("B6", "top_k%d{%d}_f32_[%s]" % (k, axis, ",".join(str(e) for e in shape)), count, 4 * count, calls, timed_only(calls[0])))
        # top_k of very long rows
        for rows_l, n_l in ((1, 1 << 24), (1, 1 << 23)):
            xl_ = gen((rows_l, n_l), torch.float32, lambda c: synth.normal(53 + 100 * c), enough((rows_l, n_l), torch.float32))
            ops += topk_ops(be, tensor, xl_, (256, 257), "B4", "[%d,2^%d]" % (rows_l, n_l.bit_length() - 1))

    # ---------------- C5: strided NCHW
    if on("all", "c5"):
        x5 = gen((32, 512, 56, 56), torch.float32, lambda c: synth.normal(8 + 100 * c), 6)
        n5 = 32 * 512 * 56 * 56
        calls, outs = reduce_calls("reduce_mean", x5, [2, 3])

        def v_mean(x=x5[0], out=outs[0], call=calls[0]):
            call()
            assert torch.allclose(out.storage[:16384].double(), x.double().mean((2, 3)).view(-1), rtol=1e-5, atol=1e-6)
        ops.append(Op("C5", "reduce_mean{2,3}_f32_[32,512,56,56]", n5, 4 * n5 + 65536, calls, v_mean, "reduce_rows_group<ValueReducer<float, 0, 0>"))
        calls, outs = reduce_calls("reduce_max", x5, [1])

        def v_max(x=x5[0], out=outs[0], call=calls[0]):
            call()
            assert torch.equal(out.storage[:100352], x.amax(1).reshape(-1))
        ops.append(Op("C5", "reduce_max{1}_f32_[32,512,56,56]", n5, 4 * n5 + 401408, calls, v_max, "reduce_cols<ValueReducer<float, 2, 0>"))
        calls, outs = argmax_calls(x5, 1)

        def v_arg(x=x5[0], out=outs[0], call=calls[0]):
            call()
            assert torch.equal(out.storage[:100352].long(), torch.argmax(x, 1).reshape(-1))
        ops.append(Op("C5", "argmax{1}_f32_[32,512,56,56]", n5, 4 * n5 + 401408, calls, v_arg, "reduce_cols<ArgReducer<float, true, int>"))
        calls, y5 = scan_calls(x5, 1)

        def v_cs(x=x5[0], y=y5, call=calls[0]):
            call()
            want = torch.cumsum(x.double(), 1)
            mag = torch.cumsum(x.double().abs(), 1)
            err = (y.double() - want).abs()
            tol = 4 * 9 * float(np.finfo(np.float32).eps) * torch.maximum(want.abs(), mag)
            assert bool((err <= tol).all())
            STRICT_FAILURES["C5 cumsum{1}_f32_[32,512,56,56]"] = int((err > 4 * 9 * float(np.finfo(np.float32).eps) * want.abs()).sum())
        ops.append(Op("C5", "cumsum{1}_f32_[32,512,56,56]", n5, 8 * n5, calls, v_cs, "scan_cols<float"))

    # ---------------- N1: count and nonzero (the callers next to reduce and scan)
    if on("all", "n1"):
        rows_n, cols_n = 4096, 16384
        xn = gen((rows_n, cols_n), torch.float32, lambda c: (lambda idx, f=synth.randint(9 + 100 * c, 0, 4): f(idx) // 3), 4)   # a quarter ones, the rest zeros
        nn = rows_n * cols_n
        zero = np.zeros(1, dtype=np.float32)
        calls, outs = [], []
        for x in xn:
            X = tensor(x)
            view, out_dims, m, n = prepare_reduce(X.shape, [1], False)
            Y = Tensor.empty(be, out_dims, np.int32)
            calls.append(be.count(dtype_code(X.dtype), m, n, 0.0, view, X.storage, Y.shape, Y.storage, defer=True))
            outs.append(Y)

        def v_count(x=xn[0], out=outs[0], call=calls[0]):
            call()
            assert torch.equal(out.storage[:rows_n].long(), (x == 0).sum(1))
        ops.append(Op("N1", "count0{1}_f32_[4096,16384]", nn, 4 * nn + 4 * rows_n, calls, v_count))

        counts = Tensor.empty(be, [nn], np.int32)
        flat = Shape([nn])
        calls = [be.scan_nonzero(dtype_code(np.float32), 1, nn, False, tensor(x).shape, tensor(x).storage,
                                 Shape([rows_n, cols_n]), counts.storage, defer=True) for x in xn]

        def v_scan_nz(x=xn[0], call=calls[0]):
            call()
            assert torch.equal(counts.storage[:nn].long(), torch.cumsum((x.view(-1) != 0).long(), 0))
        ops.append(Op("N1", "scan_nonzero_f32_[2^26]", nn, 8 * nn, calls, v_scan_nz))

        # gather_indices reads counts that must match its n: it gets its own copy of the
        # first input's counts, which the timed scan_nonzero calls (other inputs) never touch
        counts0 = Tensor.empty(be, [nn], np.int32)
        be.scan_nonzero(dtype_code(np.float32), 1, nn, False, tensor(xn[0]).shape, tensor(xn[0]).storage,
                        Shape([rows_n, cols_n]), counts0.storage)
        torch.cuda.synchronize()
        total = int(counts0.storage[nn - 1].item())
        coords = Tensor.empty(be, [total, 2], np.int32)
        gcall = be.gather_indices(nn, total, False, [rows_n, cols_n], counts0.storage, coords.storage, defer=True)

        def v_gather(x=xn[0]):
            gcall()
            assert torch.equal(coords.storage[:2 * total].view(total, 2).long(), torch.nonzero(x))
        ops.append(Op("N1", "gather_indices_[2^26]->[%d,2]" % total, nn, 4 * nn + 8 * total, [gcall], v_gather))

    # ---------------- N3: softmax family on the top_k shape and the logits head
    if on("all", "n3"):
        for rows_s, cols_s, copies in ((4096, 32000, 3), (256, 1000, 4)):
            xs_ = gen((rows_s, cols_s), torch.float32, lambda c: synth.normal(12 + 100 * c), copies)
            ys_ = empty((rows_s, cols_s), torch.float32)
            for nm in ("softmax", "logsoftmax", "hardmax"):
                calls = [be.softmax(nm, dtype_code(np.float32), rows_s, cols_s, x.view(-1), 0, ys_.view(-1), 0, defer=True)
                         for x in xs_]

                def v_soft(x=xs_[0], call=calls[0], nm=nm, ys_=ys_, rows_s=rows_s):
                    call()
                    if nm == "softmax":
                        assert torch.allclose(ys_.double(), torch.softmax(x.double(), 1), rtol=1e-5, atol=1e-12)
                    elif nm == "logsoftmax":
                        assert torch.allclose(ys_.double(), torch.log_softmax(x.double(), 1), rtol=1e-5, atol=1e-5)
                    else:
                        assert torch.equal(ys_.argmax(1), x.argmax(1)) and float(ys_.sum()) == rows_s
                ops.append(Op("N3", "%s_f32_[%d,%d]" % (nm, rows_s, cols_s), rows_s * cols_s, 8 * rows_s * cols_s, calls, v_soft))

    # ---------------- N2: merge of sorted rows
    if on("all", "n2"):
        half = 1 << 19
        am = [torch.sort(t, dim=1).values for t in gen((64, half), torch.float32, lambda c: synth.normal(10 + 100 * c), 2)]
        bm = [torch.sort(t, dim=1).values for t in gen((64, half), torch.float32, lambda c: synth.normal(11 + 100 * c), 2)]
        zm = empty((64, 2 * half), torch.float32)
        Z = tensor(zm)
        calls = [be.merge(0, dtype_code(np.float32), tensor(a).shape, tensor(a).storage, tensor(b).shape, tensor(b).storage,
                          Z.shape, Z.storage, defer=True) for a, b in zip(am, bm)]

        def v_merge(a=am[0], b=bm[0], call=calls[0]):
            call()
            assert torch.equal(zm, torch.sort(torch.cat([a, b], dim=1), dim=1).values)
        ops.append(Op("N2", "merge_f32_[64,2^19]+[64,2^19]", 64 * 2 * half, 2 * 4 * 64 * 2 * half, calls, v_merge))
    # ---------------- L1 (only on request): a few very long rows (a sampling head over a huge vocabulary)
    if on("long"):
        for rows_l, n_l in ((1, 1 << 26), (64, 1 << 20)):
            text = "[%d,2^%d]" % (rows_l, n_l.bit_length() - 1)
            xl_ = gen((rows_l, n_l), torch.float32, lambda c: synth.normal(30 + 100 * c), 2)
            yl_ = empty((rows_l, n_l), torch.float32)
            calls = [be.softmax("softmax", dtype_code(np.float32), rows_l, n_l, x.view(-1), 0, yl_.view(-1), 0, defer=True) for x in xl_]

            def v_sl(x=xl_[0], y=yl_, call=calls[0]):
                call()
                assert torch.allclose(y.double(), torch.softmax(x.double(), 1), rtol=1e-5, atol=1e-14)
            ops.append(Op("L1", "softmax_f32_" + text, rows_l * n_l, 8 * rows_l * n_l, calls, v_sl))
            ops += topk_ops(be, tensor, xl_, (5, 100), "L1", text)
    # ---------------- S1 (only on request): many short rows, and top_k along an outer axis
    if on("short"):
        for rows_s, n_s in ((1 << 20, 64), (1 << 18, 256), (1 << 16, 1024)):
            text = "[%d,%d]" % (rows_s, n_s)
            xs_ = gen((rows_s, n_s), torch.float32, lambda c: synth.normal(20 + 100 * c), 2)
            ops += [op for op in sort_ops(be, tensor, xs_, "S1", "f32_" + text) if "_asc_" in op.name]
            ops += topk_ops(be, tensor, xs_, (5,), "S1", text)
            calls, ycs = scan_calls(xs_, 1)

            def v_cs(x=xs_[0], y=ycs, call=calls[0]):
                call()
                want = torch.cumsum(x.double(), 1)
                tol = 4 * 10 * float(np.finfo(np.float32).eps) * torch.cumsum(x.double().abs(), 1)
                assert bool(((y.double() - want).abs() <= tol).all()), "short-row cumsum out of tolerance"
            ops.append(Op("S1", "cumsum_f32_" + text, rows_s * n_s, 8 * rows_s * n_s, calls, v_cs))
            ysm = empty((rows_s, n_s), torch.float32)
            calls = [be.softmax("softmax", dtype_code(np.float32), rows_s, n_s, x.view(-1), 0, ysm.view(-1), 0, defer=True)
                     for x in xs_]

            def v_sm(x=xs_[0], y=ysm, call=calls[0]):
                call()
                assert torch.allclose(y.double(), torch.softmax(x.double(), 1), rtol=1e-5, atol=1e-12)
            ops.append(Op("S1", "softmax_f32_" + text, rows_s * n_s, 8 * rows_s * n_s, calls, v_sm))
            ha = [torch.sort(x[:, :n_s // 2], dim=1).values.contiguous() for x in xs_]
            hb = [torch.sort(x[:, n_s // 2:], dim=1).values.contiguous() for x in xs_]
            zs = empty((rows_s, n_s), torch.float32)
            Z = tensor(zs)
            calls = [be.merge(0, dtype_code(np.float32), tensor(a).shape, tensor(a).storage, tensor(b).shape, tensor(b).storage,
                              Z.shape, Z.storage, defer=True) for a, b in zip(ha, hb)]

            def v_mg(x=xs_[0], z=zs, call=calls[0]):
                call()
                assert torch.equal(z, torch.sort(x, dim=1).values)
            ops.append(Op("S1", "merge_f32_%s/2+%s/2" % (text, text), rows_s * n_s, 8 * rows_s * n_s, calls, v_mg))
        xo = gen((64, 1 << 20), torch.float32, lambda c: synth.normal(21 + 100 * c), 2)
        for k in (1, 5):
            Y = Tensor.empty(be, [k, 1 << 20], np.float32)
            I = Tensor.empty(be, [k, 1 << 20], np.int32)
            calls = [be.top_k(k, 1, dtype_code(np.float32), 2, tensor(x).shape.moveaxis(0, -1), tensor(x).storage,
                              Y.shape.moveaxis(0, -1), Y.storage, I.shape.moveaxis(0, -1), I.storage, defer=True) for x in xo]

            def v_tc(x=xo[0], Y=Y, I=I, k=k, call=calls[0]):
                call()
                w = torch.sort(x, dim=0, descending=True, stable=True)
                assert torch.equal(Y.storage[:k << 20].view(k, 1 << 20), w.values[:k]), "outer-axis top_k values"
                assert torch.equal(I.storage[:k << 20].view(k, 1 << 20).long(), w.indices[:k]), "outer-axis top_k indices"
            ops.append(Op("S1", "top_k%d_axis0_f32_[64,2^20]" % k, 64 << 20, 4 * (64 << 20) + 8 * (k << 20), calls, v_tc))
    return ops


def topk_ops(be, tensor, xs, ks, config, shape_text):
    import numpy as np
    import torch
    from dlf_amd.frontend import Tensor, dtype_code
    ops = []
    rows, n = xs[0].shape
    for k in ks:
        Y = Tensor.empty(be, [rows, k], np.float32)
        I = Tensor.empty(be, [rows, k], np.int64)
        calls = []
        for x in xs:
            X = tensor(x)
            calls.append(be.top_k(k, 1, dtype_code(np.float32), 3, X.shape, X.storage, Y.shape, Y.storage,
                                  I.shape, I.storage, defer=True))

        def v(x=xs[0], Y=Y, I=I, k=k, call=calls[0], rows=rows):
            call()
            y = Y.storage[:rows * k].view(rows, k)
            i = I.storage[:rows * k].view(rows, k)
            want = torch.topk(x, k, dim=1, largest=True, sorted=True).values
            assert torch.equal(y, want), "top_k values"
            assert torch.equal(torch.gather(x, 1, i), y), "top_k gather"
            # lowest index on ties: compare against a stable descending sort on a slice of rows
            sub = x[:64]
            order = torch.sort(sub, dim=1, descending=True, stable=True).indices[:, :k]
            assert torch.equal(i[:64], order), "top_k tie order"
        ops.append(Op(config, "top_k%d_f32_%s" % (k, shape_text), rows * n, 4 * rows * n + rows * k * 12, calls, v,
                      "topk_select"))
    return ops


def split_kernels(es, pairs, rows, n):
    """The kernels that move the data of one sort / argsort of rows the bucket route takes."""
    key = "unsigned int" if es == 4 else "unsigned long"
    waves = 4 if n <= 131072 else 8
    flag = "true" if pairs else "false"
    finish = "split_finish<%s, %s, %d>" % (key, flag, waves)
    if es == 4 and waves == 4 and rows >= 512:            # one workgroup plans and moves a whole row
        return ["split_front<%s, %s," % (key, flag), finish]
    return ["split_sample<%s," % key, "split_histogram<%s," % key, "split_plan", "split_pass<%s, %s," % (key, flag), finish]


def sort_ops(be, tensor, xs, config, text):
    import numpy as np
    import torch
    from dlf_amd.frontend import Tensor, dtype_code
    ops = []
    rows, n = xs[0].shape
    es = xs[0].element_size()
    npd = {torch.float32: np.float32, torch.float64: np.float64, torch.int64: np.int64}[xs[0].dtype]
    y = torch.empty_like(xs[0])
    Y = tensor(y)
    I = Tensor.empty(be, [rows, n], np.int32)
    for desc in (0, 1):
        calls = []
        for x in xs:
            X = tensor(x)
            calls.append(be.sort(desc, dtype_code(npd), X.shape, X.storage, Y.shape, Y.storage, defer=True))

        def v(x=xs[0], y=y, desc=desc, call=calls[0]):
            call()
            assert torch.equal(y, torch.sort(x, dim=1, descending=bool(desc)).values), "sort"
        ops.append(Op(config, "sort_%s_%s" % ("desc" if desc else "asc", text), rows * n, 2 * es * rows * n, calls, v,
                      split_kernels(es, False, rows, n)))
        calls = []
        for x in xs:
            X = tensor(x)
            calls.append(be.argsort(desc, dtype_code(npd), 2, X.shape, X.storage, None, None, I.shape, I.storage, defer=True))

        def va(x=xs[0], I=I, desc=desc, call=calls[0], rows=rows, n=n):
            call()
            i = I.storage[:rows * n].view(rows, n).long()
            sub = slice(0, 16)
            want = torch.sort(x[sub], dim=1, descending=bool(desc), stable=True).indices
            assert torch.equal(i[sub], want), "argsort stable order"
            g = torch.gather(x, 1, i)
            d = g[:, 1:] - g[:, :-1] if x.dtype != torch.int64 else None
            if d is not None:
                assert bool((d <= 0).all() if desc else (d >= 0).all()), "argsort sortedness"
            else:
                assert bool((g[:, 1:] <= g[:, :-1]).all() if desc else (g[:, 1:] >= g[:, :-1]).all())
        ops.append(Op(config, "argsort_%s_%s" % ("desc" if desc else "asc", text), rows * n, (es + 4) * rows * n,
                      calls, va, split_kernels(es, True, rows, n)))
    return ops


def time_op(torch, op, iters, warm=3, same_input=False):
    """Median and mean time of one call.  same_input: every call reads the first input buffer
    (what the 256 MB Infinity Cache keeps of it is then reused) instead of rotating over all of them."""
    issue = op.calls[0] if same_input else op.issue
    for _ in range(warm):
        issue()
    torch.cuda.synchronize()
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
    evs[0].record()
    for i in range(iters):
        issue()
        evs[i + 1].record()
    torch.cuda.synchronize()
    ts = sorted(evs[i].elapsed_time(evs[i + 1]) * 1e3 for i in range(iters))   # us
    return ts[len(ts) // 2], sum(ts) / len(ts)


def cpu_baseline():
    """The CPU restatement of the reference's algorithms, timed on this box's host cores."""
    import numpy as np
    from dlf_amd import frontend as F
    from dlf_amd.frontend import Tensor
    from oracle import oracle as O
    be = O.OracleBackend()
    rng = np.random.default_rng(2)
    xi = rng.integers(0, 100, size=(64, 1 << 20), dtype=np.int32)
    xf = rng.standard_normal((64, 1 << 20), dtype=np.float32)
    xl = (rng.integers(0, 1 << 24, size=1 << 28).astype(np.float32) * np.float32(2.0 ** -23)) - np.float32(1.0)
    Xi, Xf, Xl = (Tensor.from_numpy(be, a) for a in (xi, xf, xl))
    Yi, Yf = Tensor.empty(be, xi.shape, np.int32), Tensor.empty(be, xf.shape, np.float32)
    F.cumsum(Xi, 1, out=Yi)                       # warm the pages
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        F.cumsum(Xi, 1, out=Yi)
        F.cumsum(Xf, 1, out=Yf)
        F.reduce_sum(Xl, [])
    dt = (time.perf_counter() - t0) / reps
    nbytes = 2 * 4 * (64 << 20) * 2 + 4 * (1 << 28)
    return {"value": round(nbytes / dt / 1e9, 2), "unit": "GB/s", "cores": O.threads(), "kind": "port",
            "sample": "cumsum int32 + fp32 [64,2^20] in full and reduce_sum over 2^28 of the 2^30 fp32 elements, "
                      "3 repetitions, OpenMP rows/chunks in parallel"}


def cpu_per_config():
    """The CPU restatement timed on a bounded sample of every other configuration: the same shapes
    with fewer rows where a full run would take minutes (a few seconds in all)."""
    import numpy as np
    from dlf_amd import frontend as F
    from dlf_amd.frontend import Tensor
    from oracle import oracle as O
    be = O.OracleBackend()
    rng = np.random.default_rng(3)
    out = []

    def timed(label, sample, nbytes, fn, reps=3):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        dt = (time.perf_counter() - t0) / reps
        out.append({"op": label, "sample": sample, "us": round(dt * 1e6, 1), "gb_s": round(nbytes / dt / 1e9, 2)})

    x1 = Tensor.from_numpy(be, rng.standard_normal((256, 1000), dtype=np.float32))
    timed("C1 reduce_sum+max+lse+argmax+top_k5 [256,1000]", "full", 5 * 1024000,
          lambda: (F.reduce_sum(x1, [1]), F.reduce_max(x1, [1]), F.reduce_log_sum_exp(x1, [1]), F.argmax(x1, 1),
                   F.top_k(x1, 5, 1)), reps=20)
    x3 = Tensor.from_numpy(be, (np.round(rng.standard_normal((512, 32000)) * 512) / 256).astype(np.float32))
    for k in (1, 5, 50, 256):
        timed("C3 top_k%d [4096,32000]" % k, "512 of 4096 rows", 4 * 512 * 32000, lambda k=k: F.top_k(x3, k, 1))
    x4 = Tensor.from_numpy(be, (np.floor(rng.random((128, 65536)) * 4096) / 4096).astype(np.float32))
    timed("C4a sort f32 [1024,65536]", "128 of 1024 rows", 8 * 128 * 65536, lambda: F.sort(x4, 1))
    timed("C4a argsort f32 [1024,65536]", "128 of 1024 rows", 8 * 128 * 65536, lambda: F.argsort(x4, 1))
    x4b = Tensor.from_numpy(be, rng.integers(-2 ** 63, 2 ** 63 - 1, size=(16, 1 << 20), dtype=np.int64))
    timed("C4b sort i64 [256,2^20]", "16 of 256 rows", 16 * 16 * (1 << 20), lambda: F.sort(x4b, 1), reps=2)
    timed("C4b argsort i64 [256,2^20]", "16 of 256 rows", 12 * 16 * (1 << 20), lambda: F.argsort(x4b, 1), reps=2)
    x5 = Tensor.from_numpy(be, rng.standard_normal((8, 512, 56, 56), dtype=np.float32))
    n5 = 8 * 512 * 56 * 56
    timed("C5 reduce_mean{2,3} [32,512,56,56]", "8 of 32 images", 4 * n5, lambda: F.reduce_mean(x5, [2, 3]))
    timed("C5 reduce_max{1}", "8 of 32 images", 4 * n5, lambda: F.reduce_max(x5, [1]))
    timed("C5 argmax{1}", "8 of 32 images", 4 * n5, lambda: F.argmax(x5, 1))
    timed("C5 cumsum{1}", "8 of 32 images", 8 * n5, lambda: F.cumsum(x5, 1))
    return {"cores": O.threads(), "kind": "port", "ops": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--configs", default="all", help="all | step | comma-separated subset of c1,c2,c3,c4,c5,n1,n2,n3 | short (many short rows and an outer axis; not part of all) | spread (sorts of N(0,1) rows; not part of all) | ceil (copy and read-only streams at the C2 and C5 sizes; part of all) | ceilbig (the same streams at 1 GiB and 4 GiB; not part of all) | long (softmax and top_k over a few very long rows; not part of all) | repeats (sorts of rows of one value, of ten values and of clustered keys; not part of all) | beside (shapes beside the baseline's at which sweeps found steps: outer-axis scans and reductions, statistics per channel, rows near the end of the bucket route, half elements along an outer axis, top_k along an outer axis and of very long rows; not part of all)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (read 1 GiB, write 1 GiB) so that byte counters "
                         "collected by a profiler can be scaled against a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    import torch
    from dlf_amd.hip_backend import HipBackend
    be = HipBackend("cuda:0")
    ops = make_ops(be, args.configs)
    log("inputs resident: %d operations" % len(ops))

    if not args.no_verify:
        for op in ops:
            if op.verify:
                op.verify()
        torch.cuda.synchronize()
        log("parity gates passed")

    traffic_table = profiled_traffic()

    # ---- the step: C2a + C2b + C2c back to back
    step_ops = [op for op in ops if op.config in ("C2a", "C2b", "C2c")]
    result = {"metric": METRIC, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int32+f32 (fp32 sums accumulate in f64)",
              "data": "synthetic"}
    if step_ops:
        for _ in range(args.warmup):
            for op in step_ops:
                op.issue()
        torch.cuda.synchronize()
        per_kernel = {op.name: [] for op in step_ops}
        evs = []
        t0 = time.perf_counter()
        for _ in range(args.steps):
            row = [torch.cuda.Event(enable_timing=True)]
            row[0].record()
            for op in step_ops:
                op.issue()
                e = torch.cuda.Event(enable_timing=True)
                e.record()
                row.append(e)
            evs.append(row)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        for row in evs:
            for j, op in enumerate(step_ops):
                per_kernel[op.name].append(row[j].elapsed_time(row[j + 1]) * 1e3)
        step_bytes = sum(op.alg_bytes for op in step_ops)
        ms = wall / args.steps * 1e3
        result.update({"value": round(step_bytes / (wall / args.steps) / 1e9, 1), "ms_per_step": round(ms, 4),
                       "config": {"workload": "configs[1]: cumsum int32 [64,2^20] + cumsum fp32 [64,2^20] + "
                                              "reduce_sum fp32 [2^30], last axis, contiguous",
                                  "algorithmic_bytes_per_step": step_bytes}})
        dom = max(step_ops, key=lambda op: sum(per_kernel[op.name]))
        avg_us = sum(per_kernel[dom.name]) / len(per_kernel[dom.name])
        achieved = dom.alg_bytes / avg_us / 1e3
        result["roofline"] = {"bound": "hbm", "kernel": dom.kernel, "op": dom.name, "achieved": round(achieved, 1),
                              "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                              "avg_launch_us": round(avg_us, 2),
                              "traffic": traffic_of(dom.kernel, traffic_table, dom.config)}
    else:
        result.update({"value": None, "ms_per_step": None, "config": {"workload": args.configs}})

    # ---- every operation on its own
    per_op = []
    for op in ops:
        iters = 20 if op.alg_bytes < (1 << 31) else 8
        med, avg = time_op(torch, op, iters)
        gbs = op.alg_bytes / med / 1e3
        entry = {"config": op.config, "op": op.name, "us": round(med, 2), "gelem_s": round(op.elems / med / 1e3, 2),
                 "gb_s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
        if len(op.calls) > 1:
            # the same call over one input buffer, reported apart: not an HBM figure
            entry["us_same_input"] = round(time_op(torch, op, iters, same_input=True)[0], 2)
        per_op.append(entry)
        log("%-4s %-44s %10.1f us %9.1f GB/s %6.1f%%" % (op.config, op.name, med, gbs, 100 * gbs / HBM_PEAK_GBS))
    # the C2 / C5 operations beside the plain stream of the same bytes measured in this run: a
    # dense copy (one 128-bit load and store per thread) for the scans, the read-only stream for
    # the reductions
    stream_us = {e["op"]: e["us"] for e in per_op if e["config"] == "ceil"}
    for e in per_op:
        if e["config"] in ("C2a", "C2b"):
            ref = stream_us.get("copy_f32_[64,2^20]")
        elif e["config"] == "C2c":
            ref = stream_us.get("read_f32_[2^30]")
        elif e["config"] == "C5":
            ref = stream_us.get(("copy" if e["op"].startswith("cumsum") else "read") + "_f32_[32,512,56,56]")
        else:
            ref = None
        if ref:
            e["stream_us"] = ref
            e["frac_of_stream"] = round(ref / e["us"], 4)
    result["per_op"] = per_op
    if STRICT_FAILURES:
        result["strict_relative_failures"] = dict(STRICT_FAILURES)

    # ---- each family's worst case over the bandwidth-bound configurations (C2 - C5; C1 moves
    # 1 MB and is bound by launch latency: it is reported by c1_graph below)
    by_family = {}
    for op, entry in zip(ops, per_op):
        fam = family_of(op.name)
        if fam is None or op.config not in ("C2a", "C2b", "C2c", "C3", "C4a", "C4b", "C5"):
            continue
        if fam not in by_family or entry["frac_hbm"] < by_family[fam]["frac"]:
            traffic = traffic_of(op.kernel, traffic_table, op.config)
            by_family[fam] = {"config": op.config, "op": op.name, "kernels": op.kernel, "us": entry["us"],
                              "achieved": entry["gb_s"], "unit": "GB/s", "peak": HBM_PEAK_GBS, "frac": entry["frac_hbm"],
                              "algorithmic_bytes": op.alg_bytes, "traffic": traffic,
                              "traffic_ratio": None if traffic is None else round(traffic / op.alg_bytes, 3)}
    if by_family:
        result["roofline_by_family"] = by_family
        for fam, e in by_family.items():
            log("worst %-7s %-4s %-40s %6.1f%% of peak, HBM traffic x%s" % (fam, e["config"], e["op"], 100 * e["frac"], e["traffic_ratio"]))

    # ---- the launch-bound configuration recorded once and replayed as a HIP graph
    c1 = [op for op in ops if op.config == "C1"]
    if c1:
        for op in c1:
            op.calls[0]()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for op in c1:
                op.calls[0]()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        reps = 50
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        result["c1_graph"] = {"ops": len(c1), "us_per_replay": round(us, 2), "us_per_op": round(us / len(c1), 2)}
        log("C1   %d ops replayed as one HIP graph: %.1f us per replay, %.1f us per op" % (len(c1), us, us / len(c1)))
        # the floor of this way of measuring: a one-element fill (a kernel that does nothing to
        # speak of), issued and timed exactly like the operations above
        one = torch.zeros(1, dtype=torch.float32, device=be.device)
        floor = Op("C1", "floor", 1, 4, [be.fill(0, [1], [1], one, 0, 1.0, defer=True)])
        result["c1_floor_us"] = round(time_op(torch, floor, 50)[0], 2)
        log("C1   launch floor (one-element fill, timed the same way): %.1f us" % result["c1_floor_us"])
        fused = [e for e in per_op if e["config"] == "C1f"]
        if fused:
            separate = sum(e["us"] for e in per_op if e["config"] == "C1")
            result["c1_fused"] = {"us": fused[0]["us"], "us_five_separate_calls": round(separate, 2)}

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=be.device).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
        if step_ops and len({op.config for op in ops} & {"C1", "C3", "C4a", "C4b", "C5"}) == 5:
            result["cpu_per_config"] = cpu_per_config()      # bounded samples: a few seconds in all
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
