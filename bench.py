#!/usr/bin/env python3
"""Benchmark of the helium MI355X backend's hot path on ONE GPU.

A "step" is one pass of the headline workload over one batch of synthetic, seeded input that is already
resident in HBM when the timed region starts. Prints ONE JSON line.
The other BASELINE workloads are measured in the same run and reported under "kernels".

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "fused-GEMM TFLOP/s & permute/pointwise GB/s, % of MI355X roofline"
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published
F32_PEAK_TFLOPS = 157.3      # MI355X dense fp32 matrix, published


def _traffic_table():
    """Bytes that leave the XCD L2s per step of each workload (all launches of the step), from the committed counter summary
    (profiles/traffic_per_launch.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by the COPY workload); a workload
    the file does not list reports null."""
    table = {}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "traffic_per_launch.txt")
    try:
        for line in open(path):
            parts = line.split()
            if len(parts) == 3 and not line.startswith("#"):
                table[parts[0]] = int(parts[2])
    except OSError:
        pass
    return table


TRAFFIC_BYTES = _traffic_table()
HEADLINE = "C4"              # the workload `value` is quoted on
ROTATE_BYTES = 768 << 20     # rotate operand sets so repeated steps cannot live in the 256 MB Infinity Cache


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def bf16_rne(x):
    """float32 -> bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


class PermuteWorkload:
    """BASELINE config 2: bf16 N(0,1) tensors, bit-exact permutes. Algorithmic bytes = 2 * numel * 2."""

    bound = "hbm"
    unit = "GB/s"
    dtype = "bf16"

    def __init__(self, name, shape, perm, seed):
        self.name, self.shape, self.perm, self.seed = name, shape, perm, seed
        self.numel = int(np.prod(shape))
        self.work = 2 * self.numel * 2  # bytes read + bytes written

    def describe(self):
        return f"{self.name}: bf16 {list(self.shape)} permute {self.perm}"


    def setup(self):
        import helium_amd as ha

        rng = np.random.default_rng(self.seed)
        self.host = bf16_rne(rng.standard_normal(size=self.shape, dtype=np.float32))
        self.op = ha.PermuteDims(self.shape, "bf16", perm=self.perm)
        nsets = max(2, min(16, ROTATE_BYTES // self.work + 1))
        self.sets = []
        for _ in range(nsets):
            src = ha.DeviceBuffer.from_numpy(self.host)
            dst = ha.DeviceBuffer(self.host.nbytes)
            self.sets.append((src, dst))
        log(f"[bench] {self.describe()} :: {self.op.description} :: {nsets} operand sets")

    def step(self, stream, i):
        src, dst = self.sets[i % len(self.sets)]
        self.op.execute(src, dst, stream)

    def check(self):
        from oracle import permute as oracle

        src, dst = self.sets[0]
        got = dst.to_numpy(np.uint16, self.op.out_shape)
        want = oracle.permute(self.host, self.perm)
        if not np.array_equal(got, want):
            raise SystemExit(f"[bench] PARITY FAILURE in {self.name}: output differs from the oracle")
        return "bit-exact vs numpy oracle"

    def cpu_baseline(self, budget_s=10.0):
        from oracle import permute as oracle

        oracle.permute(self.host, self.perm)
        best, reps, t_all = 1e30, 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t_all < budget_s and reps < 20):
            t0 = time.perf_counter()
            oracle.permute(self.host, self.perm)
            best = min(best, time.perf_counter() - t0)
            reps += 1
        return {"value": round(self.work / best / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"full {self.name} tensor, numpy transpose+copy (oracle), best of {reps} passes"}

    def free(self):
        for s, d in self.sets:
            s.free()
            d.free()
        self.sets = []


class ReferencePermuteWorkload:
    """The reference's own permute benchmark (helium/examples/permute_dim_benchmark.rs:13-41): f32 [2048,128,128,32],
    swap_dims(0, 3), 4.3 GB in and 4.3 GB out, so every byte comes from HBM. Input element i holds the value i, which
    makes every output element's expected value a closed form of its index."""

    bound = "hbm"
    unit = "GB/s"
    dtype = "f32"
    name = "PERM-ref"

    def __init__(self):
        from helium_amd import configs

        self.shape, self.perm = configs.PERM_REF_SHAPE, configs.PERM_REF_PERM
        self.numel = int(np.prod(self.shape))
        self.work = 2 * self.numel * 4

    def describe(self):
        return f"PERM-ref: f32 {list(self.shape)} swap_dims(0, 3) (the reference's permute_dim_benchmark)"

    def setup(self):
        import helium_amd as ha

        self.op = ha.PermuteDims(self.shape, "f32", perm=self.perm)
        self.inverse = ha.PermuteDims(self.op.out_shape, "f32", perm=self.perm)  # swap_dims(0, 3) undoes itself
        host = np.arange(self.numel, dtype=np.uint32)
        self.sets = [(ha.DeviceBuffer.from_numpy(host), ha.DeviceBuffer(host.nbytes)) for _ in range(2)]
        del host
        log(f"[bench] {self.describe()} :: {self.op.description} :: 2 operand sets")

    def step(self, stream, i):
        src, dst = self.sets[i % 2]
        self.op.execute(src, dst, stream)

    def check(self):
        from helium_amd import configs

        src, dst = self.sets[0]
        rng = np.random.default_rng(5)
        row = self.shape[0]  # the output's innermost extent
        for start in rng.integers(0, self.numel // row, size=256):
            got = dst.read(int(start) * row * 4, np.uint32, row)
            want = configs.perm_ref_expected(np.arange(int(start) * row, (int(start) + 1) * row, dtype=np.uint64))
            if not np.array_equal(got, want):
                raise SystemExit("[bench] PARITY FAILURE in PERM-ref: a sampled output row differs from the closed form")
        # and back: the same permute applied to the output restores the input bit for bit (sampled rows of 1 MiB)
        back = self.sets[1][1]
        self.inverse.execute(dst, back)
        for start in rng.integers(0, self.numel // (1 << 18), size=64):
            got = back.read(int(start) * (1 << 20), np.uint32, 1 << 18)
            if not np.array_equal(got, np.arange(int(start) << 18, (int(start) + 1) << 18, dtype=np.uint32)):
                raise SystemExit("[bench] PARITY FAILURE in PERM-ref: permuting twice does not restore the input")
        return "256 sampled output rows equal the closed form; permuting twice restores 64 sampled MiB of the input bit for bit"

    def cpu_baseline(self, budget_s=10.0):
        return None

    def free(self):
        for s_, d in self.sets:
            s_.free()
            d.free()
        self.sets = []


class AuxChainWorkload:
    """BASELINE config 3: the 10-op f32 pointwise chain ending in Sum(batch) and Sum(columns), one fused kernel.
    Algorithmic bytes: four [1,4096,4096] f32 inputs + the bias + both outputs = 268,468,228."""

    bound = "hbm"
    unit = "GB/s"
    dtype = "f32"
    name = "C3"

    def __init__(self):
        self.work = 4 * 4096 * 4096 * 4 + 4096 * 4 + (4096 + 1) * 4

    def describe(self):
        return "C3: f32 [1,4096,4096] 10-op chain + Sum(batch) + Sum(columns), one kernel"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs

        self.graph, self.inputs, self.outs = configs.c3_chain()
        self.kernel = ha.TileKernel.auxiliary(self.graph)
        nsets = 4  # 4 x 268 MB of operands rotate through the caches
        self.sets = []
        for s in range(nsets):
            bufs = []
            for a in self.kernel.args:
                if a["is_output"]:
                    bufs.append(ha.DeviceBuffer(a["numel"] * 4))
                else:
                    bufs.append(ha.DeviceBuffer.from_numpy(self.inputs[a["node"]]))
            self.sets.append(bufs)
        log(f"[bench] {self.describe()} :: {self.kernel.description} :: {nsets} operand sets")

    def step(self, stream, i):
        self.kernel.execute(self.sets[i % len(self.sets)], stream)

    def check(self):
        from oracle import fusion_ir as oracle

        want = oracle.outputs(self.graph.nodes, self.inputs)
        for a, buf in zip(self.kernel.args, self.sets[0]):
            if not a["is_output"]:
                continue
            got = buf.to_numpy(np.float32)[: a["numel"]]
            w = want[a["node"]].reshape(-1)
            err = np.max(np.abs(got.astype(np.float64) - w) / np.maximum(np.abs(w), 1e-30))
            if not err <= 1e-3:
                raise SystemExit(f"[bench] PARITY FAILURE in C3 output {a['node']}: max rel err {err}")
        return "reductions within 1e-3 relative of the f64-summed oracle"

    def cpu_baseline(self, budget_s=20.0):
        from oracle import fusion_ir as oracle

        rows = 512  # bounded sample: the first 512 of 4096 rows of every operand
        sample = {k: np.ascontiguousarray(v[:, :rows]) if v.shape[1] == 4096 else v for k, v in self.inputs.items()}
        nodes = [dict(n) for n in self.graph.nodes]
        for n in nodes:
            if n["op"] == "producer" and n["shape"][1] == 4096:
                n["shape"] = [1, rows, n["shape"][2]]
            if n["op"] == "broadcast" and n["axis"] == 1:
                n["amount"] = rows
        best, reps, t_all = 1e30, 0, time.perf_counter()
        while reps < 2 or (time.perf_counter() - t_all < budget_s and reps < 5):
            t0 = time.perf_counter()
            oracle.evaluate(nodes, sample)
            best = min(best, time.perf_counter() - t0)
            reps += 1
        work = self.work * rows / 4096
        return {"value": round(work / best / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"first {rows} of 4096 rows of the C3 operands, numpy oracle, best of {reps} passes"}

    def free(self):
        for bufs in self.sets:
            for b in bufs:
                b.free()
        self.sets = []


class LinearLayerWorkload:
    """BASELINE config 1 through the whole backend path: execute_graph on the lazy-graph form of
    Y = relu(X W + b) plus the column sums (plan generation from cache, pooled allocation, a fused f32 GEMM with
    its epilogue and one pointwise/reduction kernel). 0.13 GFLOP: latency-bound, reported as time per graph.
    The executor owns its streams, so the time is the host's wall clock around K executions and one device sync."""

    bound = "mfma"
    unit = "TFLOP/s"
    dtype = "f32"
    name = "C1"
    peak = F32_PEAK_TFLOPS
    wall_timed = True

    def __init__(self):
        self.work = 2.0 * 256 * 512 * 512

    def describe(self):
        return "C1: f32 X[256,512] W[512,512] + b, relu, column sums via execute_graph (1 kernel)"

    def setup(self):
        from helium_amd import configs
        from helium_amd.backend import Plan, Tensor

        self.graph, self.names = configs.c1_ir_graph()
        self.host = configs.c1_inputs(self.names, batched=False)
        self.tensors = {i: Tensor.from_numpy(a, "f32") for i, a in self.host.items()}
        self.plan = Plan(self.graph)
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + self.plan.text.replace("\n", " ; "))

    def step(self, stream, i):
        from helium_amd.backend import execute_graph

        self.last = execute_graph(self.graph, self.tensors)

    def check(self):
        from oracle import helium_ir as oracle

        val, _ = oracle.evaluate(self.graph.nodes, self.host)
        y = self.last[self.names["y"]].to_numpy().astype(np.float64)
        want = val[self.names["y"]].astype(np.float64).reshape(-1)
        if not (np.abs(y - want) <= 1e-4 * np.maximum(np.abs(want), 1.0)).all():
            raise SystemExit("[bench] PARITY FAILURE in C1: Y differs from the oracle")
        cs = self.last[self.names["colsum"]].to_numpy().astype(np.float64)
        want_cs = val[self.names["y"]].astype(np.float64).sum(axis=0)
        if not (np.abs(cs - want_cs) <= 1e-3 * np.abs(want_cs) + 1e-4).all():
            raise SystemExit("[bench] PARITY FAILURE in C1: column sums differ from the oracle")
        return "Y within 1e-4, column sums within 1e-3 relative of the f64 oracle"

    def cpu_baseline(self, budget_s=5.0):
        from oracle import helium_ir as oracle

        best, reps, t_all = 1e30, 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t_all < budget_s and reps < 50):
            t0 = time.perf_counter()
            oracle.evaluate(self.graph.nodes, self.host)
            best = min(best, time.perf_counter() - t0)
            reps += 1
        return {"value": round(self.work / best / 1e12, 5), "unit": "TFLOP/s", "cores": os.cpu_count(), "kind": "port",
                "sample": f"the whole C1 graph, numpy oracle (float64 BLAS matmul), best of {reps} passes"}

    def free(self):
        self.tensors, self.last = {}, None


class BatchNormWorkload:
    """The non-convolution part of BASELINE config 5b that dominates its memory traffic: BatchNorm2d::forward in
    Train mode followed by Relu (helium/src/modules/batch_norm.rs:32-72) on an NHWC bf16 activation of
    [64,56,56,256], through execute_graph. Algorithmic bytes: x is read for the statistics and again to normalise
    (the second pass needs the first one's result), y is written once: 3 * 64*56*56*256 * 2 B."""

    bound = "hbm"
    unit = "GB/s"
    dtype = "bf16 storage, f32 math"
    name = "C5b-bn"
    wall_timed = True
    shape = (64, 56, 56, 256)

    def __init__(self):
        self.work = 3 * int(np.prod(self.shape)) * 2

    def describe(self):
        return "C5b-bn: bf16 [64,56,56,256] BatchNorm2d train forward + relu via execute_graph"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs
        from harness import frontend
        from helium_amd.backend import Plan, Tensor

        g = ha.ir.OpGraph()
        rec = frontend.Recorder(g)
        c = self.shape[3]
        x = g.new_input(list(self.shape), "bf16")
        params = [g.new_input([c], "f32") for _ in range(4)]
        y, new_mean, new_var = frontend.batch_norm_train(rec, x, *params)
        self.outs = {"y": g.new_output(y), "mean": g.new_output(new_mean), "var": g.new_output(new_var)}
        rng = np.random.default_rng(52)
        self.host = {x: configs.bf16_rne((rng.standard_normal(self.shape, dtype=np.float32) * 1.5 + 0.3)),
                     params[0]: np.zeros(c, np.float32), params[1]: np.ones(c, np.float32),
                     params[2]: rng.uniform(0.5, 1.5, c).astype(np.float32),
                     params[3]: rng.standard_normal(c).astype(np.float32), **rec.scalars}
        self.x, self.params, self.graph = x, params, g
        by_id = {n["id"]: n for n in g.nodes}
        self.tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(g).text.replace("\n", " ; "))

    def step(self, stream, i):
        from helium_amd.backend import execute_graph

        self.last = execute_graph(self.graph, self.tensors)

    def check(self):
        """Closed form of the graph in float64: per-channel statistics over all of x, y on 4096 sampled pixels."""
        from oracle import numerics as nm

        c = self.shape[3]
        x = nm.bf16_bits_to_f32(self.host[self.x]).reshape(-1, c)
        mean = x.mean(axis=0, dtype=np.float64)
        var = (x.astype(np.float64) ** 2).mean(axis=0) - mean ** 2
        got_mean = self.last[self.outs["mean"]].to_numpy().astype(np.float64)
        got_var = self.last[self.outs["var"]].to_numpy().astype(np.float64)
        # running statistics start at 0 / 1 and move by a tenth of the batch statistics
        if not np.allclose(got_mean, 0.1 * mean, rtol=1e-3, atol=1e-4) or not np.allclose(got_var, 0.9 + 0.1 * var, rtol=1e-3, atol=1e-4):
            raise SystemExit("[bench] PARITY FAILURE in C5b-bn: running statistics differ from the closed form")
        rows = np.random.default_rng(3).integers(0, x.shape[0], 4096)
        scale, bias = self.host[self.params[2]].astype(np.float64), self.host[self.params[3]].astype(np.float64)
        want = np.maximum((x[rows] - mean) / np.sqrt(var + 1e-3) * scale + bias, 0.0)
        y = nm.bf16_bits_to_f32(self.last[self.outs["y"]].to_numpy()).reshape(-1, c)[rows].astype(np.float64)
        if not np.allclose(y, want, rtol=2e-2, atol=2e-2):
            raise SystemExit("[bench] PARITY FAILURE in C5b-bn: y differs from the closed form")
        return "running statistics within 1e-3, y (4096 sampled pixels) within 2e-2 of the f64 closed form"

    def cpu_baseline(self, budget_s=5.0):
        return None

    def free(self):
        self.tensors, self.last = {}, None


class ConvWorkload:
    """One convolution of BASELINE config 5b's network through execute_graph: the 3x3, stride-1 convolution of a
    64-channel residual block on a bf16 NHWC activation of [64,56,56,64] (resnet-train/src/model.rs), run as an
    implicit GEMM: M = 64*56*56 output pixels, N = 64 output channels, K = 3*3*64 filter taps."""

    bound = "mfma"
    unit = "TFLOP/s"
    dtype = "bf16 x bf16 -> f32 accumulate, bf16 output"
    name = "C5b-conv"
    wall_timed = True
    image = (64, 56, 56, 64)
    out_channels = 64
    kernel = (3, 3)

    def __init__(self):
        n, h, w, c = self.image
        self.work = 2.0 * n * h * w * self.out_channels * self.kernel[0] * self.kernel[1] * c

    def describe(self):
        return "C5b-conv: bf16 [64,56,56,64] conv 3x3 -> 64 channels via execute_graph (implicit GEMM 200704 x 64 x 576)"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs
        from helium_amd.backend import Plan, Tensor

        g = ha.ir.OpGraph()
        c = self.image[3]
        fshape = [self.out_channels, self.kernel[0], self.kernel[1], c]
        x = g.new_input(list(self.image), "bf16")
        w = g.new_input(fshape, "bf16")
        self.params = {"in_channels": c, "out_channels": self.out_channels, "kernel_size": list(self.kernel)}
        y = g.conv(x, w, self.params)
        self.out = g.new_output(y)
        rng = np.random.default_rng(53)
        self.host = {x: configs.bf16_rne(rng.standard_normal(self.image, dtype=np.float32)),
                     w: configs.bf16_rne(rng.standard_normal(fshape, dtype=np.float32) * 0.05)}
        self.x, self.w, self.graph = x, w, g
        self.tensors = {i: Tensor.from_numpy(a, "bf16", a.size) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(g).text.replace("\n", " ; "))

    def step(self, stream, i):
        from helium_amd.backend import execute_graph

        self.last = execute_graph(self.graph, self.tensors)

    def check(self):
        """The oracle's cross-correlation on the first two images of the batch."""
        from oracle import helium_ir as oracle
        from oracle import numerics as nm

        img = nm.bf16_bits_to_f32(self.host[self.x]).reshape(self.image)[:2]
        flt = nm.bf16_bits_to_f32(self.host[self.w]).reshape(self.out_channels, *self.kernel, self.image[3])
        want = oracle.conv(img, flt, self.params, "bf16").astype(np.float64)
        got = nm.bf16_bits_to_f32(self.last[self.out].to_numpy()).reshape(self.image[0], -1)[:2].reshape(want.shape).astype(np.float64)
        if not (np.abs(got - want) <= 1e-2 * np.maximum(np.abs(want), 1.0)).all():
            raise SystemExit("[bench] PARITY FAILURE in C5b-conv: output differs from the oracle")
        return "first two images within 1e-2 of the oracle's float64 cross-correlation"

    def cpu_baseline(self, budget_s=5.0):
        return None

    def free(self):
        self.tensors, self.last = {}, None


class ConvBatchNormWorkload(ConvWorkload):
    """The first half of a residual block of BASELINE config 5b (resnet-train/src/model.rs): 3x3 convolution ->
    BatchNorm2d in Train mode -> relu, one graph through execute_graph. The convolution's kernel also folds its output
    per channel (the batch norm's statistics); two pointwise kernels finish the batch norm. Work = the convolution's
    FLOP."""

    name = "C5b-conv-bn"

    def describe(self):
        return "C5b-conv-bn: bf16 [64,56,56,64] conv 3x3 -> 64 channels -> BatchNorm2d train -> relu via execute_graph"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs
        from harness import frontend
        from helium_amd.backend import Plan, Tensor

        g = ha.ir.OpGraph()
        rec = frontend.Recorder(g)
        c, oc = self.image[3], self.out_channels
        fshape = [oc, self.kernel[0], self.kernel[1], c]
        x = g.new_input(list(self.image), "bf16")
        w = g.new_input(fshape, "bf16")
        self.params = {"in_channels": c, "out_channels": oc, "kernel_size": list(self.kernel)}
        conv = g.conv(x, w, self.params)
        bn = [g.new_input([oc], "f32") for _ in range(4)]
        y, new_mean, new_var = frontend.batch_norm_train(rec, conv, *bn)
        self.outs = {"conv": g.new_output(conv), "y": g.new_output(y), "mean": g.new_output(new_mean), "var": g.new_output(new_var)}
        rng = np.random.default_rng(58)
        self.host = {x: configs.bf16_rne(rng.standard_normal(self.image, dtype=np.float32)),
                     w: configs.bf16_rne(rng.standard_normal(fshape, dtype=np.float32) * 0.05),
                     bn[0]: np.zeros(oc, np.float32), bn[1]: np.ones(oc, np.float32),
                     bn[2]: rng.uniform(0.5, 1.5, oc).astype(np.float32), bn[3]: rng.standard_normal(oc).astype(np.float32),
                     **rec.scalars}
        self.x, self.w, self.bn, self.graph = x, w, bn, g
        by_id = {n["id"]: n for n in g.nodes}
        self.tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(g).text.replace("\n", " ; "))

    def check(self):
        """The convolution's first two images against the oracle; statistics and y against the f64 closed form of the
        batch norm applied to the convolution output the device stored."""
        from oracle import helium_ir as oracle
        from oracle import numerics as nm

        oc = self.out_channels
        img = nm.bf16_bits_to_f32(self.host[self.x]).reshape(self.image)[:2]
        flt = nm.bf16_bits_to_f32(self.host[self.w]).reshape(oc, *self.kernel, self.image[3])
        want = oracle.conv(img, flt, self.params, "bf16").astype(np.float64)
        conv = nm.bf16_bits_to_f32(self.last[self.outs["conv"]].to_numpy()).reshape(-1, oc)
        got = conv.reshape(self.image[0], -1)[:2].reshape(want.shape).astype(np.float64)
        if not (np.abs(got - want) <= 1e-2 * np.maximum(np.abs(want), 1.0)).all():
            raise SystemExit("[bench] PARITY FAILURE in C5b-conv-bn: convolution differs from the oracle")
        mean = conv.mean(axis=0, dtype=np.float64)
        var = (conv.astype(np.float64) ** 2).mean(axis=0) - mean ** 2
        got_mean = self.last[self.outs["mean"]].to_numpy().astype(np.float64)
        got_var = self.last[self.outs["var"]].to_numpy().astype(np.float64)
        if not np.allclose(got_mean, 0.1 * mean, rtol=1e-3, atol=1e-4) or not np.allclose(got_var, 0.9 + 0.1 * var, rtol=1e-3, atol=1e-4):
            raise SystemExit("[bench] PARITY FAILURE in C5b-conv-bn: running statistics differ from the closed form")
        rows = np.random.default_rng(3).integers(0, conv.shape[0], 4096)
        scale, bias = self.host[self.bn[2]].astype(np.float64), self.host[self.bn[3]].astype(np.float64)
        want_y = np.maximum((conv[rows] - mean) / np.sqrt(var + 1e-3) * scale + bias, 0.0)
        y = nm.bf16_bits_to_f32(self.last[self.outs["y"]].to_numpy()).reshape(-1, oc)[rows].astype(np.float64)
        if not np.allclose(y, want_y, rtol=2e-2, atol=2e-2):
            raise SystemExit("[bench] PARITY FAILURE in C5b-conv-bn: y differs from the closed form")
        return "conv (2 images) within 1e-2 of the oracle; statistics within 1e-3, y (4096 pixels) within 2e-2 of the f64 closed form"


class ConvBackwardDataWorkload(ConvWorkload):
    """The gradient of the same layer with respect to its input (Op::ConvBackwardData): an implicit GEMM whose rows are
    the image pixels, A the flow gathered through the filter taps, B the filter's [o][r][s][:] rows."""

    name = "C5b-conv-bwd-data"

    def describe(self):
        return "C5b-conv-bwd-data: bf16 flow [64,56,56,64] x filter [64,3,3,64] -> image gradient via execute_graph (implicit GEMM 200704 x 64 x 576)"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs
        from helium_amd.backend import Plan, Tensor

        g = ha.ir.OpGraph()
        n, h, w_, c = self.image
        fshape = [self.out_channels, self.kernel[0], self.kernel[1], c]
        dy = g.new_input([n, h, w_, self.out_channels], "bf16")
        w = g.new_input(fshape, "bf16")
        self.params = {"in_channels": c, "out_channels": self.out_channels, "kernel_size": list(self.kernel)}
        self.out = g.new_output(g.conv_backward_data(dy, w, self.params, [h, w_]))
        rng = np.random.default_rng(54)
        self.host = {dy: configs.bf16_rne(rng.standard_normal((n, h, w_, self.out_channels), dtype=np.float32)),
                     w: configs.bf16_rne(rng.standard_normal(fshape, dtype=np.float32) * 0.05)}
        self.dy, self.w, self.graph = dy, w, g
        self.tensors = {i: Tensor.from_numpy(a, "bf16", a.size) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(g).text.replace("\n", " ; "))

    def check(self):
        from oracle import helium_ir as oracle
        from oracle import numerics as nm

        n, h, w_, c = self.image
        flow = nm.bf16_bits_to_f32(self.host[self.dy]).reshape(n, h, w_, self.out_channels)[:2]
        flt = nm.bf16_bits_to_f32(self.host[self.w]).reshape(self.out_channels, *self.kernel, c)
        want = oracle.conv_backward_data(flow, flt, self.params, (h, w_)).astype(np.float64)
        got = nm.bf16_bits_to_f32(self.last[self.out].to_numpy()).reshape(n, -1)[:2].reshape(want.shape).astype(np.float64)
        if not (np.abs(got - want) <= 1e-2 * np.maximum(np.abs(want), 1.0)).all():
            raise SystemExit("[bench] PARITY FAILURE in C5b-conv-bwd-data: output differs from the oracle")
        return "first two images within 1e-2 of the oracle's float64 adjoint"


class ConvBackwardFilterWorkload(ConvWorkload):
    """The gradient of the same layer with respect to its filter (Op::ConvBackwardFilter): rows = output channels,
    k = the 200704 output pixels, split over many workgroups per tile whose partial tiles a second launch adds."""

    name = "C5b-conv-bwd-filter"

    def describe(self):
        return "C5b-conv-bwd-filter: bf16 flow [64,56,56,64] x image [64,56,56,64] -> filter gradient via execute_graph (implicit GEMM 64 x 576 x 200704, split-k)"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs
        from helium_amd.backend import Plan, Tensor

        g = ha.ir.OpGraph()
        n, h, w_, c = self.image
        dy = g.new_input([n, h, w_, self.out_channels], "bf16")
        x = g.new_input(list(self.image), "bf16")
        self.params = {"in_channels": c, "out_channels": self.out_channels, "kernel_size": list(self.kernel)}
        self.out = g.new_output(g.conv_backward_filter(dy, x, self.params))
        rng = np.random.default_rng(55)
        self.host = {dy: configs.bf16_rne(rng.standard_normal((n, h, w_, self.out_channels), dtype=np.float32) * 0.05),
                     x: configs.bf16_rne(rng.standard_normal(self.image, dtype=np.float32))}
        self.dy, self.x, self.graph = dy, x, g
        self.tensors = {i: Tensor.from_numpy(a, "bf16", a.size) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(g).text.replace("\n", " ; "))

    def check(self):
        """32 filter taps, each as one float64 dot product over all output pixels (zero padding by slicing)."""
        from oracle import numerics as nm

        n, h, w_, c = self.image
        flow = nm.bf16_bits_to_f32(self.host[self.dy]).reshape(n, h, w_, self.out_channels)
        img = nm.bf16_bits_to_f32(self.host[self.x]).reshape(self.image)
        got = nm.bf16_bits_to_f32(self.last[self.out].to_numpy()).reshape(self.out_channels, *self.kernel, c).astype(np.float64)
        rng = np.random.default_rng(56)
        for _ in range(32):
            o, r, s_, ch = (int(rng.integers(self.out_channels)), int(rng.integers(self.kernel[0])),
                            int(rng.integers(self.kernel[1])), int(rng.integers(c)))
            dr, ds = r - self.kernel[0] // 2, s_ - self.kernel[1] // 2   # image pixel = output pixel + (dr, ds)
            p0, p1 = max(0, -dr), min(h, h - dr)
            q0, q1 = max(0, -ds), min(w_, w_ - ds)
            want = float(np.sum(flow[:, p0:p1, q0:q1, o].astype(np.float64) * img[:, p0 + dr:p1 + dr, q0 + ds:q1 + ds, ch].astype(np.float64)))
            scale = max(abs(want), 5.0)   # a sum of 200704 products of magnitude 0.05: the bf16 result carries 2^-9 relative
            if abs(got[o, r, s_, ch] - want) > 1e-2 * scale:
                raise SystemExit(f"[bench] PARITY FAILURE in C5b-conv-bwd-filter: tap {(o, r, s_, ch)} is {got[o, r, s_, ch]}, want {want}")
        return "32 sampled taps within 1e-2 of float64 dot products over all 200704 output pixels"


class SgdWorkload:
    """The optimizer step of BASELINE config 5b for one parameter tensor (helium/src/optimizer/sgd.rs:42-66): momentum
    average and weight update of a bf16 [512,3,3,512] filter (the largest of the network) with its f32 average, one
    pointwise kernel through execute_graph. Bytes: weights and gradient read as bf16, average read and written as f32,
    weights written as bf16."""

    bound = "hbm"
    unit = "GB/s"
    dtype = "bf16 storage, f32 math"
    name = "C5b-sgd"
    wall_timed = True
    shape = (512, 3, 3, 512)

    def __init__(self):
        n = int(np.prod(self.shape))
        self.work = n * (2 + 2 + 4 + 4 + 2)

    def describe(self):
        return "C5b-sgd: SGD momentum step of a bf16 [512,3,3,512] filter (f32 average) via execute_graph"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs
        from harness import frontend
        from helium_amd.backend import Plan, Tensor

        g = ha.ir.OpGraph()
        rec = frontend.Recorder(g)
        w = g.new_input(list(self.shape), "bf16")
        grad = g.new_input(list(self.shape), "bf16")
        avg = g.new_input(list(self.shape), "f32")
        new_w, new_avg = frontend.sgd_momentum_step(rec, w, grad, avg, momentum=0.9, learning_rate=0.1)
        self.out_w, self.out_avg = g.new_output(new_w), g.new_output(new_avg)
        rng = np.random.default_rng(57)
        self.host = {w: configs.bf16_rne(rng.standard_normal(self.shape, dtype=np.float32) * 0.05),
                     grad: configs.bf16_rne(rng.standard_normal(self.shape, dtype=np.float32) * 0.01),
                     avg: (rng.standard_normal(self.shape, dtype=np.float32) * 0.01), **rec.scalars}
        self.w, self.grad, self.avg, self.graph = w, grad, avg, g
        by_id = {n["id"]: n for n in g.nodes}
        self.tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(g).text.replace("\n", " ; "))

    def step(self, stream, i):
        from helium_amd.backend import execute_graph

        self.last = execute_graph(self.graph, self.tensors)

    def check(self):
        from oracle import numerics as nm

        w = nm.bf16_bits_to_f32(self.host[self.w]).astype(np.float64).reshape(-1)
        gr = nm.bf16_bits_to_f32(self.host[self.grad]).astype(np.float64).reshape(-1)
        av = self.host[self.avg].astype(np.float64).reshape(-1)
        want_avg = 0.1 * gr + 0.9 * av
        got_avg = self.last[self.out_avg].to_numpy().astype(np.float64)
        got_w = nm.bf16_bits_to_f32(self.last[self.out_w].to_numpy()).astype(np.float64)
        if not np.allclose(got_avg, want_avg, rtol=1e-5, atol=1e-7):
            raise SystemExit("[bench] PARITY FAILURE in C5b-sgd: momentum average differs from the closed form")
        want_w = w - 0.1 * want_avg
        if not (np.abs(got_w - want_w) <= 2.0 ** -8 * np.maximum(np.abs(want_w), 1e-4)).all():
            raise SystemExit("[bench] PARITY FAILURE in C5b-sgd: weights differ from the closed form")
        return "average within 1e-5 (f32), weights within one bf16 rounding of the f64 closed form"

    def cpu_baseline(self, budget_s=5.0):
        return None

    def free(self):
        self.tensors, self.last = {}, None


class BasicBlockWorkload:
    """One residual block of BASELINE config 5b's network, forward in Train mode (BasicBlock::forward,
    resnet-train/src/model.rs:155-165): bn -> relu -> conv 3x3 -> bn -> relu -> conv 3x3 -> + shortcut on a bf16 NHWC
    activation of [64,56,56,64], one graph through execute_graph. Work = the two convolutions' FLOP."""

    bound = "mfma"
    unit = "TFLOP/s"
    dtype = "bf16 storage, bf16 x bf16 -> f32 products, f32 math"
    name = "C5b-block"
    wall_timed = True
    shape = (64, 56, 56, 64)

    def __init__(self):
        n, h, w, c = self.shape
        self.work = 2 * 2.0 * n * h * w * c * 9 * c

    def describe(self):
        return "C5b-block: bf16 [64,56,56,64] residual block forward (bn, relu, conv 3x3, bn, relu, conv 3x3, + shortcut) via execute_graph"

    @staticmethod
    def build(shape, seed):
        import helium_amd as ha
        from helium_amd import configs
        from harness import frontend

        g = ha.ir.OpGraph()
        rec = frontend.Recorder(g)
        c = shape[3]
        x = g.new_input(list(shape), "bf16")
        bn1 = [g.new_input([c], "f32") for _ in range(4)]
        bn2 = [g.new_input([c], "f32") for _ in range(4)]
        k1, b1 = g.new_input([c, 3, 3, c], "bf16"), g.new_input([c], "bf16")
        k2, b2 = g.new_input([c, 3, 3, c], "bf16"), g.new_input([c], "bf16")
        out, stats = frontend.basic_block_forward(rec, x, bn1, k1, b1, bn2, k2, b2)
        outs = [g.new_output(out)] + [g.new_output(s) for s in stats]
        rng = np.random.default_rng(seed)
        host = {x: configs.bf16_rne(rng.standard_normal(shape, dtype=np.float32) * 1.2 + 0.2)}
        for bn in (bn1, bn2):
            host[bn[0]] = np.zeros(c, np.float32)
            host[bn[1]] = np.ones(c, np.float32)
            host[bn[2]] = rng.uniform(0.5, 1.5, c).astype(np.float32)
            host[bn[3]] = rng.standard_normal(c).astype(np.float32) * 0.5
        for k, b in ((k1, b1), (k2, b2)):
            host[k] = configs.bf16_rne(rng.standard_normal((c, 3, 3, c), dtype=np.float32) * 0.06)   # Kaiming: sqrt(2 / (9 c))
            host[b] = configs.bf16_rne(rng.standard_normal(c, dtype=np.float32) * 0.1)
        host.update(rec.scalars)
        return g, host, outs

    def setup(self):
        from helium_amd.backend import Plan, Tensor

        self.graph, self.host, self.outs = self.build(self.shape, 59)
        by_id = {n["id"]: n for n in self.graph.nodes}
        self.tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in self.host.items()}
        self.last = None
        log(f"[bench] {self.describe()} :: plan: " + Plan(self.graph).text.replace("\n", " ; "))

    def step(self, stream, i):
        from helium_amd.backend import execute_graph

        self.last = execute_graph(self.graph, self.tensors)

    def check(self):
        """The same graph at [4,12,12,64] against the oracle (kernel by kernel, as the plan groups it), and the full-size
        run's running statistics of the first batch norm against the float64 closed form."""
        from helium_amd.backend import Plan, Tensor, execute_graph
        from oracle import helium_ir as oracle
        from oracle import numerics as nm

        g, host, outs = self.build((4, 12, 12, 64), 60)
        by_id = {n["id"]: n for n in g.nodes}
        got = execute_graph(g, {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in host.items()})
        want = oracle.plan_outputs(g.nodes, host, Plan(g).steps)
        _, desc = oracle.evaluate(g.nodes, host)
        for o in outs:
            dt = desc[o][1]
            a = nm.from_storage(got[o].to_numpy(), dt, [got[o].len]).astype(np.float64)
            b = nm.from_storage(want[o].reshape(-1), dt, [want[o].size]).astype(np.float64)
            tol = 4e-2 if dt == "bf16" else 2e-3
            if not np.allclose(a, b, rtol=tol, atol=tol):
                raise SystemExit(f"[bench] PARITY FAILURE in C5b-block: output {o} differs from the oracle by {np.abs(a - b).max()}")
        c = self.shape[3]
        x = nm.bf16_bits_to_f32(self.host[next(iter(self.host))]).reshape(-1, c)
        mean = x.mean(axis=0, dtype=np.float64)
        var = (x.astype(np.float64) ** 2).mean(axis=0) - mean ** 2
        got_mean = self.last[self.outs[1]].to_numpy().astype(np.float64)
        got_var = self.last[self.outs[2]].to_numpy().astype(np.float64)
        if not np.allclose(got_mean, 0.1 * mean, rtol=1e-3, atol=1e-4) or not np.allclose(got_var, 0.9 + 0.1 * var, rtol=1e-3, atol=1e-4):
            raise SystemExit("[bench] PARITY FAILURE in C5b-block: running statistics differ from the closed form")
        return "all outputs of the same graph at [4,12,12,64] within 4e-2 (bf16) / 2e-3 (f32) of the oracle; first batch norm's statistics at full size within 1e-3"

    def cpu_baseline(self, budget_s=5.0):
        return None

    def free(self):
        self.tensors, self.last = {}, None


class FusedGemmWorkload:
    """BASELINE configs 4 / 5a: 4096^3 bf16 GEMM with fused mainloop / epilogue. Work = 2*M*N*K FLOP."""

    bound = "mfma"
    unit = "TFLOP/s"
    dtype = "bf16 x bf16 -> f32 accumulate, f32 epilogue"

    def __init__(self, name, size=4096):
        self.name, self.size = name, size
        self.work = 2 * size ** 3

    def describe(self):
        what = {"C4": "README 40-op LSTM-cell epilogue, 5 bf16 aux tensors, 3 reductions",
                "C4m": "C4 plus mainloop Relu*tensor on A and two bf16 full-size outputs",
                "C5a": "mainloop Relu*tensor on A, bias+Relu epilogue, bf16 output",
                "GEMM": "no fusion, bf16 output"}[self.name]
        return f"{self.name}: bf16 {self.size}^3 fused GEMM ({what})"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs

        n = self.size
        if self.name == "C4":
            self.graph, _ = configs.c4_graph(n)
            self.inputs = configs.c4_inputs(self.graph, n)
        elif self.name == "C4m":
            self.graph, _ = configs.c4_graph(n, mainloop=True, full_size_outputs=True)
            self.inputs = configs.c4_inputs(self.graph, n)
        elif self.name == "C5a":
            self.graph, names = configs.c5a_graph(n)
            self.inputs = configs.c5a_inputs(names, n)
        else:
            g = ha.fusion.OpGraph()
            a, b = g.producer([1, n, n], "bf16"), g.producer([1, n, n], "bf16")
            g.consumer(g.matmul(a, b), "bf16")
            rng = np.random.default_rng(61)
            self.graph = g
            self.inputs = {a: configs.bf16_rne((rng.standard_normal((1, n, n)) * 0.02).astype(np.float32)),
                           b: configs.bf16_rne((rng.standard_normal((1, n, n)) * 0.02).astype(np.float32))}
        self.kernel = ha.TileKernel.fused(self.graph)
        per_set = sum(v.nbytes for v in self.inputs.values())
        nsets = max(2, min(6, ROTATE_BYTES // per_set + 1))
        self.sets = []
        itemsize = {"bf16": 2, "f16": 2, "f32": 4}
        for _ in range(nsets):
            bufs = []
            for a in self.kernel.args:
                if a["is_output"]:
                    bufs.append(ha.DeviceBuffer(max(16, a["numel"] * itemsize[a["dtype"]])))
                else:
                    bufs.append(ha.DeviceBuffer.from_numpy(self.inputs[a["node"]]))
            self.sets.append(bufs)
        log(f"[bench] {self.describe()} :: {self.kernel.description} :: {nsets} operand sets")

    def step(self, stream, i):
        self.kernel.execute(self.sets[i % len(self.sets)], stream)

    def check(self):
        from oracle import fusion_ir as oracle
        from oracle import numerics as nm

        want = oracle.outputs(self.graph.nodes, self.inputs, round_mainloop_to="bf16")
        worst = 0.0
        for a, buf in zip(self.kernel.args, self.sets[0]):
            if not a["is_output"]:
                continue
            w = want[a["node"]].reshape(-1)
            if a["dtype"] == "bf16":
                got, w = nm.bf16_bits_to_f32(buf.to_numpy(np.uint16)[: a["numel"]]), nm.bf16_bits_to_f32(w)
                # full-size tensors: approx::relative_eq(epsilon 1e-3, max_relative 1e-2)
                d = np.abs(got.astype(np.float64) - w)
                ok = (d <= 1e-3) | (d <= 1e-2 * np.maximum(np.abs(got), np.abs(w)))
                if not ok.all():
                    raise SystemExit(f"[bench] PARITY FAILURE in {self.name} output {a['node']}: {int((~ok).sum())} elements off")
            else:
                got = buf.to_numpy(np.float32)[: a["numel"]].astype(np.float64)
                scale = max(float(np.abs(w).max()), 1e-30)
                err = float(np.max(np.abs(got - w)) / scale)
                worst = max(worst, err)
                if not err <= 1e-3:
                    raise SystemExit(f"[bench] PARITY FAILURE in {self.name} reduction {a['node']}: {err} of the largest element")
        return f"full-size outputs within 1e-2 relative, reductions within 1e-3 (worst {worst:.1e}) of the f64-accumulated oracle"

    def cpu_baseline(self, budget_s=25.0):
        from oracle import fusion_ir as oracle

        if self.name == "C4":
            return self.cpu_baseline_c()
        rows = 256  # bounded sample: the first 256 rows of A (and of every [1,M,N] tensor)
        n = self.size
        nodes = [dict(x) for x in self.graph.nodes]
        anchor = next(x for x in nodes if x["op"] == "matmul")
        m_side = set()
        stack = [anchor["a"]]
        by_id = {x["id"]: x for x in nodes}
        while stack:  # producers feeding the A operand keep their K extent, lose rows
            i = stack.pop()
            m_side.add(i)
            for key in ("a", "b", "x", "lhs", "rhs"):
                if key in by_id[i]:
                    stack.append(by_id[i][key])
        b_side = {anchor["b"]}
        sample = {}
        for x in nodes:
            if x["op"] in ("producer", "constant") and x["shape"][1] == n and x["id"] not in b_side:
                x["shape"] = [x["shape"][0], rows, x["shape"][2]]
            if x["op"] == "broadcast" and x["axis"] == 1:
                x["amount"] = rows
        for k, v in self.inputs.items():
            keep = v.reshape(by_id[k]["shape"] if v.ndim != 3 else v.shape)
            full = np.asarray(keep).reshape(self.graph.nodes[[y["id"] for y in self.graph.nodes].index(k)]["shape"])
            sample[k] = np.ascontiguousarray(full[:, :rows]) if (full.shape[1] == n and k not in b_side) else full
        best, reps, t_all = 1e30, 0, time.perf_counter()
        while reps < 2 or (time.perf_counter() - t_all < budget_s and reps < 4):
            t0 = time.perf_counter()
            oracle.evaluate(nodes, sample, round_mainloop_to="bf16")
            best = min(best, time.perf_counter() - t0)
            reps += 1
        flops = 2.0 * rows * n * n
        return {"value": round(flops / best / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count(), "kind": "port",
                "sample": f"first {rows} of {n} rows of the {self.name} problem, numpy oracle (float64 BLAS matmul on all "
                          f"cores + f32 epilogue), best of {reps} passes"}

    def cpu_baseline_c(self, reps=3):
        """The whole C4 problem on all host cores: oracle/c4_cpu.c (C + OpenMP restatement of the README fusion; the
        reference has no CPU path), checked against the GPU's outputs before it is timed."""
        from oracle import c4_cpu

        got = c4_cpu.c4(self.inputs, self.size)
        for a, buf in zip(self.kernel.args, self.sets[0]):
            if not a["is_output"]:
                continue
            gpu = buf.to_numpy(np.float32)[: a["numel"]].astype(np.float64)
            err = float(np.max(np.abs(gpu - got[a["node"]])) / max(float(np.abs(gpu).max()), 1e-30))
            if not err <= 1e-3:
                raise SystemExit(f"[bench] PARITY FAILURE: C restatement and GPU differ on C4 output {a['node']}: {err}")
        best = 1e30
        for _ in range(reps):
            t0 = time.perf_counter()
            c4_cpu.c4(self.inputs, self.size)
            best = min(best, time.perf_counter() - t0)
        return {"value": round(self.work / best / 1e12, 4), "unit": "TFLOP/s", "cores": c4_cpu.threads(), "kind": "port",
                "sample": f"the whole C4 problem ({self.size}^3 GEMM + 39-op epilogue + 3 reductions), C + OpenMP restatement of the "
                          f"reference's semantics (the reference has no CPU path), f32 accumulate, best of {reps} passes of "
                          f"{best:.2f} s, outputs within 1e-3 of the GPU's"}

    def free(self):
        for bufs in self.sets:
            for b in bufs:
                b.free()
        self.sets = []


class TrainStepWorkload:
    """BASELINE config 5b: one whole training step of the resnet-train example (resnet-train/src/train.rs:383-396 on the
    model of model.rs) through execute_graph: forward in Train mode, cross-entropy, backward, SGD with momentum 0.9.
    Every step feeds the previous step's parameters, gradient averages and running statistics back in. The work figure
    is the matrix-core FLOP of the step's convolutions (forward, data and filter gradients; the data gradient of the
    3-channel image is never asked for); images/s is reported next to it."""

    bound = "mfma"
    unit = "TFLOP/s"
    dtype = "bf16 activations and flows, f32 parameters and accumulation"
    wall_timed = True

    def __init__(self, name, batch, image):
        self.name, self.batch, self.image = name, batch, image
        self.work = 0

    def describe(self):
        return (f"{self.name}: resnet-train training step (forward, cross-entropy, backward, SGD momentum), batch {self.batch}, "
                f"{self.image}x{self.image}x3 bf16 images, 1000 classes, via execute_graph")

    def setup(self):
        from harness import resnet
        from helium_amd.backend import Tensor, stats

        self.rec = resnet.record_training_step(self.batch, self.image)
        G = self.rec["graph"]
        self.g = G.g
        by_id = {n["id"]: n for n in self.g.nodes}
        flop = 0
        for n in self.g.nodes:
            if n.get("op") in ("conv", "conv_bwd_data", "conv_bwd_filter"):
                p = n["params"]
                if n["op"] == "conv_bwd_data" and p["in_channels"] == 3:
                    continue  # the image has no gradient: pruned
                pixels = by_id[n["inputs"][0]]["shape"] if n["op"] != "conv" else n["shape"]
                flop += 2 * int(np.prod(pixels[:3])) * p["out_channels"] * p["kernel_size"][0] * p["kernel_size"][1] * p["in_channels"]
        self.work = flop
        self.tensors = {i: Tensor.from_numpy(a, by_id[i]["dtype"], int(np.prod(by_id[i]["shape"]))) for i, a in G.feeds.items()}
        self.outs = None
        self._stats = stats
        log(f"[bench] {self.describe()} :: {len(self.g.nodes)} graph nodes, {self.work / 1e9:.1f} GFLOP of convolutions per step")

    def step(self, stream, i):
        from helium_amd.backend import execute_graph

        outs = execute_graph(self.g, self.tensors)
        for src, dst in self.rec["carried"]:
            self.tensors[src] = outs[dst]
        self.outs = outs

    def check(self):
        st = self._stats()
        loss = float(self.outs[self.rec["loss"]].to_numpy()[0])
        probs = self.outs[self.rec["probs"]].to_numpy().reshape(self.batch, -1).astype(np.float64)
        if not (abs(loss - np.log(1000.0)) < 0.35 and np.allclose(probs.sum(axis=1), 1.0, atol=1e-3)):
            raise SystemExit(f"[bench] PARITY FAILURE in {self.name}: first-step loss {loss}, probabilities sum to {probs.sum(axis=1)[:4]}")
        self.instrs = st["instrs"]
        return (f"first step: loss {loss:.4f} (ln 1000 = 6.9078), probabilities sum to 1 per image; {st['instrs']} instructions in {st['steps']} plan "
                f"steps; the same graph at [8,64,64,3] agrees with the oracle output by output (tests/test_resnet_step_gpu.py)")

    def cpu_baseline(self, budget_s=5.0):
        return None

    def free(self):
        self.tensors, self.outs = {}, None


class PlannedGemmWorkload(FusedGemmWorkload):
    """The same graphs, run the way the fusion search plans them under the MI355X cost model (he_fusion_search with
    HE_FUSE_MIN_MI355X_COST, then he_fusion_plan_execute): a mainloop chain that 16 tile columns would each repeat is
    split off into a kernel of its own and the product reads its finished operand."""

    def __init__(self, name, size=4096):
        super().__init__(name, size)
        self.graph_name = name

    def describe(self):
        return super().describe() + " as planned by the fusion search (MI355X cost model)"

    def setup(self):
        import helium_amd as ha
        from helium_amd import configs, fusion_search as fs

        n = self.size
        if self.name == "C4m":
            self.graph, outs = configs.c4_graph(n, mainloop=True, full_size_outputs=True)
            self.inputs = configs.c4_inputs(self.graph, n)
            for node in ("loss", "db8", "db6"):  # bare reductions of the README listing: the search keeps what a Consumer reads
                self.graph.consumer(outs[node], "f32")
        else:
            self.graph, names = configs.c5a_graph(n)
            self.inputs = configs.c5a_inputs(names, n)
        self.plan = fs.FusionPlan(self.graph, fs.MIN_MI355X_COST)
        self.plan.precompile()
        itemsize = {"bf16": 2, "f16": 2, "f32": 4}
        used = {nd[k] for nd in self.graph.nodes for k in ("a", "b", "x", "lhs", "rhs") if k in nd}
        self.leaves = [nd for nd in self.graph.nodes if nd["id"] not in used]
        per_set = sum(v.nbytes for v in self.inputs.values())
        nsets = max(2, min(6, ROTATE_BYTES // per_set + 1))
        self.sets = []
        for _ in range(nsets):
            prod = {k: ha.DeviceBuffer.from_numpy(v) for k, v in self.inputs.items()}
            cons = {nd["id"]: ha.DeviceBuffer(max(16, int(np.prod(nd["shape"])) * itemsize[nd["dtype"]])) for nd in self.leaves}
            self.sets.append((prod, cons))
        kinds = " + ".join(("core(mainloop %d, epilogue %d)" % (len(f["mainloop"]), len(f["epilogue"]))) if f["core"] else "aux(%d ops)" % len(f["aux"])
                           for f in self.plan.fusions)
        log(f"[bench] {self.describe()} :: plan = {kinds}; predicted {self.plan.cost(fs.MIN_MI355X_COST) * 1e6:.1f} us :: {nsets} operand sets")
        log("[bench] chosen plan:\n" + self.plan.text)

    def step(self, stream, i):
        prod, cons = self.sets[i % len(self.sets)]
        self.plan.execute(prod, cons, stream=stream)

    def check(self):
        from oracle import fusion_ir as oracle
        from oracle import numerics as nm

        # values that cross from one kernel to the next are stored as bf16 (f32 for reductions)
        crossing = {}
        by_id = {nd["id"]: nd for nd in self.graph.nodes}
        for f in self.plan.fusions[:-1]:
            members = set(f["mainloop"] + f["epilogue"] + f["aux"])
            for nd in self.graph.nodes:
                for k in ("a", "b", "x", "lhs", "rhs"):
                    if k in nd and nd[k] in members and nd["id"] not in members and nd["op"] != "consumer":
                        crossing[nd[k]] = "f32" if by_id[nd[k]]["op"] == "reduction" else "bf16"
        want = oracle.outputs(self.graph.nodes, self.inputs, round_mainloop_to="bf16", materialize=crossing)
        worst = 0.0
        for nd in self.leaves:
            buf = self.sets[0][1][nd["id"]]
            numel = int(np.prod(nd["shape"]))
            w = want[nd["id"]].reshape(-1)
            if nd["dtype"] == "bf16":
                got, w = nm.bf16_bits_to_f32(buf.to_numpy(np.uint16)[:numel]), nm.bf16_bits_to_f32(w)
                d = np.abs(got.astype(np.float64) - w)
                ok = (d <= 1e-3) | (d <= 1e-2 * np.maximum(np.abs(got), np.abs(w)))
                if not ok.all():
                    raise SystemExit(f"[bench] PARITY FAILURE in {self.name} output {nd['id']}: {int((~ok).sum())} elements off")
            else:
                got = buf.to_numpy(np.float32)[:numel].astype(np.float64)
                err = float(np.max(np.abs(got - w)) / max(float(np.abs(w).max()), 1e-30))
                worst = max(worst, err)
                if not err <= 1e-3:
                    raise SystemExit(f"[bench] PARITY FAILURE in {self.name} reduction {nd['id']}: {err} of the largest element")
        return f"full-size outputs within 1e-2 relative, reductions within 1e-3 (worst {worst:.1e}) of the f64-accumulated oracle"

    def cpu_baseline(self, budget_s=25.0):
        return None

    def free(self):
        for prod, cons in self.sets:
            for b in list(prod.values()) + list(cons.values()):
                b.free()
        self.sets = []


CEILING_CHILD = r"""
import json, sys
import torch
assert torch.cuda.is_available()
n = 4096
sets = [(torch.randn(n, n, device='cuda', dtype=torch.bfloat16) * 0.02, torch.randn(n, n, device='cuda', dtype=torch.bfloat16) * 0.02) for _ in range(8)]
out = torch.empty(n, n, device='cuda', dtype=torch.bfloat16)
def run(fn):
    for i in range(200): fn(*sets[i % 8])
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for i in range(100): fn(*sets[i % 8])
    e.record(); torch.cuda.synchronize()
    return 2 * n ** 3 / (s.elapsed_time(e) / 100 * 1e-3) / 1e12
print("CEILINGS " + json.dumps({"hipblaslt_nn_TFLOPs": round(run(lambda a, b: torch.matmul(a, b, out=out)), 1),
                                "hipblaslt_nt_TFLOPs": round(run(lambda a, b: torch.matmul(a, b.t(), out=out)), 1)}))
"""


def vendor_gemm_ceiling():
    """The vendor library's bf16 4096^3 GEMM on the same box (torch.matmul -> hipBLASLt; NN, and NT = B stored [n][k]),
    with the same warm-up and operand rotation as the GEMM workload: the analogue of the reference's benchmark printing
    its kernel next to cuBLASLt (helium-kernel-generator/benches/src/main.rs:35-46). Measured in a child process of its
    own before this process touches the device, so nothing of it lies inside a timed region. Returns the two figures, or
    a reason string when torch is not usable."""
    import subprocess

    try:
        r = subprocess.run([sys.executable, "-c", CEILING_CHILD], capture_output=True, text=True, timeout=420)
    except Exception as e:  # noqa: BLE001
        return {"skipped": f"child process failed: {e}"}
    for line in r.stdout.splitlines():
        if line.startswith("CEILINGS "):
            return json.loads(line[9:])
    return {"skipped": "torch not usable: " + (r.stderr.strip().splitlines() or ["no output"])[-1][:200]}


def make_workloads():
    from helium_amd import configs

    w = {name: PermuteWorkload(name, shape, perm, {"C2a": 21, "C2b": 22, "C2c": 23}[name])
         for name, (shape, perm) in configs.PERMUTES.items()}
    # a plain copy of known size (identity permute): the measured ceiling the permute kernels are read against and
    # the scale for the FETCH_SIZE / WRITE_SIZE counters
    w["COPY"] = PermuteWorkload("COPY", (8192, 8192), (0, 1), 24)
    w["PERM-ref"] = ReferencePermuteWorkload()
    w["C1"] = LinearLayerWorkload()
    w["C3"] = AuxChainWorkload()
    w["C5b-bn"] = BatchNormWorkload()
    w["C5b-conv"] = ConvWorkload()
    w["C5b-conv-bn"] = ConvBatchNormWorkload()
    w["C5b-conv-bwd-data"] = ConvBackwardDataWorkload()
    w["C5b-conv-bwd-filter"] = ConvBackwardFilterWorkload()
    w["C5b-sgd"] = SgdWorkload()
    w["C5b-block"] = BasicBlockWorkload()
    w["C5b"] = TrainStepWorkload("C5b", 128, 224)          # BASELINE's batch and image size
    w["C5b-ref"] = TrainStepWorkload("C5b-ref", 64, 256)   # the reference's own (train.rs:33,286-287)
    for name in ("C4", "C5a", "C4m", "GEMM"):
        w[name] = FusedGemmWorkload(name)
    # C5a and C4m as one kernel each (every mainloop op fused) stay measurable next to the planned form
    w["C5a-fused"], w["C4m-fused"] = w.pop("C5a"), w.pop("C4m")
    w["C5a-fused"].traffic_key, w["C4m-fused"].traffic_key = "C5a-fused", "C4m-fused"
    w["C5a"], w["C4m"] = PlannedGemmWorkload("C5a"), PlannedGemmWorkload("C4m")
    w["C5a"].traffic_key, w["C4m"].traffic_key = "C5a-planned", "C4m-planned"
    return w


SETTLE_LAUNCHES = 200  # launches after which the device's clock has settled (see --warmup's comment in main)


def time_workload(wl, stream, steps, warmup, batches=1):
    """Returns (ms_per_step from HIP events on the launch stream, wall ms per step). When fewer warm-up steps are asked
    for than the clock needs to settle, the difference is run first, untimed like the warm-up itself. `batches` > 1:
    that many timed regions of `steps` steps each, one after the other, and the median of them (a region of twenty
    launches of a few microseconds is at the mercy of one hiccup of the host)."""
    import helium_amd as ha

    for i in range(max(0, SETTLE_LAUNCHES - warmup)):
        wl.step(stream, i)
    for i in range(warmup):
        wl.step(stream, i)
    results = []
    for b in range(batches):
        stream.synchronize()
        ha.device.synchronize()
        start, stop = ha.Event(), ha.Event()
        t0 = time.perf_counter()
        start.record(stream)
        for i in range(steps):
            wl.step(stream, warmup + b * steps + i)
        stop.record(stream)
        stop.synchronize()
        ha.device.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        results.append((start.elapsed_ms(stop) / steps, wall_ms))
    results.sort(key=lambda r: (r[1] if getattr(wl, "wall_timed", False) else r[0]))
    return results[len(results) // 2]


def roofline(wl, ms):
    if wl.bound == "hbm":
        achieved = wl.work / (ms * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = wl.work / (ms * 1e-3) / 1e12
        peak, unit = getattr(wl, "peak", BF16_PEAK_TFLOPS), "TFLOP/s"
    return {"bound": wl.bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": TRAFFIC_BYTES.get(getattr(wl, "traffic_key", wl.name))}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The device's clock settles only after some milliseconds of load: right after an idle phase it runs fast for a
    # few launches, dips for some tens, then recovers (the 4096^3 GEMM: 115 us, then 128-147 us, then 115 us again
    # from about the 100th launch on). 200 warm-up launches put the timed ones into the settled state.
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default=None, help="headline workload (default: the best-covered BASELINE config)")
    ap.add_argument("--only", action="store_true", help="measure the headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the vendor-library GEMM measured on the same box")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    ceilings = {"skipped": "--only / --no-ceilings"} if (args.only or args.no_ceilings) else vendor_gemm_ceiling()
    if "skipped" not in ceilings:
        log(f"[bench] same-box ceilings: hipBLASLt bf16 4096^3 NN {ceilings['hipblaslt_nn_TFLOPs']} / NT {ceilings['hipblaslt_nt_TFLOPs']} TFLOP/s")
    import helium_amd as ha

    ha.device.init(0)
    arch = ha.device.device_arch(0)
    cus = ha.device.device_attr(0)
    log(f"[bench] device 0: {arch}, {cus} CUs; roofline constants: HBM {HBM_PEAK_GBS} GB/s, "
        f"bf16 MFMA {BF16_PEAK_TFLOPS} TFLOP/s")
    workloads = make_workloads()
    headline = args.workload or HEADLINE
    if headline not in workloads:
        raise SystemExit(f"unknown workload {headline}; have {sorted(workloads)}")
    stream = ha.Stream()

    kernels = {}
    head = None
    order = [headline] + ([] if args.only else [k for k in workloads if k != headline])
    for name in order:
        wl = workloads[name]
        wl.setup()
        wl.step(stream, 0)
        stream.synchronize()
        parity = wl.check()
        # the headline is timed over exactly --steps steps; the other workloads, when --steps is small, over five such
        # regions of which the median is reported
        batches = 1 if name == headline or args.steps >= 100 else 5
        ms, wall = time_workload(wl, stream, args.steps, args.warmup, batches)
        if getattr(wl, "wall_timed", False):
            ms = wall  # launched on the executor's own streams: only the host clock brackets them
        rl = roofline(wl, ms)
        kernels[name] = {"workload": wl.describe(), "ms": round(ms, 5), "wall_ms": round(wall, 5), "parity": parity,
                         "roofline": rl}
        if isinstance(wl, TrainStepWorkload):
            kernels[name]["images_per_s"] = round(wl.batch / (ms * 1e-3), 1)
            log(f"[bench] {name}: {kernels[name]['images_per_s']} images/s")
        log(f"[bench] {name}: {ms * 1e3:.1f} us/step -> {rl['achieved']} {rl['unit']} ({rl['frac'] * 100:.1f}% of peak)")
        if name == headline:
            cpu = None if args.no_cpu else wl.cpu_baseline()
            head = (wl, ms, rl, cpu)
        wl.free()

    wl, ms, rl, cpu = head
    line = {
        "metric": METRIC,
        "value": rl["achieved"],
        "unit": rl["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl.dtype,
        "data": "synthetic",
        "config": {"workload": wl.describe(), "device": arch, "cus": cus,
                   "host_cores": os.cpu_count(), "untimed_launches_before_timing": max(SETTLE_LAUNCHES, args.warmup)},
        "roofline": rl,
        "cpu_baseline": cpu,
        # measured on this box in this run, outside every timed region: what a plain copy kernel of the permutes' design
        # reaches (the permute and pointwise figures are to be read against it, the published 8 TB/s is not reachable by
        # any copy) and the vendor library's GEMM
        "ceilings": dict(ceilings, copy_GBps=kernels["COPY"]["roofline"]["achieved"] if "COPY" in kernels else None),
        "kernels": kernels,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
