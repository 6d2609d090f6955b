#!/usr/bin/env python3
"""Headline benchmark: the single-op suite (matmul, batch_matmul, fused add+relu, softmax,
layernorm; fp32 and bf16) run through the C-ABI kernel library on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-models] [--only a,b]

A step is one pass over all ten ops with their inputs already resident in HBM.  Prints ONE JSON
line: whole-suite latency per pass, the roofline of the kernel that dominates the pass (and of
every other kernel under "kernels"), contraction shapes outside the suite ("extra_kernels"), the end-to-end latencies
of the four model configurations with percentiles and achieved TFLOP/s ("model_configs"; medians also under
"model_latency_ms"), and the CPU stand-ins timed on this host in the same run ("cpu_baseline": the C oracle on a
bounded sample and torch CPU eager, for the suite and for every model configuration).
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f32": 157.3}

WORKLOAD = "single-op suite fp32+bf16: matmul 2048^3, batch_matmul [32,512,64]x[32,64,512], add+relu [64,1024,1024], softmax [4096,4096], layernorm [8192,1024]"


def _uniform(shape, dtype, gen, device):
    # values ~U(-1,1), generated on the CPU so that every run sees the same bits
    t = torch.rand(shape, generator=gen, dtype=torch.float32) * 2 - 1
    return t.to(dtype).to(device)


class Case:
    """One op of the suite with `sets` rotating operand sets (so HBM-bound kernels cannot live in
    the 256 MB last-level cache) and its algorithmic work."""

    def __init__(self, name, dtype_name, bound, flops, bytes_, make, run, sets):
        self.name, self.dtype_name, self.bound, self.flops, self.bytes = name, dtype_name, bound, flops, bytes_
        # descriptors are built once per operand set; a timed call only crosses the C-ABI
        self.calls = [run(*make()) for _ in range(sets)]
        self.sets = sets

    def run(self, i):
        self.calls[i % self.sets].launch()


class _Sequence:
    """Several prepared calls launched one after the other: a group of kernels timed as one case."""

    def __init__(self, calls):
        self.calls = calls

    def launch(self, stream=None):
        for c in self.calls:
            c.launch(stream)


class _Cases(list):
    """Collects the suite; with a filter only the named cases are built (their operands allocated)."""

    def __init__(self, only):
        super().__init__()
        self.only = only

    def add(self, name, dtype_name, *rest):
        if not self.only or "all" in self.only or ("%s_%s" % (name, dtype_name)) in self.only:
            self.append(Case(name, dtype_name, *rest))


def build_cases(ops, device, only=()):
    gen = torch.Generator().manual_seed(0)
    cases = _Cases(list(only))
    for dt_name, dt, es in (("f32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
        M = N = K = 2048
        cases.add("matmul", dt_name, "mfma", 2.0 * M * N * K, (M * K + K * N + M * N) * es,
                          lambda: (_uniform((M, K), dt, gen, device), _uniform((K, N), dt, gen, device),
                                   torch.empty((M, N), dtype=dt, device=device)),
                          lambda a, b, o: ops.matmul(a, b, out=o, defer=True), 1)
        B, m, k, n = 32, 512, 64, 512
        nbytes = (B * m * k + B * k * n + B * m * n) * es
        cases.add("batch_matmul", dt_name, "hbm", 2.0 * B * m * n * k, nbytes,
                          lambda: (_uniform((B, m, k), dt, gen, device), _uniform((B, k, n), dt, gen, device),
                                   torch.empty((B, m, n), dtype=dt, device=device)),
                          lambda a, b, o: ops.batch_matmul(a, b, out=o, defer=True), max(1, int(1.2e9 // nbytes)))
        shape = (64, 1024, 1024)
        numel = 64 * 1024 * 1024
        prog = ops.make_program([("add", "r0", "in0", "in1"), ("relu", "r0", "r0")], "r0")
        cases.add("add_relu", dt_name, "hbm", 0.0, 3 * numel * es,
                          lambda: (_uniform(shape, dt, gen, device), _uniform(shape, dt, gen, device),
                                   torch.empty(shape, dtype=dt, device=device)),
                          lambda a, b, o, prog=prog, shape=shape, dt=dt: ops.elementwise(prog, [a, b], shape, dt, out=o, defer=True), 2)
        cases.add("softmax", dt_name, "hbm", 0.0, 2 * 4096 * 4096 * es,
                          lambda: (_uniform((4096, 4096), dt, gen, device), torch.empty((4096, 4096), dtype=dt, device=device)),
                          lambda x, o: ops.softmax(x, out=o, defer=True), 8)
        cases.add("layernorm", dt_name, "hbm", 0.0, (2 * 8192 * 1024 + 2 * 1024) * es,
                          lambda: (_uniform((8192, 1024), dt, gen, device), torch.ones(1024, dtype=dt, device=device),
                                   torch.zeros(1024, dtype=dt, device=device), torch.empty((8192, 1024), dtype=dt, device=device)),
                          lambda x, g, b, o: ops.layer_norm(x, g, b, 1e-5, out=o, defer=True), 16)
    # not part of the suite (config 3's hot kernel, for counter runs: bench.py --only conv_f32,conv_bf16): the 3x3
    # convolution of a ResNet-18 body layer at batch 16, 64 -> 64 channels on 56x56, channels-last
    for dt_name, dt, es in (("f32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
        if "conv_%s" % dt_name in cases.only:
            cl = torch.channels_last
            n, c, hw, f = 16, 64, 56, 64
            cases.add("conv", dt_name, "mfma", 2.0 * n * hw * hw * f * c * 9, (n * c * hw * hw + f * c * 9 + n * f * hw * hw) * es,
                      lambda: (_uniform((n, c, hw, hw), dt, gen, device).contiguous(memory_format=cl),
                               (_uniform((f, c, 3, 3), dt, gen, device) * 0.05).contiguous(memory_format=cl),
                               torch.empty((n, f, hw, hw), dtype=dt, device=device).contiguous(memory_format=cl)),
                      lambda x, w, o: ops.conv2d(x, w, pad=(1, 1, 1, 1), out=o, defer=True), 4)
    # not part of the suite: a plain device copy of known size, used to calibrate the profiler's
    # FETCH_SIZE / WRITE_SIZE counters (bench.py --only copy_f32)
    if "copy_f32" in cases.only:
        n = 64 * 1024 * 1024
        cases.add("copy", "f32", "hbm", 0.0, 2 * n * 4,
                  lambda: (_uniform((n,), torch.float32, gen, device), torch.empty(n, dtype=torch.float32, device=device)),
                  lambda x, o: ops.copy(x, out=o, defer=True), 2)
    return cases


def build_extra_cases(ops, device, only=()):
    """Contractions outside the suite that the model configurations are made of, reported under "extra_kernels" (not
    part of `value`): the bf16 matmul at 4096^3, the feed-forward products of the encoder block at batch 32 with their
    fused epilogues (Linear weights [N,K] consumed as transposed views), and the convolution classes of ResNet-18 at
    batch 16 (3x3 body layers channels-last in fp32 and bf16, the 7x7 stride-2 stem in NCHW)."""
    gen = torch.Generator().manual_seed(1)
    cases = _Cases(list(only))
    bf = torch.bfloat16
    n = 4096
    cases.add("matmul_4096", "bf16", "mfma", 2.0 * n * n * n, 3 * n * n * 2,
              lambda: (_uniform((n, n), bf, gen, device), _uniform((n, n), bf, gen, device), torch.empty((n, n), dtype=bf, device=device)),
              lambda a, b, o: ops.matmul(a, b, out=o, defer=True), 1)

    def linear(name, M, N, K, act, with_res):
        def make():
            return (_uniform((M, K), bf, gen, device), _uniform((N, K), bf, gen, device) * 0.05, _uniform((N,), bf, gen, device),
                    _uniform((M, N), bf, gen, device) if with_res else None, torch.empty((M, N), dtype=bf, device=device))
        cases.add(name, "bf16", "mfma", 2.0 * M * N * K, (M * K + N * K + M * N * (2 if with_res else 1) + N) * 2, make,
                  lambda x, w, b, r, o: ops.matmul(x, w.t(), ops.Epilogue(bias=b, residual=r, act=act), out=o, defer=True), 1)

    linear("encoder_ffn1_16384x3072x768_gelu", 16384, 3072, 768, "gelu", False)
    linear("encoder_ffn2_16384x768x3072_residual", 16384, 768, 3072, "none", True)
    linear("encoder_proj_16384x768x768_residual", 16384, 768, 768, "none", True)
    cl = torch.channels_last
    for dt_name, dt, es in (("f32", torch.float32, 4), ("bf16", bf, 2)):
        for c, hw in ((64, 56), (128, 28), (256, 14), (512, 7)):
            cases.add("conv3x3_%dch_%dx%d" % (c, hw, hw), dt_name, "mfma", 2.0 * 16 * hw * hw * c * c * 9,
                      (16 * c * hw * hw * 2 + c * c * 9) * es,
                      lambda c=c, hw=hw, dt=dt: (_uniform((16, c, hw, hw), dt, gen, device).contiguous(memory_format=cl),
                                                 (_uniform((c, c, 3, 3), dt, gen, device) * 0.05).contiguous(memory_format=cl),
                                                 torch.empty((16, c, hw, hw), dtype=dt, device=device).contiguous(memory_format=cl)),
                      lambda x, w, o: ops.conv2d(x, w, pad=(1, 1, 1, 1), out=o, defer=True), 2)
    # layers with work for the whole chip (batch 32): what the bf16 convolution reaches when it is not launch-bound
    for c, f, hw in ((256, 256, 56), (128, 128, 56), (128, 256, 28)):
        cases.add("conv3x3_%dto%d_%dx%d_batch32" % (c, f, hw, hw), "bf16", "mfma", 2.0 * 32 * hw * hw * c * f * 9,
                  (32 * (c + f) * hw * hw + c * f * 9) * 2,
                  lambda c=c, f=f, hw=hw: (_uniform((32, c, hw, hw), bf, gen, device).contiguous(memory_format=cl),
                                           (_uniform((f, c, 3, 3), bf, gen, device) * 0.05).contiguous(memory_format=cl),
                                           torch.empty((32, f, hw, hw), dtype=bf, device=device).contiguous(memory_format=cl)),
                  lambda x, w, o: ops.conv2d(x, w, pad=(1, 1, 1, 1), out=o, defer=True), 2)
    # The fallbacks: shapes the fast paths do not take.  Convolutions whose channel count is no multiple of 128 bytes'
    # worth of values, or that are grouped, run in NCHW on conv_f32_kernel (fp32) / conv_kernel (16-bit, element-wise
    # gather); attention layers whose head dim is not 64 keep their three kernels (scores with the scale in the
    # epilogue, softmax, probabilities x values), the [B H, S, S] scores going through HBM.
    for dt_name, dt, es in (("f32", torch.float32, 4), ("bf16", bf, 2)):
        cases.add("conv3x3_48ch_56x56_nchw", dt_name, "mfma", 2.0 * 16 * 56 * 56 * 48 * 48 * 9, (16 * 48 * 56 * 56 * 2 + 48 * 48 * 9) * es,
                  lambda dt=dt: (_uniform((16, 48, 56, 56), dt, gen, device), _uniform((48, 48, 3, 3), dt, gen, device) * 0.05,
                                 torch.empty((16, 48, 56, 56), dtype=dt, device=device)),
                  lambda x, w, o: ops.conv2d(x, w, pad=(1, 1, 1, 1), out=o, defer=True), 2)
        cases.add("conv3x3_128ch_groups32_28x28_nchw", dt_name, "mfma", 2.0 * 16 * 28 * 28 * 128 * 4 * 9, (16 * 128 * 28 * 28 * 2 + 128 * 4 * 9) * es,
                  lambda dt=dt: (_uniform((16, 128, 28, 28), dt, gen, device), _uniform((128, 4, 3, 3), dt, gen, device) * 0.05,
                                 torch.empty((16, 128, 28, 28), dtype=dt, device=device)),
                  lambda x, w, o: ops.conv2d(x, w, pad=(1, 1, 1, 1), group=32, out=o, defer=True), 2)
    for hd in (32, 128):
        bh, sq = 8 * 12, 512

        def make_attn(hd=hd):
            q, k, v = (_uniform((bh, sq, hd), bf, gen, device) for _ in range(3))
            return (q, k, v, torch.empty((bh, sq, sq), dtype=bf, device=device), torch.empty((bh, sq, sq), dtype=bf, device=device),
                    torch.empty((bh, sq, hd), dtype=bf, device=device))

        def run_attn(q, k, v, sc, pr, o, hd=hd):
            return _Sequence([ops.batch_matmul(q, k.transpose(1, 2), ops.Epilogue(alpha=hd ** -0.5), out=sc, defer=True),
                              ops.softmax(sc, out=pr, defer=True), ops.batch_matmul(pr, v, out=o, defer=True)])
        # algorithmic bytes: q, k, v in and the result out, once (what a fused kernel moves); the three kernels move the
        # scores four more times
        cases.add("attention_unfused_headdim%d_batch8_seq512" % hd, "bf16", "mfma", 4.0 * bh * sq * sq * hd, 4 * bh * sq * hd * 2,
                  make_attn, run_attn, 2)
    # the fused kernel at the head dims it takes (the same operands as [B, H, S, D])
    for hd in (32, 64, 128):
        cases.add("attention_headdim%d_batch8_seq512" % hd, "bf16", "mfma", 4.0 * 96 * 512 * 512 * hd, 4 * 96 * 512 * hd * 2,
                  lambda hd=hd: tuple(_uniform((8, 12, 512, hd), bf, gen, device) for _ in range(3)) +
                  (torch.empty((8, 12, 512, hd), dtype=bf, device=device),),
                  lambda q, k, v, o, hd=hd: ops.attention(q, k, v, None, hd ** -0.5, out=o, defer=True), 2)
    cases.add("conv7x7_stem_3to64_224", "f32", "mfma", 2.0 * 16 * 112 * 112 * 64 * 147, (16 * 3 * 224 * 224 + 64 * 147 + 16 * 64 * 112 * 112) * 4,
              lambda: (_uniform((16, 3, 224, 224), torch.float32, gen, device), _uniform((64, 3, 7, 7), torch.float32, gen, device) * 0.05,
                       torch.empty((16, 64, 112, 112), dtype=torch.float32, device=device)),
              lambda x, w, o: ops.conv2d(x, w, pad=(3, 3, 3, 3), stride=(2, 2), out=o, defer=True), 2)
    # the same layer as the bf16 network runs it: NCHW operands, the result channels-last for the layers behind it
    cases.add("conv7x7_stem_3to64_224_channels_last_result", "bf16", "mfma", 2.0 * 16 * 112 * 112 * 64 * 147,
              (16 * 3 * 224 * 224 + 64 * 147 + 16 * 64 * 112 * 112) * 2,
              lambda: (_uniform((16, 3, 224, 224), bf, gen, device), _uniform((64, 3, 7, 7), bf, gen, device) * 0.05,
                       torch.empty((16, 64, 112, 112), dtype=bf, device=device).contiguous(memory_format=torch.channels_last)),
              lambda x, w, o: ops.conv2d(x, w, pad=(3, 3, 3, 3), stride=(2, 2), out=o, defer=True), 2)
    return cases


def time_gpu(fn, steps, warmup):
    """Average milliseconds per call of fn(i), HIP events on the stream the kernels are launched on."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn(warmup + i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def launch_spread_us(fn, n=100):
    """p10 / median / p90 of single launches in microseconds, each between its own pair of events with the device
    idle before it: what one isolated call costs, launch latency included (the averages above are of launches
    issued back to back, where that latency is hidden behind the previous kernel)."""
    times = []
    for i in range(n):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        fn(i)
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b) * 1e3)
    times.sort()
    return {"p10": round(times[n // 10], 2), "median": round(times[n // 2], 2), "p90": round(times[(9 * n) // 10], 2)}


_COPY_FLOOR = {}


def copy_floor_us(ops, device, nbytes):
    """Microseconds a plain streaming kernel (one fp32 tensor in, relu, one out; 16 bytes per lane, the suite's own
    elementwise kernel) takes to move `nbytes` in total, half read and half written, on rotating operand sets like
    the cases themselves: what the memory system of this box delivers at that size, launch and ramp-up included.
    The HBM-bound rows are reported against it next to the published 8 TB/s."""
    n = max(1024, int(nbytes // 8) // 1024 * 1024)
    if n not in _COPY_FLOOR:
        sets = max(2, int(1.2e9 // (8 * n)))
        prog = ops.make_program([("relu", "r0", "in0")], "r0")
        xs = [torch.zeros(n, dtype=torch.float32, device=device) for _ in range(sets)]
        outs = [torch.empty(n, dtype=torch.float32, device=device) for _ in range(sets)]
        calls = [ops.elementwise(prog, [x], (n,), torch.float32, out=o, defer=True) for x, o in zip(xs, outs)]
        _COPY_FLOOR[n] = time_gpu(lambda i: calls[i % sets].launch(), 100, 20) * 1e3
        del xs, outs, calls
    return _COPY_FLOOR[n]


def measured_traffic():
    """HBM bytes per launch (reads + writes) of each case's kernel, read from the table in
    profiles/single_op_suite_hbm_counters.md: two rocprofv3 counter runs over this same workload (FETCH_SIZE and
    WRITE_SIZE, each scaled by what a plain copy of known size reads; the file holds the commands).  Counters
    cannot be read from inside a timed run; a case the table does not list reports null."""
    path = os.path.join(ROOT, "profiles", "single_op_suite_hbm_counters.md")
    table = {}
    try:
        for line in open(path):
            parts = line.split()
            # case name first, then the kernel's name, then five numbers: read, write, total, algorithmic MB, ratio
            if len(parts) >= 7 and parts[0].count("_") >= 1:
                try:
                    nums = [float(x) for x in parts[-5:]]
                except ValueError:
                    continue
                table[parts[0]] = int(round(nums[2] * 1e6))
    except OSError:
        pass
    return table


MEASURED_TRAFFIC_BYTES = measured_traffic()


def roofline_of(case, ms):
    if case.bound == "mfma":
        achieved = case.flops / (ms * 1e-3) / 1e12
        peak = PEAK_MFMA_TFLOPS[case.dtype_name]
        unit = "TFLOP/s"
    else:
        achieved = case.bytes / (ms * 1e-3) / 1e9
        peak = PEAK_HBM_GBS
        unit = "GB/s"
    name = "%s_%s" % (case.name, case.dtype_name)
    return {"kernel": name, "bound": case.bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(name), "avg_ms": round(ms, 5)}


def cpu_baseline():
    """The CPU oracle (the reference's loop nests restated in C, one thread) on a bounded sample of
    each fp32 op of the suite, extrapolated linearly to the full op; about 10-30 s of CPU work."""
    from oracle import ref
    r = np.random.default_rng(0)
    parts = {}

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    a = r.uniform(-1, 1, (256, 2048)).astype(np.float32)
    b = r.uniform(-1, 1, (2048, 2048)).astype(np.float32)
    parts["matmul"] = timed(lambda: ref.matmul(a, b, "mnk")) * (2048 / 256)
    a3 = r.uniform(-1, 1, (4, 512, 64)).astype(np.float32)
    b3 = r.uniform(-1, 1, (4, 64, 512)).astype(np.float32)
    parts["batch_matmul"] = timed(lambda: ref.batch_matmul(a3, b3, "mnk")) * (32 / 4)
    x = r.uniform(-1, 1, (8, 1024, 1024)).astype(np.float32)
    y = r.uniform(-1, 1, (8, 1024, 1024)).astype(np.float32)
    parts["add_relu"] = timed(lambda: ref.unary("relu", ref.binary("add", x, y))) * (64 / 8)
    s = r.uniform(-1, 1, (1024, 4096)).astype(np.float32)
    parts["softmax"] = timed(lambda: ref.softmax_lastdim(s)) * (4096 / 1024)
    l = r.uniform(-1, 1, (2048, 1024)).astype(np.float32)
    g = np.ones(1024, np.float32)
    parts["layernorm"] = timed(lambda: ref.layernorm_lastdim(l, g, np.zeros(1024, np.float32))) * (8192 / 2048)
    total_ms = sum(parts.values()) * 1e3
    # the same five fp32 ops, full size, in torch eager on all host threads: what the reference checks its
    # results against and runs the nodes it does not compile with (one pass each after one warm-up pass)
    eager = {}
    ta, tb = torch.from_numpy(r.uniform(-1, 1, (2048, 2048)).astype(np.float32)), torch.from_numpy(b)
    t3a = torch.from_numpy(r.uniform(-1, 1, (32, 512, 64)).astype(np.float32))
    t3b = torch.from_numpy(r.uniform(-1, 1, (32, 64, 512)).astype(np.float32))
    tx = torch.from_numpy(r.uniform(-1, 1, (64, 1024, 1024)).astype(np.float32))
    ts = torch.from_numpy(r.uniform(-1, 1, (4096, 4096)).astype(np.float32))
    tl = torch.from_numpy(r.uniform(-1, 1, (8192, 1024)).astype(np.float32))
    for name, fn in (("matmul", lambda: ta @ tb), ("batch_matmul", lambda: torch.bmm(t3a, t3b)),
                     ("add_relu", lambda: torch.relu(tx + tx)), ("softmax", lambda: torch.softmax(ts, -1)),
                     ("layernorm", lambda: torch.nn.functional.layer_norm(tl, (1024,)))):
        fn()
        eager[name] = timed(fn)
    return {"value": round(total_ms, 1), "unit": "ms", "cores": 1, "kind": "port",
            "sample": "fp32 half of the suite on the C oracle, 1 thread: matmul 256 of 2048 rows, batch_matmul 4 of 32 "
                      "batches, add+relu 8 of 64 slabs, softmax 1024 of 4096 rows, layernorm 2048 of 8192 rows; each "
                      "extrapolated linearly and summed (the bf16 half has no CPU path in the reference)",
            "per_op_ms": {k: round(v * 1e3, 1) for k, v in parts.items()},
            "torch_cpu_eager": {"value": round(sum(eager.values()) * 1e3, 2), "unit": "ms", "threads": torch.get_num_threads(),
                                "per_op_ms": {k: round(v * 1e3, 2) for k, v in eager.items()}}}


MODELS = ("mlp", "resnet18", "encoder", "bert")

# algorithmic flops per forward pass of each configuration (multiply-adds counted as two): the contractions only
FLOP_MLP = 2.0 * 4 * (784 * 512 + 512 * 10)
FLOP_RESNET18_B16 = 58.0e9 + 16.4e6
FLOP_ENCODER_PER_SAMPLE = 8.05e9


def flop_bert(seq, batch=8, layers=12, hidden=768):
    return layers * batch * seq * (14.16e6 + 4.0 * seq * hidden)


def _call_times_ms(f, n, warmup):
    """Time per call of f(), calls issued back to back, host dispatch included in what the device sees: HIP events on
    the stream the kernels are launched on (torch's current stream) around GROUPS of calls, each group's time divided
    by its size.  Recording an event costs 4 us of host time on this platform, which a call of 10 us (the MLP: two
    kernels, host-bound) would be charged with if every call had an event pair of its own; groups are sized so that one
    lasts about 200 us (one call per group from 0.2 ms per call upwards)."""
    for _ in range(warmup):
        f()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(5):
        f()
    b.record()
    torch.cuda.synchronize()
    group = max(1, min(32, int(0.2 / max(a.elapsed_time(b) / 5, 1e-4))))
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
    evs[0].record()
    for i in range(n):
        for _ in range(group):
            f()
        evs[i + 1].record()
    torch.cuda.synchronize()
    return sorted(evs[i].elapsed_time(evs[i + 1]) / group for i in range(n))


def _stats(times, flops, dtype_name):
    n = len(times)
    med = times[n // 2]
    tf = flops / (med * 1e-3) / 1e12
    return {"median_ms": round(med, 4), "p10_ms": round(times[n // 10], 4), "p90_ms": round(times[(9 * n) // 10], 4), "calls": n,
            "gflop": round(flops / 1e9, 3), "achieved_tflops": round(tf, 2), "peak_tflops": PEAK_MFMA_TFLOPS[dtype_name],
            "frac_of_peak": round(tf / PEAK_MFMA_TFLOPS[dtype_name], 4), "dtype": dtype_name}


def model_latencies(which=MODELS, calls=100):
    """End-to-end latency per batch of the other four configurations (whole compiled graphs through the executor,
    inputs resident on the GPU): an MLP, ResNet-18 with folded batch norm, a bf16 encoder block compiled once with a
    symbolic batch, and a 12-layer BERT-base shaped encoder compiled once with a symbolic sequence length.  Median, p10
    and p90 over `calls` event-timed calls each, and the achieved TFLOP/s against the peak of the type the contractions
    run in.  Reported next to the suite, not part of `value`.  `which` selects a subset."""
    import warnings
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.test_models import (MLP, BertEncoder, EncoderBlock, ResNet18BN, ResNet18Folded, make_bert_inputs,
                                            make_encoder_inputs, make_mlp_inputs, make_resnet_inputs)
    warnings.filterwarnings("ignore")
    res = {}
    with torch.no_grad():
        if "mlp" in which:
            x = make_mlp_inputs()[0].cuda()
            cm = compile_module(MLP().cuda(), (x,))
            res["mlp_f32_batch4"] = _stats(_call_times_ms(lambda: cm(x), max(calls, 200), 20), FLOP_MLP, "f32")
        if "resnet18" in which:
            xs = make_resnet_inputs(16, 224)[0].cuda()
            cr = compile_module(ResNet18Folded().cuda(), (xs,))
            res["resnet18_f32_batch16"] = _stats(_call_times_ms(lambda: cr(xs), calls, 3), FLOP_RESNET18_B16, "f32")
            # the network as torchvision spells it (Conv2d without bias -> BatchNorm2d, eval mode, randomised statistics):
            # the batch norms are folded into the filters when the plan is made, a call launches the same kernels
            cn = compile_module(ResNet18BN().cuda(), (xs,))
            res["resnet18_batchnorm_f32_batch16"] = _stats(_call_times_ms(lambda: cn(xs), calls, 3), FLOP_RESNET18_B16, "f32")
            # the same network in bf16 storage (not one of the five configurations: its convolutions run on the
            # bf16 matrix instructions, which the fp32 configuration cannot show)
            xh = xs.to(torch.bfloat16)
            ch = compile_module(ResNet18Folded().to(torch.bfloat16).cuda(), (xh,))
            res["resnet18_bf16_batch16"] = _stats(_call_times_ms(lambda: ch(xh), calls, 3), FLOP_RESNET18_B16, "bf16")
        if "encoder" in which:
            xe = make_encoder_inputs(8, 512)[0].to(torch.bfloat16).cuda()
            ce = compile_module(EncoderBlock().to(torch.bfloat16).cuda(), (xe,),
                                dynamic_shapes=({0: torch.export.Dim("batch")},))
            for b in (1, 8, 32):
                xb = make_encoder_inputs(b, 512, seed=b)[0].to(torch.bfloat16).cuda()
                res["encoder_block_bf16_seq512_batch%d" % b] = _stats(_call_times_ms(lambda: ce(xb), calls, 5),
                                                                      FLOP_ENCODER_PER_SAMPLE * b, "bf16")
        if "bert" in which:
            cb = compile_module(BertEncoder().cuda(), tuple(t.cuda() for t in make_bert_inputs(8, 128)),
                                dynamic_shapes=({1: torch.export.Dim("seq")}, {3: torch.export.Dim("seq")}))
            for sl in (128, 256, 512):
                xi, mi = (t.cuda() for t in make_bert_inputs(8, sl, seed=sl))
                res["bert_base_f32_batch8_seq%d" % sl] = _stats(_call_times_ms(lambda: cb(xi, mi), calls, 2), flop_bert(sl), "f32")
    return res


def cpu_model_baselines(which=MODELS):
    """The two CPU stand-ins for the model configurations, on this host: torch eager on all host threads, one timed
    forward pass each after one warm-up pass (what the reference asserts equality with and falls back to), and the
    C oracle (one thread, the reference's generated loop nests restated) on a sample whose rate is extrapolated by
    flops to the whole pass."""
    import warnings
    from oracle import ref
    from llcompiler_amd.test_models import (MLP, BertEncoder, EncoderBlock, ResNet18Folded, make_bert_inputs,
                                            make_encoder_inputs, make_mlp_inputs, make_resnet_inputs)
    warnings.filterwarnings("ignore")

    def once(f):
        f()
        t0 = time.perf_counter()
        f()
        return round((time.perf_counter() - t0) * 1e3, 2)

    eager, port = {}, {}
    r = np.random.default_rng(1)
    # oracle rates on samples: a Linear layer of the transformer configurations, one 3x3 body convolution and the stem
    # of one image of the ResNet
    a = r.uniform(-1, 1, (256, 768)).astype(np.float32)
    w = r.uniform(-1, 1, (768, 768)).astype(np.float32)
    t0 = time.perf_counter()
    ref.matmul(a, w, "mnk")
    linear_rate = 2.0 * 256 * 768 * 768 / (time.perf_counter() - t0)
    xc = r.standard_normal((1, 64, 56, 56)).astype(np.float32)
    wc = r.standard_normal((64, 64, 3, 3)).astype(np.float32)
    t0 = time.perf_counter()
    ref.conv2d(xc, wc, None, (1, 1, 1, 1))
    conv_rate = 2.0 * 56 * 56 * 64 * 64 * 9 / (time.perf_counter() - t0)
    sample = ("C oracle, 1 thread: a [256,768]x[768,768] matmul (%.2f GFLOP/s) stands for the Linear layers and attention "
              "products, a 64->64 3x3 convolution of one 56x56 image (%.2f GFLOP/s) for the convolutions; each pass is its "
              "flops divided by that rate" % (linear_rate / 1e9, conv_rate / 1e9))
    with torch.no_grad():
        if "mlp" in which:
            m, x = MLP().eval(), make_mlp_inputs()[0]
            eager["mlp_f32_batch4"] = once(lambda: m(x))
            port["mlp_f32_batch4"] = round(FLOP_MLP / linear_rate * 1e3, 3)
        if "resnet18" in which:
            m, x = ResNet18Folded().eval(), make_resnet_inputs(16, 224)[0]
            eager["resnet18_f32_batch16"] = once(lambda: m(x))
            port["resnet18_f32_batch16"] = round(FLOP_RESNET18_B16 / conv_rate * 1e3, 1)
        if "encoder" in which:
            m = EncoderBlock().to(torch.bfloat16).eval()
            for b in (1, 8, 32):
                x = make_encoder_inputs(b, 512, seed=b)[0].to(torch.bfloat16)
                eager["encoder_block_bf16_seq512_batch%d" % b] = once(lambda: m(x))
                port["encoder_block_bf16_seq512_batch%d" % b] = round(FLOP_ENCODER_PER_SAMPLE * b / linear_rate * 1e3, 1)
        if "bert" in which:
            m = BertEncoder().eval()
            for sl in (128, 256, 512):
                xi, mi = make_bert_inputs(8, sl, seed=sl)
                eager["bert_base_f32_batch8_seq%d" % sl] = once(lambda: m(xi, mi))
                port["bert_base_f32_batch8_seq%d" % sl] = round(flop_bert(sl) / linear_rate * 1e3, 1)
    return {"torch_cpu_eager_ms": eager, "threads": torch.get_num_threads(), "c_oracle_extrapolated_ms": port, "cores": 1,
            "sample": sample}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-models", action="store_true", help="skip the end-to-end latencies of the model configurations")
    ap.add_argument("--no-extra", action="store_true", help="skip the contraction rows outside the suite (extra_kernels)")
    ap.add_argument("--models", default="", help="comma-separated subset of %s whose end-to-end latencies to "
                    "measure (default: all of them, or none when --only is given)" % ",".join(MODELS))
    ap.add_argument("--only", default="", help="comma-separated kernel names (e.g. matmul_bf16,softmax_f32): run just "
                    "these cases, for profiling one kernel at a time (`all` = the whole suite, `copy_f32` adds the "
                    "counter calibration copy); the JSON line then describes that subset")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus)
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU; there is no CPU fallback")
    from llcompiler_amd import ops
    device = torch.device("cuda", 0)
    only = [n for n in args.only.split(",") if n]
    models = tuple(n for n in args.models.split(",") if n) or (() if only else MODELS)
    if set(models) - set(MODELS):
        sys.exit("--models takes names from %s" % ",".join(MODELS))
    cases = build_cases(ops, device, only)

    def step(i):
        for c in cases:
            c.run(i)

    torch.cuda.synchronize()
    ms_per_step = time_gpu(step, args.steps, args.warmup)
    # per-kernel average durations, each in its own timed loop of at least 100 launches after 20 untimed ones:
    # a few milliseconds of work after an idle period run below the sustained clocks (the fp32 matmul reads 155 us
    # over 20 launches and 134 us over 100)
    kernels = [roofline_of(c, time_gpu(c.run, max(args.steps, 100), max(args.warmup, 20))) for c in cases]
    for c, k in zip(cases, kernels):
        k["single_launch_us"] = launch_spread_us(c.run)
        if c.bound == "hbm":
            k["copy_same_bytes_us"] = round(copy_floor_us(ops, device, c.bytes), 2)
            k["frac_of_copy"] = round(k["copy_same_bytes_us"] / (k["avg_ms"] * 1e3), 3)
    extra_rows = []
    if not args.no_extra:
        # with --only, the rows outside the suite that it names (for counter runs on one of them)
        extra = build_extra_cases(ops, device, only)
        extra_rows = [roofline_of(c, time_gpu(c.run, 50, 10)) for c in extra]
        del extra
        torch.cuda.empty_cache()
    if not kernels and not extra_rows:
        raise SystemExit("bench.py: --only %s selects no case (with --no-extra only the single-op suite's names count)" % args.only)
    dominant = max(kernels or extra_rows, key=lambda k: k["avg_ms"])
    out = {
        "metric": "end-to-end latency ms/batch", "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32+bf16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": WORKLOAD if not only else "subset for profiling: " + ",".join(only), "values": "U(-1,1), seed 0",
                   "ops_per_step": len(cases)},
        "roofline": {k: dominant[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")},
        "dominant_kernel": dominant["kernel"],
        "kernels": kernels,
    }
    if extra_rows:
        out["extra_kernels"] = extra_rows
    # `roofline` describes the kernel that takes the largest share of the pass (the fp32 matmul, measured against the
    # fp32 matrix peak).  The rows the throughput targets are written for, side by side: contractions on the bf16
    # matrix instructions against 2.5 PFLOP/s (target 0.50) and the bandwidth-bound kernels against 8 TB/s (target 0.70).
    rows = kernels + extra_rows
    out["target_rows"] = {
        "mfma_bf16_frac_of_2500_tflops": {k["kernel"]: k["frac"] for k in rows if k["bound"] == "mfma" and k["kernel"].endswith("bf16")},
        "hbm_frac_of_8000_gbs": {k["kernel"]: k["frac"] for k in rows if k["bound"] == "hbm"},
    }
    if not args.no_models and models:
        try:
            configs = model_latencies(models)
            out["model_configs"] = configs
            out["model_latency_ms"] = {k + "_ms": v["median_ms"] for k, v in configs.items()}
        except Exception as e:  # the suite's line is still worth printing
            out["model_latency_ms"] = {"error": "%s: %s" % (type(e).__name__, e)}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        if not args.no_models and models:
            try:
                out["cpu_baseline"]["model_configs"] = cpu_model_baselines(models)
            except Exception as e:
                out["cpu_baseline"]["model_configs"] = {"error": "%s: %s" % (type(e).__name__, e)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
