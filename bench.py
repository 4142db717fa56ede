"""Throughput of the quantized-matmul hot path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints one JSON line.  A step
is one Q4_K GEMV, y[17408] = W[17408, 5120] . x[5120] with fp32 activations (the
FFN gate/up projection of a 27B-class decode layer).  Twelve distinct copies of
the weight matrix (600 MB) are visited in turn so every step streams its 50 MB
from HBM rather than from the 256 MB last-level cache.  The K steps are
recorded once into a HIP graph and replayed, so the timed region holds kernel
launches only; HIP events on the library's own stream bracket it.

``value`` is algorithmic bytes per step / time per step.  ``roofline`` prices the
GEMV kernel against the 8 TB/s HBM peak; its ``traffic`` is read from the HBM
counter summary under ``profiles/`` when that summary was taken from the kernel
sources as they are now, and is null otherwise.  ``cases`` carries the other
shapes of the dense-decode, Q6_K, small-M / prefill GEMM and MoE workloads
(GB/s and TFLOP/s against both peaks).  ``cpu_baseline`` is the CPU oracle on
the host's cores over a bounded sample: the sequential-fp32 GEMV beside the
metric, dequantize-once + blocked sgemm beside ``gemm_m512``, and the routed
FFN chain beside the two MoE cases.

``--cases read`` times a plain 128-bit read of the same rotating matrices (the
HBM rate a kernel gets that does nothing with the bytes) and ``--cases mfma``
times MFMA issue loops from registers (the matrix-core rate per instruction
shape); ``--cases copy`` launches a row copy of known size, the calibration of
the HBM counters.
"""
from __future__ import annotations

import argparse
import glob
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA, published
Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS = 8, 12, 13, 14, 23
BLOCK_BYTES = {Q8_0: 272, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ4_XS: 136}    # per 256 weights
ROTATE_BYTES = 600 << 20     # distinct weight bytes visited before a buffer repeats

CSRC = os.path.join(ROOT, "ferrum_amd", "csrc")
GEMV_SOURCES = ("gemv_stream.hip", "gemv.hip", "device_utils.hpp", "lds_direct.hpp")
GEMM_SOURCES = ("gemm.hip", "tile_decode.hpp", "device_utils.hpp")


def sources_digest(names):
    """First 16 hex digits of the SHA-256 over the named kernel sources, in order."""
    h = hashlib.sha256()
    for name in names:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload_key, names):
    """HBM bytes per launch from the counter summaries under profiles/: a line
    `traffic: workload=<key> sources=<digest> bytes=<n>` counts only while the
    digest equals that of the kernel sources here, so a figure taken from an
    older kernel is never reported for a newer one."""
    digest = sources_digest(names)
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*hbm_counters.txt"))):
        with open(path) as f:
            for text in f:
                if not text.startswith("traffic:"):
                    continue
                fields = dict(part.split("=", 1) for part in text.split()[1:] if "=" in part)
                if fields.get("workload") == workload_key and fields.get("sources") == digest:
                    return int(fields["bytes"])
    return None


def host_info():
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for text in f:
                if text.lower().startswith("model name"):
                    model = text.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu_model": model, "cpu_count": os.cpu_count()}


def algorithmic_bytes(ggml, n, k, m, x_size, y_size):
    return n * (k // 256) * BLOCK_BYTES[ggml] + m * k * x_size + m * n * y_size


class Case:
    """One projection shape with its rotating weight copies resident in HBM."""

    def __init__(self, api, synth, dev, ggml, n, k, m, x_dtype, label, copies=None):
        self.api, self.dev = api, dev
        self.ggml, self.n, self.k, self.m, self.label = ggml, n, k, m, label
        wbytes = n * (k // 256) * BLOCK_BYTES[ggml]
        if copies is None:
            copies = max(2, -(-ROTATE_BYTES // wbytes))
        base = synth.matrix(ggml, n, k, seed=1).reshape(n, -1)
        self.packed = base
        fmt = api.QuantizationFormat.from_ggml_type(ggml)
        self.weights = [
            api.QuantizedMatrix.from_bytes(dev, n, k, fmt, np.roll(base, i, axis=0).reshape(-1))
            for i in range(copies)
        ]
        half = x_dtype != api.DType.F32
        self.x_host = synth.activations(m, k, seed=3, f16=half)
        self.x = api.Tensor.from_f32(dev, (m, k), x_dtype, self.x_host)
        self.y = api.Tensor.zeros(dev, (m, n), api.DType.F32)
        self.bytes = algorithmic_bytes(ggml, n, k, m, x_dtype.size_bytes(), 4)
        self.weight_bytes = wbytes
        self.flops = 2 * m * n * k
        self.operation = ""

    def enqueue(self, i):
        self.dev.project_quantized(self.x, self.weights[i % len(self.weights)], out=self.y)


EAGER = False   # --eager: launch step by step instead of replaying a recording (for profilers)


def run_graph(dev, enqueue, steps, warmup):
    """Replays `steps` recorded launches; returns (wall seconds, event seconds)."""
    for i in range(max(warmup, 1)):
        enqueue(i)
    dev.synchronize()
    if EAGER:
        start, stop = dev.event(), dev.event()
        t0 = time.perf_counter()
        start.record()
        for i in range(steps):
            enqueue(i)
        stop.record()
        dev.synchronize()
        return time.perf_counter() - t0, start.elapsed_ms(stop) * 1e-3
    with dev.execution() as ex:
        for i in range(steps):
            enqueue(i)
    graph = ex.graph
    start, stop = dev.event(), dev.event()
    start.record()
    graph.launch()  # first replay uploads the graph; untimed
    stop.record()
    dev.synchronize()
    first = max(start.elapsed_ms(stop) * 1e-3, 1e-6)
    # A short recording (the driver's --steps 20 is a quarter of a millisecond) would otherwise be timed on a
    # device that has just been idle: a burst of untimed replays of about 4 ms comes first, then several timed
    # replays, each exactly `steps` steps between two synchronizations, of which the median wall time is reported.
    # The events around one such replay also see the latency of the graph launch itself (about 20 us between
    # the start event and the first kernel of an idle stream, a microsecond per launch of a 20-launch
    # recording, nothing of a 2400-launch one), which is not kernel time: the kernels' duration is taken from
    # one more region in which the same recording is replayed back to back, so that every launch but the
    # first is queued while the device is busy, divided by the number of replays.
    short = first < 2e-3
    if short:
        for _ in range(min(400, int(4e-3 / first) + 1)):
            graph.launch()
        dev.synchronize()
    walls, events = [], []
    for _ in range(7 if short else 1):
        t0 = time.perf_counter()
        start.record()
        graph.launch()
        stop.record()
        dev.synchronize()
        walls.append(time.perf_counter() - t0)
        events.append(start.elapsed_ms(stop) * 1e-3)
    walls.sort()
    events.sort()
    event = events[len(events) // 2]
    if short:
        replays = min(64, int(3e-3 / first) + 2)
        start.record()
        for _ in range(replays):
            graph.launch()
        stop.record()
        dev.synchronize()
        event = start.elapsed_ms(stop) * 1e-3 / replays
    return walls[len(walls) // 2], event


def measure(dev, case, steps, warmup, repeats=3):
    best_wall, best_event = float("inf"), float("inf")
    for _ in range(repeats):
        wall, event = run_graph(dev, case.enqueue, steps, warmup)
        best_wall, best_event = min(best_wall, wall), min(best_event, event)
    case.operation = dev.last_operation()
    return best_wall, best_event


def report(case, seconds_per_step):
    gbs = case.bytes / seconds_per_step / 1e9
    tf = case.flops / seconds_per_step / 1e12
    return {
        "workload": case.label,
        "operation": case.operation,
        "us": round(seconds_per_step * 1e6, 3),
        "GB/s": round(gbs, 1),
        "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
        "TFLOP/s": round(tf, 2),
        "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
        "weight_copies": len(case.weights),
        "rotated_bytes": len(case.weights) * case.weight_bytes,
    }


def host_threads():
    return max(1, min(16, os.cpu_count() or 1))


def _repeat(fn, budget_seconds, limit=20000):
    fn()   # page in
    runs, spent = 0, 0.0
    while spent < budget_seconds and runs < limit:
        t0 = time.perf_counter()
        fn()
        spent += time.perf_counter() - t0
        runs += 1
    return runs, spent / runs


def cpu_baseline(case, budget_seconds=8.0):
    """The CPU oracle's sequential-fp32 GEMV on the same tensors: all host threads
    (`value`) and one thread."""
    import oracle
    threads = host_threads()
    packed = case.packed.reshape(-1)
    x = case.x_host
    runs, per = _repeat(lambda: oracle.project(case.ggml, packed, case.n, case.k, x, threads=threads), budget_seconds)
    runs1, per1 = _repeat(lambda: oracle.project(case.ggml, packed, case.n, case.k, x, threads=1), 4.0)
    return {
        "value": round(case.bytes / per / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{runs} repeats of the same {case.label} step ({per * 1e3:.1f} ms each), "
                  f"dequant + sequential fp32 dot, rows split over {threads} threads",
        "one_thread": {"value": round(case.bytes / per1 / 1e9, 3), "unit": "GB/s", "cores": 1,
                       "sample": f"{runs1} repeats ({per1 * 1e3:.1f} ms each)"},
    }


def cpu_baseline_gemm(case, sample_columns=1024):
    """CPU figures for the prefill GEMM on the same tensors.  `value`: every
    weight dequantized once by the oracle, then numpy's blocked sgemm over the
    whole [M,K] x [K,N] product.  `oracle_sequential`: the oracle's own product
    (each row dequantized once, then M sequential-fp32 dots) on a sample of the
    output columns."""
    import oracle
    threads = host_threads()
    blas_threads = None
    try:
        from threadpoolctl import threadpool_info
        blas = [p.get("num_threads") for p in threadpool_info() if p.get("user_api") == "blas"]
        blas_threads = blas[0] if blas else None
    except Exception:
        pass
    x = np.ascontiguousarray(case.x_host, dtype=np.float32).reshape(case.m, case.k)
    t0 = time.perf_counter()
    w = oracle.dequantize(case.ggml, case.packed.reshape(-1), case.n, case.k)
    t_dequant = time.perf_counter() - t0
    t0 = time.perf_counter()
    y = x @ w.T
    t_gemm = time.perf_counter() - t0
    del w, y
    total = t_dequant + t_gemm
    cols = np.linspace(0, case.n - 1, sample_columns).astype(np.int64)
    sub = np.ascontiguousarray(case.packed[cols]).reshape(-1)
    t0 = time.perf_counter()
    oracle.project(case.ggml, sub, len(cols), case.k, x, threads=threads)
    t_seq = time.perf_counter() - t0
    t0 = time.perf_counter()
    few = cols[: max(1, sample_columns // 8)]
    oracle.project(case.ggml, np.ascontiguousarray(case.packed[few]).reshape(-1), len(few), case.k, x, threads=1)
    t_seq1 = time.perf_counter() - t0
    return {
        "value": round(case.flops / total / 1e9, 1),
        "unit": "GFLOP/s",
        "cores": blas_threads or threads,
        "kind": "port",
        "sample": f"one whole {case.label} product: oracle dequantize of all {case.n}x{case.k} weights on one thread "
                  f"({t_dequant:.2f} s) + numpy sgemm on {blas_threads or '?'} BLAS threads ({t_gemm:.2f} s)",
        "sgemm_alone": {"value": round(case.flops / t_gemm / 1e9, 1), "unit": "GFLOP/s"},
        "oracle_sequential": {
            "value": round(2.0 * case.m * len(cols) * case.k / t_seq / 1e9, 2), "unit": "GFLOP/s", "cores": threads,
            "sample": f"{len(cols)} of {case.n} output columns, all {case.m} rows ({t_seq:.2f} s), "
                      f"row dequantized once then sequential fp32 dots",
            "one_thread": {"value": round(2.0 * case.m * len(few) * case.k / t_seq1 / 1e9, 2), "unit": "GFLOP/s",
                           "cores": 1, "sample": f"{len(few)} columns ({t_seq1:.2f} s)"},
        },
    }


def gemm_distance(api, dev, case, sample_columns=96):
    """How far the tile GEMM's output is from the oracle on a sample of columns:
    against the product with weights rounded to f16 first (what the tiles multiply)
    and against the unrounded product, both accumulated in f64."""
    import oracle
    dev.project_quantized(case.x, case.weights[0], out=case.y)
    dev.synchronize()
    got = case.y.to_f32().reshape(case.m, case.n)
    cols = np.unique(np.concatenate([np.linspace(0, case.n - 1, sample_columns).astype(np.int64),
                                     np.arange(case.n - 8, case.n)]))
    sub = np.ascontiguousarray(case.packed[cols]).reshape(-1)
    x = np.ascontiguousarray(case.x_host, dtype=np.float32).reshape(case.m, case.k)
    out = {}
    for name, rounding in (("tile_rounded_oracle", oracle.F16), ("unrounded_oracle", 0)):
        want = oracle.project(case.ggml, sub, len(cols), case.k, x, accumulate="f64", weight_round=rounding,
                              threads=host_threads()).astype(np.float64)
        diff = got[:, cols].astype(np.float64) - want
        floor = float(np.sqrt(np.mean(want * want)))
        out[name] = {"rel_l2": float(np.linalg.norm(diff) / np.linalg.norm(want)),
                     "max_rel": float(np.max(np.abs(diff) / np.maximum(np.abs(want), floor)))}
    out["sample"] = f"{len(cols)} of {case.n} columns, all {case.m} rows; max_rel = |err| / max(|ref|, rms(ref))"
    return out


def layer_case(api, synth, dev, steps, layers=4):
    """One dense decode layer's four Q4_K GEMVs back to back (attention
    projection 5120x5120, FFN gate and up 17408x5120, FFN down 5120x17408;
    165 MB), over `layers` distinct sets of weights so nothing is cache resident."""
    fmt = api.QuantizationFormat.Q4_K
    f32 = api.DType.F32
    shapes = [(5120, 5120), (17408, 5120), (17408, 5120), (5120, 17408)]
    bases = {shape: synth.matrix(Q4_K, shape[0], shape[1], seed=21).reshape(shape[0], -1) for shape in set(shapes)}
    sets = []
    for layer in range(layers):
        sets.append([api.QuantizedMatrix.from_bytes(dev, n, k, fmt, np.roll(bases[(n, k)], 4 * layer + i, axis=0).reshape(-1))
                     for i, (n, k) in enumerate(shapes)])
    x5 = api.Tensor.from_f32(dev, (1, 5120), f32, synth.activations(1, 5120, seed=22))
    x17 = api.Tensor.from_f32(dev, (1, 17408), f32, synth.activations(1, 17408, seed=23))
    outs = [api.Tensor.zeros(dev, (1, n), f32) for n, _ in shapes]

    def enqueue(i):
        mats = sets[i % layers]
        dev.project_quantized(x5, mats[0], out=outs[0])
        dev.project_quantized(x5, mats[1], out=outs[1])
        dev.project_quantized(x5, mats[2], out=outs[2])
        dev.project_quantized(x17, mats[3], out=outs[3])

    best = min(run_graph(dev, enqueue, steps, layers)[1] for _ in range(2)) / steps
    nbytes = sum(algorithmic_bytes(Q4_K, n, k, 1, 4, 4) for n, k in shapes)
    flops = sum(2 * n * k for n, k in shapes)
    return {
        "workload": "Q4_K decode layer: attn 5120x5120 + gate/up 2 x (17408x5120) + down 5120x17408, M=1",
        "operation": "4 x q4_k_gemv",
        "us": round(best * 1e6, 2),
        "GB/s": round(nbytes / best / 1e9, 1),
        "frac_hbm": round(nbytes / best / 1e9 / HBM_PEAK_GBS, 4),
        "TFLOP/s": round(flops / best / 1e12, 2),
        "frac_mfma_f16": round(flops / best / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
        "weight_copies": layers,
    }


def moe_case(api, synth, dev, tokens, steps, cpu=True):
    """A3B-style routed FFN: hidden 2048, 256 experts x intermediate 512 in Q4_K,
    top-8 softmax routing with renormalised weights, plus one shared expert
    whose output the combine adds; f16 activations.  One step =
    SparseMoe.forward: route, gate|up, SiLU*up, down and the shared expert's
    two projections, combine.  Distinct router logits per step move the set of
    experts that are hit."""
    hidden, inter, experts, top_k = 2048, 512, 256, 8
    fmt = api.QuantizationFormat.Q4_K
    f16, f32 = api.DType.F16, api.DType.F32
    eight_in = synth.matrix(Q4_K, 8 * 2 * inter, hidden, seed=11).reshape(8, -1)
    eight_out = synth.matrix(Q4_K, 8 * hidden, inter, seed=12).reshape(8, -1)
    packed_in = np.tile(eight_in, (experts // 8, 1)).reshape(-1)
    packed_out = np.tile(eight_out, (experts // 8, 1)).reshape(-1)
    shared_in = synth.matrix(Q4_K, 2 * inter, hidden, seed=13)
    shared_out = synth.matrix(Q4_K, hidden, inter, seed=14)
    win = api.QuantizedExpertMatrix.new(dev, packed_in, fmt, experts, 2 * inter, hidden)
    wout = api.QuantizedExpertMatrix.new(dev, packed_out, fmt, experts, hidden, inter)
    sin = api.QuantizedMatrix.from_bytes(dev, 2 * inter, hidden, fmt, shared_in)
    sout = api.QuantizedMatrix.from_bytes(dev, hidden, inter, fmt, shared_out)
    moe = api.SparseMoe(dev, win, wout, api.MoeRoutingPolicy(experts, top_k), shared_input=sin, shared_output=sout)
    moe.workspace(tokens, f16)
    x_host = synth.activations(tokens, hidden, seed=15, f16=True) * np.float32(2.0 ** -6)
    x = api.Tensor.from_f32(dev, (tokens, hidden), f16, x_host)
    # distinct experts hit over one rotation of the logit sets: all 256 (453 MB) at 512 tokens; for one token
    # 96 sets reach about 95% of them (~430 MB), more than the 256 MB last-level cache
    variants = 16 if tokens >= 64 else 96
    logit_sets, hit, first_logits, touched = [], [], None, set()
    for i in range(variants):
        values = synth.rng(16, i).standard_normal((tokens, experts)).astype(np.float32)
        if first_logits is None:
            first_logits = values
        logit_sets.append(api.Tensor.from_f32(dev, values.shape, f32, values))
        chosen = np.unique(np.argsort(-values, axis=1)[:, :top_k])
        hit.append(len(chosen))
        touched.update(int(e) for e in chosen)
    names = []

    def enqueue(i):
        moe.forward(x, logit_sets[i % variants])
        names.append(dev.last_operation())

    best = min(run_graph(dev, enqueue, steps, 2)[1] for _ in range(2)) / steps
    # The same FFN through fh_moe_ffn (the same bits).  For one token it routes inside the gate|up
    # launch and adds the weighted sum inside the down projection's (two launches); for many it groups
    # the records by expert once for both projections.  The separate calls of SparseMoe.forward are
    # reported beside it.
    out = api.Tensor.zeros(dev, (tokens, hidden), f16)

    def enqueue_one(i):
        moe.forward_in_one_call(x, logit_sets[i % variants], out=out)

    enqueue_one(0)
    dev.synchronize()
    separate = best
    best = min(run_graph(dev, enqueue_one, steps, 2)[1] for _ in range(2)) / steps
    per_expert = (2 * inter * hidden + hidden * inter) // 256 * BLOCK_BYTES[Q4_K]
    mean_hit = float(np.mean(hit))
    act_bytes = tokens * hidden * 2 * 2 + tokens * experts * 4
    nbytes = mean_hit * per_expert + per_expert + act_bytes
    flops = 2 * tokens * (top_k + 1) * (2 * inter * hidden + hidden * inter)
    cpu_line = None
    if cpu:
        # the same step on the CPU oracle, one thread, for a bounded number of the tokens
        import oracle
        sample = min(tokens, 8)
        code = oracle.F16
        xs = oracle.round_storage(x_host.reshape(tokens, hidden)[:sample], code).reshape(sample, hidden)

        def chain():
            meta = oracle.select_routes(first_logits[:sample], experts, top_k)
            up = oracle.round_storage(oracle.expert_project(Q4_K, packed_in, experts, 2 * inter, hidden,
                                                            oracle.expert_assign(xs, meta), meta), code)
            down = oracle.round_storage(oracle.expert_project(Q4_K, packed_out, experts, hidden, inter,
                                                              oracle.expert_silu_mul(up, inter, code), meta), code)
            sup = oracle.round_storage(oracle.project(Q4_K, shared_in, 2 * inter, hidden, xs), code)
            sdown = oracle.round_storage(oracle.project(Q4_K, shared_out, hidden, inter,
                                                        oracle.expert_silu_mul(sup, inter, code)), code)
            return oracle.expert_combine_shared(down, meta, sample, hidden, top_k, sdown, None, dtype=code)

        runs, per = _repeat(chain, 4.0, limit=50)
        per_token = per / sample
        cpu_line = {
            "value": round(flops / tokens / per_token / 1e9, 3), "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "us_per_step": round(per_token * tokens * 1e6, 1),
            "sample": f"{runs} repeats of the oracle chain (route, gate|up, SiLU*up, down, shared expert, combine) "
                      f"over {sample} of the step's {tokens} tokens ({per * 1e3:.1f} ms each), scaled by tokens; "
                      f"every assignment dequantizes its expert's rows, sequential fp32 dots, one thread",
        }
    return {
        "cpu_baseline": cpu_line,
        "workload": f"Q4_K MoE FFN T={tokens} hidden=2048 experts=256 top-8 + shared expert, f16 x",
        "operation": ("fh_moe_ffn: (moe_route + expert_project with the shared expert riding) + (expert_project + combine)"
                      if tokens * top_k <= 31 else
                      "fh_moe_ffn: moe_route + expert_group + 2 x (expert_project grouped, shared expert pieces inside) "
                      "+ silu_mul + combine"),
        "us": round(best * 1e6, 2),
        "us_as_separate_calls": round(separate * 1e6, 2),
        "GB/s": round(nbytes / best / 1e9, 1),
        "frac_hbm": round(nbytes / best / 1e9 / HBM_PEAK_GBS, 4),
        "TFLOP/s": round(flops / best / 1e12, 2),
        "frac_mfma_f16": round(flops / best / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
        "experts_hit_mean": mean_hit,
        "algorithmic_bytes": int(nbytes),
        "rotated_bytes": int((len(touched) + 1) * per_expert),
        "logit_sets": variants,
    }


def copy_calibration(api, dev, rows=65536, width=1024, launches=10):
    """Launches expert_assign with identity routing: a row copy that reads and
    writes rows*width*4 bytes each, the known size the HBM counters are scaled by."""
    hidden = api.Tensor.from_f32(dev, (rows, width), api.DType.F32,
                                 np.arange(rows * width, dtype=np.float32) % 251.0)
    meta = np.zeros((rows, 3), dtype=np.uint32)
    meta[:, 0] = 0
    meta[:, 1] = np.arange(rows, dtype=np.uint32)
    meta[:, 2] = np.float32(1.0).view(np.uint32)
    metadata = api.Tensor.from_bits(dev, (rows, 3), meta)
    out = None
    for _ in range(launches):
        out = dev.expert_assign(hidden, metadata, 1)
    dev.synchronize()
    same = np.array_equal(out.to_f32(), hidden.to_f32())
    print(json.dumps({"copy_kernel": dev.last_operation(), "launches": launches,
                      "read_bytes": rows * width * 4 + rows * 12, "write_bytes": rows * width * 4,
                      "copied_correctly": bool(same)}), flush=True)


READ_FORMS = (0, 25604, 25616, 51204, 51208, 102404, 102408, 1025608, 1025616, 1051208)


def read_probe_case(api, synth, dev, steps, warmup):
    """A kernel that only loads the rotating matrices: (1) every launch shape of the probe on the
    headline's matrices, the best of which is the ceiling a streaming kernel of that size has;
    (2) that shape and the GEMV, back to back, on every GEMV shape of the benchmark."""
    head = Case(api, synth, dev, Q4_K, 17408, 5120, 1, api.DType.F32, "plain 128-bit read of the 17408x5120 Q4_K matrices")
    head.enqueue = lambda i: dev.probe_read(head.weights[i % len(head.weights)])
    sweep = {}
    for form in READ_FORMS:
        dev.set_tuning("probe_read_form", form)
        _, event = measure(dev, head, steps, warmup)
        sweep[head.operation] = round(event / steps * 1e6, 3)
    best_name = min(sweep, key=sweep.get)
    best_form = READ_FORMS[list(sweep).index(best_name)]
    dev.set_tuning("probe_read_form", best_form)
    rows = []
    shapes = ((Q4_K, 4096, 4096), (Q4_K, 5120, 5120), (Q4_K, 17408, 5120), (Q4_K, 5120, 17408),
              (Q6_K, 5120, 17408), (Q6_K, 151936, 5120))
    for ggml, n, k in shapes:
        name = "Q4_K" if ggml == Q4_K else "Q6_K"
        case = head if (ggml, n, k) == (Q4_K, 17408, 5120) else Case(
            api, synth, dev, ggml, n, k, 1, api.DType.F32, f"{name} GEMV M=1 K={k} N={n} f32 x")
        case.enqueue = lambda i, c=case: dev.probe_read(c.weights[i % len(c.weights)])
        _, event = measure(dev, case, steps, warmup)
        per, probe_kernel = event / steps, case.operation
        case.enqueue = lambda i, c=case: dev.project_quantized(c.x, c.weights[i % len(c.weights)], out=c.y)
        _, gevent = measure(dev, case, steps, warmup)
        gper = gevent / steps
        rows.append({
            "shape": f"{name} N={n} K={k}", "weight_bytes": case.weight_bytes, "rotated_bytes": len(case.weights) * case.weight_bytes,
            "read_probe_us": round(per * 1e6, 3), "read_probe_frac_hbm": round(case.weight_bytes / per / 1e9 / HBM_PEAK_GBS, 4),
            "gemv_kernel": case.operation, "gemv_us": round(gper * 1e6, 3),
            "gemv_frac_hbm": round(case.bytes / gper / 1e9 / HBM_PEAK_GBS, 4), "gemv_over_read": round(gper / per, 3)})
        del case
    print(json.dumps({"read_probe_forms_on_17408x5120_q4k_us": sweep, "best_form": best_name, "probe_kernel": probe_kernel,
                      "per_shape": rows, "steps": steps}), flush=True)


def mfma_probe_case(dev, steps):
    """Matrix-core rates: MFMA issue loops from registers with one and with four waves per
    SIMD, and an MFMA wave beside a VALU wave on the same SIMD."""
    cus = int(dev.properties().get("compute_units") or 256)
    iterations = 4096
    out = {}
    for shape, name in ((0, "v_mfma_f32_16x16x32_f16"), (1, "v_mfma_f32_32x32x16_f16"),
                        (2, "v_mfma_f32_32x32x16_f16 on random f16 operands")):
        for waves in (1, 4):
            flops = [0.0]

            def enqueue(i):
                flops[0] = dev.probe_mfma(shape, waves * cus, iterations)

            best = min(run_graph(dev, enqueue, steps, 2)[1] for _ in range(3)) / steps
            out[f"{name}, {waves} wave(s) per SIMD"] = {
                "kernel": dev.last_operation(), "us": round(best * 1e6, 2),
                "TFLOP/s": round(flops[0] / best / 1e12, 1),
                "frac_published_peak": round(flops[0] / best / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}
    together = {}

    def timed(mfma, rounds):
        def enqueue(i):
            dev.probe_coissue(cus, iterations, mfma, rounds)
        return min(run_graph(dev, enqueue, steps, 2)[1] for _ in range(3)) / steps * 1e6

    together["mfma_wave_alone_us"] = round(timed(True, 0), 1)
    for rounds in (1, 2, 4, 8):
        alone, both = timed(False, rounds), timed(True, rounds)
        together[f"valu_{8 * rounds}_fma_per_8_mfma"] = {
            "valu_wave_alone_us": round(alone, 1), "both_us": round(both, 1),
            "sum_us": round(alone + together["mfma_wave_alone_us"], 1)}
    print(json.dumps({"mfma_probe": out, "independent_chains_per_wave": 8, "iterations": iterations,
                      "mfma_and_valu_waves_on_one_simd": together}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2400)
    ap.add_argument("--warmup", type=int, default=240)
    ap.add_argument("--cases", choices=["headline", "all", "copy", "read", "mfma"], default="all",
                    help="'headline' times only the metric's GEMV; 'all' adds the other shapes; "
                         "'copy' launches a plain row copy of known size (counter calibration); "
                         "'read' times a plain read of the metric's matrices beside the GEMV; "
                         "'mfma' times matrix-core issue loops")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="with --cases all: run only the cases whose label contains this text")
    ap.add_argument("--eager", action="store_true",
                    help="launch every step from the host instead of replaying a HIP graph (timings then "
                         "include launch gaps; meant for kernel traces)")
    args = ap.parse_args()
    global EAGER
    EAGER = args.eager
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; every box has one and no multi-GPU "
                 f"path exists (asked for --gpus {args.gpus})")

    from ferrum_amd import api, synth
    dev = api.Device.new(0)
    props = dev.properties()
    f32, f16 = api.DType.F32, api.DType.F16
    if args.cases == "copy":
        return copy_calibration(api, dev)
    if args.cases == "read":
        return read_probe_case(api, synth, dev, args.steps, args.warmup)
    if args.cases == "mfma":
        return mfma_probe_case(dev, min(args.steps, 20))

    head = Case(api, synth, dev, Q4_K, 17408, 5120, 1, f32, "Q4_K GEMV M=1 K=5120 N=17408 f32 x")
    wall, event = measure(dev, head, args.steps, args.warmup)
    step_wall, step_event = wall / args.steps, event / args.steps
    gbs = head.bytes / step_wall / 1e9
    kernel_gbs = head.bytes / step_event / 1e9
    head_report = report(head, step_event)
    cpu = None if args.no_cpu else cpu_baseline(head)

    cases = [head_report]
    gemm = None
    if args.cases == "all":
        def timed(ggml, n, k, m, xd, label, steps, copies=None, after=None):
            if args.only and args.only not in label:
                return None
            c = Case(api, synth, dev, ggml, n, k, m, xd, label, copies)
            _, ev = measure(dev, c, steps, min(args.warmup, len(c.weights)), repeats=2)
            r = report(c, ev / steps)
            cases.append(r)
            if after is not None:
                after(c)
            del c
            return r

        gemm_extra = {}

        def gemm_checks(c):
            gemm_extra["distance_to_oracle"] = gemm_distance(api, dev, c)
            if not args.no_cpu:
                gemm_extra["cpu_baseline"] = cpu_baseline_gemm(c)

        timed(Q4_K, 4096, 4096, 1, f32, "Q4_K GEMV M=1 K=4096 N=4096", 1200)
        timed(Q4_K, 5120, 5120, 1, f32, "Q4_K GEMV M=1 K=5120 N=5120", 1200)
        timed(Q4_K, 5120, 17408, 1, f32, "Q4_K GEMV M=1 K=17408 N=5120", 1200)
        if not args.only or args.only in "decode layer":
            cases.append(layer_case(api, synth, dev, 400))
        timed(Q5_K, 17408, 5120, 1, f32, "Q5_K GEMV M=1 K=5120 N=17408", 600)
        timed(IQ4_XS, 17408, 5120, 1, f32, "IQ4_XS GEMV M=1 K=5120 N=17408", 600)
        timed(Q8_0, 17408, 5120, 1, f32, "Q8_0 GEMV M=1 K=5120 N=17408", 400)
        timed(Q6_K, 5120, 17408, 1, f32, "Q6_K GEMV M=1 K=17408 N=5120", 600)
        timed(Q6_K, 151936, 5120, 1, f32, "Q6_K GEMV M=1 K=5120 N=151936", 40, copies=2)
        for m in (8, 16, 128):
            timed(Q4_K, 17408, 5120, m, f16, f"Q4_K GEMM M={m} K=5120 N=17408 f16 x", 240)
        gemm = timed(Q4_K, 17408, 5120, 512, f16, "Q4_K GEMM M=512 K=5120 N=17408 f16 x", 240, after=gemm_checks)
        for m in (8, 512):
            timed(IQ4_XS, 17408, 5120, m, f16, f"IQ4_XS GEMM M={m} K=5120 N=17408 f16 x", 240)
            timed(Q8_0, 17408, 5120, m, f16, f"Q8_0 GEMM M={m} K=5120 N=17408 f16 x", 240)
        if not args.only or args.only in "Q4_K GEMM M=512 K=5120 N=17408 f32 x":
            dev.set_tuning("gemm_f32_min_rows", 5)   # the hybrid engine's tiering: f16 tiles from 5 rows on
            timed(Q4_K, 17408, 5120, 512, f32, "Q4_K GEMM M=512 K=5120 N=17408 f32 x (rounded to f16 for the tiles)", 120)
            dev.set_tuning("gemm_f32_min_rows", 0)
        # rows short enough to stay in LDS (an A3B-sized model's attention projections)
        for m in (8, 64, 512):
            timed(Q4_K, 4096, 2048, m, f16, f"Q4_K GEMM M={m} K=2048 N=4096 f16 x", 400)
        if not args.only or args.only in "MoE FFN T=1":
            cases.append(moe_case(api, synth, dev, 1, 200, cpu=not args.no_cpu))
        if not args.only or args.only in "MoE FFN T=512":
            cases.append(moe_case(api, synth, dev, 512, 20, cpu=not args.no_cpu))

    line = {
        "metric": "Q4_K GEMV GB/s at M=1, K=5120, N=17408",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_wall * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": head.label,
            "weights": "Q4_K super-blocks, seeded (d=|N|*0.01, dmin=|N|*0.005, 6-bit scales/mins, nibbles)",
            "weight_copies_rotated": len(head.weights),
            "bytes_per_step": head.bytes,
            "device": props.get("name") or props.get("arch"),
            "arch": props.get("arch"),
            "compute_units": props.get("compute_units"),
        },
        "host": host_info(),
        "roofline": {
            "bound": "hbm",
            "achieved": round(kernel_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(kernel_gbs / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic("gemv_q4k_n17408_k5120_m1", GEMV_SOURCES),
            "kernel": head.operation,
            "kernel_us": round(step_event * 1e6, 3),
            "kernel_us_from": "HIP events on the library's stream around the recorded launches replayed back to back "
                              "(one replay when the recording is longer than 2 ms), divided by the launches",
        },
        "cpu_baseline": cpu,
        "gemm_m512": None if gemm is None else {
            "metric": "Q4_K GEMM TFLOP/s at M=512, K=5120, N=17408, f16 activations, f32 output",
            "value": gemm["TFLOP/s"],
            "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": gemm["TFLOP/s"], "peak": MFMA_F16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": gemm["frac_mfma_f16"],
                         "traffic": measured_traffic("gemm_q4k_n17408_k5120_m512", GEMM_SOURCES),
                         "kernel": gemm["operation"], "kernel_us": gemm["us"]},
            "cpu_baseline": gemm_extra.get("cpu_baseline"),
            "distance_to_oracle": gemm_extra.get("distance_to_oracle"),
        },
        "cases": cases,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
