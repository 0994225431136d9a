#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sweep] [--no-cpu] [--no-mmq]

Headline workload (BASELINE.json configs[1], Q4_K, batch 1): the three decode
matvec shapes of the 27B-class layer -- K=5120 -> N=5120, the fused gate+up
K=5120 -> N=34816 and down K=17408 -> N=5120 -- with weights ~N(0,0.02) quantized
to Q4_K and repacked, activations ~N(0,1) quantized to BlockQ8.  One *step* is one
pass of each shape over a rotation of distinct weight buffers (each rotation larger
than L2 + Infinity Cache, so every launch streams its weights from HBM), captured
in one hipGraph per shape.  `value` is total algorithmic bytes / total time over
the three shapes; everything is resident in HBM before the timed region.  Prints
ONE JSON line.

The same line carries the per-shape figures, the roofline object of the dominant
kernel (the gate+up launch), the MMQ prefill GEMM (Q4_K, 512 x 5120 x 17408) in
"mmq", one compact object per remaining BASELINE configuration in "configs"
(configs[2]: Q4_K / Q6_K / Q8_0 x M 128 / 512 / 2048; configs[3]: the MoE expert FFN;
configs[4]: the 64-layer decode weight stream under one hipGraph) and the CPU baseline
(the oracle's restatement of the reference CPU path: dequantize once, then the f32
matvec of src/cpu/ops.rs:108-140 over the host cores, plus the int8 restatement of
the kernel formulas on one and on all cores) timed on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import reinstinct_amd as rein  # noqa: E402
from reinstinct_amd import hip, quant, runtime  # noqa: E402
from reinstinct_amd._lib import init  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0        # MI355X dense int8 MFMA
CACHE_BYTES = 512 << 20        # rotate over more than L2 (32 MB) + Infinity Cache (256 MB)
MMQ_ROTATION_BYTES = 320 << 20  # the same for the GEMM legs (fewer, longer launches)

FMT_NAME = {rein.Q4_0: "q4_0", rein.Q4_K: "q4_k", rein.Q5_K: "q5_k", rein.Q6_K: "q6_k", rein.Q8_0: "q8_0",
            rein.IQ4_XS: "iq4_xs", rein.IQ3_S: "iq3_s"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def synth_weights(fmt, in_dim, out_dim, seed):
    """fp32 ~N(0,0.02) -> on-disk blocks -> repacked-v2 slab (host)."""
    rng = np.random.default_rng(seed)
    if fmt == rein.IQ3_S:
        # no fp32 -> IQ3_S quantizer exists (the reference has none either): seeded random
        # blocks with a tame fp16 scale; the kernels' speed does not depend on the values
        raw = rng.integers(0, 256, (out_dim * in_dim // 256, 110), dtype=np.uint8)
        raw[:, 0:2] = np.frombuffer(np.float16(0.002).tobytes(), np.uint8)
        raw = raw.reshape(-1)
        return raw, quant.repack_for_matvec(fmt, raw, in_dim, out_dim)
    w = (rng.standard_normal((out_dim, in_dim), dtype=np.float32) * np.float32(0.02))
    raw = quant.quantize_weights(fmt, w)
    return raw, quant.repack_for_matvec(fmt, raw, in_dim, out_dim)


def matvec_bytes(fmt, in_dim, out_dim, batch):
    """algorithmic bytes of one launch: weights + BlockQ8 activations + fp32 outputs"""
    return quant.repacked_len(fmt, in_dim, out_dim) + batch * (in_dim // 32) * 40 + batch * out_dim * 4


def weight_rotation(packed, min_bytes=CACHE_BYTES):
    """Distinct device copies of one slab, together larger than L2 + Infinity Cache."""
    first = hip.DeviceBuf.from_host(packed)
    bufs = [first]
    for _ in range(max(2, -(-min_bytes // packed.nbytes)) - 1):
        b = hip.DeviceBuf(packed.nbytes)
        rein.lib.rein_memcpy_d2d(b.ptr, first.ptr, packed.nbytes)
        bufs.append(b)
    return bufs


CLOCK_SETTLE_S = 0.08


def settle(launch, stream, seconds=CLOCK_SETTLE_S):
    """Untimed repetitions of the launches about to be timed, for `seconds` of wall time.  The GPU raises its
    clocks over tens of milliseconds of continuous work: the first 4 ms after an idle stretch (host-side
    preparation of the next case) run the 512-token prefill GEMM at 176 us per launch, the steady state is
    143-156 us.  Every timed region of this file starts from that steady state; the W warm-up steps follow.
    `launch` issues the kernels one by one, not as a graph: rocprofv3 7.2 ends a process with a segmentation
    fault once about 16 000 kernels have been dispatched from hipGraphs (plain launches: 43 000 and counting),
    and this file has to run under it."""
    t_end = time.perf_counter() + seconds
    while True:
        launch()
        stream.synchronize()
        if time.perf_counter() >= t_end:
            return


class MatvecCase:
    """A rotation of weight buffers and a captured graph of one pass over them."""

    def __init__(self, fmt, in_dim, out_dim, batch, stream, seed=0, min_bytes=CACHE_BYTES, packed=None, weights=None):
        self.fmt, self.in_dim, self.out_dim, self.batch, self.stream = fmt, in_dim, out_dim, batch, stream
        if weights is None:
            if packed is None:
                _, packed = synth_weights(fmt, in_dim, out_dim, seed)
            weights = weight_rotation(packed, min_bytes)
        self.weights = weights
        self.n_buf = len(weights)
        x = np.random.default_rng(seed + 1).standard_normal((batch, in_dim)).astype(np.float32)
        self.x = x
        self.dx = hip.DeviceBuf.from_host(x)
        self.dq = hip.DeviceBuf(batch * (in_dim // 32) * 40)
        self.dy = hip.DeviceBuf(batch * out_dim * 4)
        runtime.quantize_q8(self.dx, self.dq, in_dim, batch, stream)
        stream.synchronize()
        self.bytes_per_launch = matvec_bytes(fmt, in_dim, out_dim, batch)
        stream.begin_capture()
        for wbuf in self.weights:
            self.launch(wbuf)
        self.graph = stream.end_capture()
        self.exe = self.graph.instantiate()

    def launch(self, wbuf):
        if self.batch == 1:
            runtime.matvec_xq8(self.fmt, wbuf, self.dq, self.dy, self.in_dim, self.out_dim, self.stream)
        else:
            runtime.matvec_batched_xq8(self.fmt, wbuf, self.dq, self.dy, self.in_dim, self.out_dim, self.batch,
                                       self.stream)

    def step(self):
        self.exe.launch(self.stream)

    def time(self, steps, warmup):
        """-> (seconds per step, seconds per launch), events on the launch stream"""
        settle(lambda: [self.launch(w) for w in self.weights], self.stream)
        for _ in range(warmup):
            self.step()
        self.stream.synchronize()
        e0, e1 = hip.Event(), hip.Event()
        e0.record(self.stream)
        for _ in range(steps):
            self.step()
        e1.record(self.stream)
        e1.synchronize()
        sec = e0.elapsed_ms(e1) * 1e-3
        return sec / steps, sec / (steps * self.n_buf)


class MmqCase:
    def __init__(self, fmt, p_rows, in_dim, out_dim, stream, seed=0):
        self.fmt, self.p, self.in_dim, self.out_dim, self.stream = fmt, p_rows, in_dim, out_dim, stream
        _, packed = synth_weights(fmt, in_dim, out_dim, seed)
        # more than L2 (32 MB) + Infinity Cache (256 MB) of distinct weights: Q4_K 5120 x 17408 is 51.5 MB -> 7 copies
        self.weights = weight_rotation(packed, MMQ_ROTATION_BYTES)
        self.n_buf = len(self.weights)
        x = np.random.default_rng(seed + 1).standard_normal((p_rows, in_dim)).astype(np.float32)
        self.dx = hip.DeviceBuf.from_host(x)
        self.dq = hip.DeviceBuf(p_rows * (in_dim // 32) * 40)
        self.dy = hip.DeviceBuf(p_rows * out_dim * 4)
        runtime.quantize_q8(self.dx, self.dq, in_dim, p_rows, stream)
        stream.synchronize()
        self.ops = 2.0 * p_rows * in_dim * out_dim      # reference convention, kernels.rs:2917
        # the workspace launch (activation operand image + GEMM) where the format has one
        self.ws_bytes = runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
        self.ws = hip.DeviceBuf(self.ws_bytes) if self.ws_bytes else None

    def launch(self, i):
        runtime.mmq_xq8_ws(self.fmt, self.weights[i % self.n_buf], self.dq, self.dy, self.in_dim, self.out_dim,
                           self.p, self.ws, self.ws_bytes, self.stream)

    def time(self, launches, warmup):
        settle(lambda: [self.launch(i) for i in range(self.n_buf)], self.stream)
        for i in range(warmup):
            self.launch(i)
        self.stream.synchronize()
        e0, e1 = hip.Event(), hip.Event()
        e0.record(self.stream)
        for i in range(launches):
            self.launch(i)
        e1.record(self.stream)
        e1.synchronize()
        return e0.elapsed_ms(e1) * 1e-3 / launches


def cpu_threads():
    """Threads for the CPU legs: the CPU share the box grants this job (OMP_NUM_THREADS where it
    is set -- 16 on a one-GPU box, whatever the host's core count), else every core."""
    host = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    return (max(1, min(int(env), host)) if env and env.isdigit() else host), host


def best_of(fn, budget_s, max_reps=2000):
    fn()
    best, reps, t_start = 1e30, 0, time.perf_counter()
    while time.perf_counter() - t_start < budget_s and reps < max_reps:
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
        reps += 1
    return best, reps


def cpu_baseline(fmt, in_dim, out_dim, seed, budget_s=10.0):
    """The reference CPU path (dequantize once, untimed; then the f32 matvec of
    src/cpu/ops.rs:108-140 over the granted cores) on the headline shape, and beside it the
    int8 restatement of the kernel formulas (quantized activations against the repacked
    weights) on one thread and on all of them; each leg repeats for a bounded time."""
    from oracle import orc          # the checker, used here only as the timed CPU baseline

    cores, host = cpu_threads()
    raw, packed = synth_weights(fmt, in_dim, out_dim, seed)
    w = orc.dequantize_to_f32(fmt, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    x = np.random.default_rng(seed + 1).standard_normal(in_dim).astype(np.float32)
    nbytes = matvec_bytes(fmt, in_dim, out_dim, 1)
    best, reps = best_of(lambda: orc.matvec_f32(x, w, n_threads=cores), budget_s * 0.5)
    xq = orc.quantize_q8(x[None, :])
    i1, r1 = best_of(lambda: orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, 1, n_threads=1), budget_s * 0.25, 200)
    ia, ra = best_of(lambda: orc.matvec_q8(fmt, packed, in_dim, out_dim, xq, 1, n_threads=cores), budget_s * 0.25)
    return {"value": round(nbytes / best / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "host_hardware_concurrency": host,
            "sample": f"dequantize_to_f32 once (untimed) + f32 matvec {in_dim}->{out_dim} on {cores} threads (the CPU share "
                      f"of this job; the host reports {host}), best of {reps} runs, algorithmic (repacked) bytes / time; "
                      f"{round(in_dim * out_dim * 4 / best / 1e9, 2)} GB/s of f32 traffic",
            "int8_restatement": {"unit": "GB/s", "threads_1": round(nbytes / i1 / 1e9, 3), "runs_1": r1,
                                 f"threads_{cores}": round(nbytes / ia / 1e9, 3), "runs_all": ra,
                                 "sample": f"oracle int8 matvec (BlockQ8 x repacked {FMT_NAME[fmt]}) {in_dim}->{out_dim}, "
                                           "best run, same algorithmic bytes"}}


def tiled_weights(fmt, in_dim, out_dim, seed, base_rows=512):
    """Repacked weights for timing only: quantize base_rows rows and tile them (the
    kernels' speed does not depend on the values)."""
    base_rows = min(base_rows, out_dim)
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((base_rows, in_dim), dtype=np.float32) * np.float32(0.02))
    raw = quant.quantize_weights(fmt, w)
    reps = -(-out_dim // base_rows)
    raw = np.tile(raw, reps)[: out_dim * in_dim // quant.block_size(fmt) * quant.bytes_per_block(fmt)]
    return quant.repack_for_matvec(fmt, raw, in_dim, out_dim)


def time_graph(stream, launch_all, n_launches, steps=5):
    """seconds per launch of a captured train of launches"""
    stream.begin_capture()
    launch_all()
    g = stream.end_capture()
    ex = g.instantiate()
    settle(launch_all, stream)
    ex.launch(stream)
    stream.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    e0.record(stream)
    for _ in range(steps):
        ex.launch(stream)
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_ms(e1) * 1e-3 / (steps * n_launches)


def mmq_kernel_name(fmt, in_dim, out_dim, p_rows):
    """the kernels the MMQ launch of this shape runs"""
    tag = {rein.Q4_K: "q4k", rein.Q5_K: "q5k", rein.Q6_K: "q6k"}.get(fmt, FMT_NAME[fmt])
    ws_bytes = runtime.mmq_workspace_bytes(fmt, in_dim, p_rows)
    form = runtime.mmq_form_ws(fmt, in_dim, out_dim, p_rows, ws_bytes)
    if form == 4:
        return "rein_mmq16_prep + rein_mmq16_q4k (fp16 formulation, REIN_MMQ16=1)"
    if form == 2:
        return f"rein_mmq6_prep + rein_mmq6_{tag}_sk (split-tail launch) + rein_mmq6_tail_sum"
    if form == 3:
        return f"rein_mmq_{tag}_sk / _sk32 (split-tail launch of the int8 tile) + rein_mmq_tail_sum_t64 / _t32"
    if form == 1:
        n4, n2 = runtime.mmq_tile_plan_ws(fmt, out_dim, p_rows)
        return f"rein_mmq6_prep + rein_mmq6_{tag}_mix (n4 = {n4}, n2 = {n2})"
    n64 = runtime.mmq_tile_plan(fmt, in_dim, out_dim, p_rows)
    return f"rein_mmq_{tag}_mix (n64 = {n64})" if n64 else f"rein_mmq_{tag}_t32"


def extras_mmq(stream):
    """BASELINE configs[2]: B in {Q4_K, Q6_K, Q8_0} x M in {128, 512, 2048}, 5120 x 17408; Q5_K beside them (the
    reference publishes its MMQ figure too, src/runtime/kernels.rs:2852-2944)"""
    out = []
    k, n = 5120, 17408
    for f in (rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.Q8_0):
        packed = tiled_weights(f, k, n, seed=3)
        ws = weight_rotation(packed, MMQ_ROTATION_BYTES)                    # > L2 + Infinity Cache of distinct weights
        for m in (128, 512, 2048):
            x = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
            dx, dq, dy = hip.DeviceBuf.from_host(x), hip.DeviceBuf(m * (k // 32) * 40), hip.DeviceBuf(m * n * 4)
            runtime.quantize_q8(dx, dq, k, m, stream)
            wsb = runtime.mmq_workspace_bytes(f, k, m)
            wsp = hip.DeviceBuf(wsb) if wsb else None
            sec = time_graph(stream, lambda: [runtime.mmq_xq8_ws(f, w_, dq, dy, k, n, m, wsp, wsb, stream) for w_ in ws], len(ws))
            tops = 2.0 * m * k * n / sec / 1e12
            out.append({"fmt": FMT_NAME[f], "M": m, "us": round(sec * 1e6, 1), "TOPS": round(tops, 1),
                        "frac_int8_peak": round(tops / INT8_PEAK_TOPS, 4)})
            log("mmq", out[-1])
            del dx, dq, dy, wsp
        del ws
    return out


def extras_mmq_small(stream):
    """Short prompts against the narrow projections (the decode shapes of BASELINE configs[1] as prefill
    GEMMs): too few workgroup tiles for 256 CUs, which the split-tail launch of rein_mmq_xq8_ws repairs
    when the caller provides the workspace; `us_no_workspace` is the plain launch of rein_mmq_xq8."""
    out = []
    for f in (rein.Q4_K, rein.Q6_K, rein.Q8_0):
        for (k, n) in ((17408, 5120), (5120, 5120)):
            packed = tiled_weights(f, k, n, seed=4)
            ws = [hip.DeviceBuf.from_host(packed) for _ in range(max(4, (300 << 20) // packed.nbytes))]
            for m in (32, 128):
                x = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
                dx, dq, dy = hip.DeviceBuf.from_host(x), hip.DeviceBuf(m * (k // 32) * 40), hip.DeviceBuf(m * n * 4)
                runtime.quantize_q8(dx, dq, k, m, stream)
                wsb = runtime.mmq_workspace_bytes(f, k, m)
                wsp = hip.DeviceBuf(wsb) if wsb else None
                sec = time_graph(stream, lambda: [runtime.mmq_xq8_ws(f, w_, dq, dy, k, n, m, wsp, wsb, stream) for w_ in ws], len(ws))
                sec0 = time_graph(stream, lambda: [runtime.mmq_xq8(f, w_, dq, dy, k, n, m, stream) for w_ in ws], len(ws))
                out.append({"fmt": FMT_NAME[f], "M": m, "K": k, "N": n, "us": round(sec * 1e6, 1),
                            "us_no_workspace": round(sec0 * 1e6, 1), "launch": runtime.mmq_form_ws(f, k, n, m, wsb)})
                log("mmq small", out[-1])
                del dx, dq, dy, wsp
            del ws
    return out


def extras_moe(stream):
    """BASELINE configs[3]: 512 tokens, hidden 2048, 128 experts, top-8, expert ff 768; gate/up Q4_K,
    down Q6_K; top-k -> sort -> gather -> grouped GEMMs with SwiGLU -> scatter -> combine."""
    n_tok, hidden, n_expert, n_used, ff = 512, 2048, 128, 8, 768
    rng = np.random.default_rng(11)
    gate1 = tiled_weights(rein.Q4_K, hidden, ff, seed=1, base_rows=ff)
    up1 = tiled_weights(rein.Q4_K, hidden, ff, seed=2, base_rows=ff)
    down1 = tiled_weights(rein.Q6_K, ff, hidden, seed=3, base_rows=hidden)
    gate = hip.DeviceBuf.from_host(np.tile(gate1, n_expert))
    up = hip.DeviceBuf.from_host(np.tile(up1, n_expert))
    down = hip.DeviceBuf.from_host(np.tile(down1, n_expert))
    weight_bytes = (gate1.nbytes + up1.nbytes + down1.nbytes) * n_expert
    x = rng.standard_normal((n_tok, hidden)).astype(np.float32)
    logits = rng.standard_normal((n_tok, n_expert)).astype(np.float32)
    dx, dl = hip.DeviceBuf.from_host(x), hip.DeviceBuf.from_host(logits)
    ds = hip.DeviceBuf.from_host(np.ones(n_expert, np.float32))
    shape = runtime.moe_shape(n_tok, hidden, n_expert, n_used, ff, rein.Q4_K, rein.Q6_K)
    wsb = hip.DeviceBuf(runtime.moe_workspace_bytes(shape))
    dout = hip.DeviceBuf(n_tok * hidden * 4)
    reps = 4
    sec = time_graph(stream, lambda: [runtime.moe_ffn(shape, dx, dl, gate, up, down, ds, wsb, dout, stream)
                                      for _ in range(reps)], reps)
    ops = 2.0 * n_tok * n_used * (2 * hidden * ff + ff * hidden)
    res = {"workload": "MoE expert FFN, 512 tok x 128 experts top-8, hidden 2048, ff 768 (Q4_K gate/up, Q6_K down)",
           "us": round(sec * 1e6, 1), "weight_GBs": round(weight_bytes / sec / 1e9, 0),
           "frac_hbm_peak": round(weight_bytes / sec / 1e9 / HBM_PEAK_GBS, 4), "TOPS": round(ops / sec / 1e12, 1),
           "frac_int8_peak": round(ops / sec / 1e12 / INT8_PEAK_TOPS, 4), "weight_bytes": weight_bytes,
           "note": "the 401 MB of expert weights are re-read from the 256 MB Infinity Cache + HBM on every repetition"}
    log("moe", res)
    return res


def extras_moe_decode(stream):
    """One decode token through the MoE expert FFN of configs[3] (128 experts, top-8, hidden 2048,
    ff 768): gate+up+SwiGLU+quantize (Q4_K) -> down+combine (Q6_K) in two launches, and the four-launch
    chain of the reference (gate+up+SwiGLU matvec -> quantize -> down matvec -> combine) beside it; expert
    ids read on the device.  16 tokens with disjoint expert sets per graph, so every launch streams
    experts that are not in cache."""
    hidden, n_expert, n_used, ff = 2048, 128, 8, 768
    gate1 = tiled_weights(rein.Q4_K, hidden, ff, seed=1, base_rows=ff)
    up1 = tiled_weights(rein.Q4_K, hidden, ff, seed=2, base_rows=ff)
    down1 = tiled_weights(rein.Q6_K, ff, hidden, seed=3, base_rows=hidden)
    gate = hip.DeviceBuf.from_host(np.tile(gate1, n_expert))
    up = hip.DeviceBuf.from_host(np.tile(up1, n_expert))
    down = hip.DeviceBuf.from_host(np.tile(down1, n_expert))
    per_token = (gate1.nbytes + up1.nbytes + down1.nbytes) * n_used
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, hidden)).astype(np.float32)
    dxq = hip.DeviceBuf(hidden // 32 * 40)
    runtime.quantize_q8(hip.DeviceBuf.from_host(x), dxq, hidden, 1, stream)
    toks = n_expert // n_used
    ids = [hip.DeviceBuf.from_host(np.arange(t * n_used, (t + 1) * n_used, dtype=np.int32)) for t in range(toks)]
    wts = hip.DeviceBuf.from_host(np.full(n_used, 1.0 / n_used, np.float32))
    ones = hip.DeviceBuf.from_host(np.ones(n_expert, np.float32))
    act, aq = hip.DeviceBuf(n_used * ff * 4), hip.DeviceBuf(n_used * ff // 32 * 40)
    eo, out = hip.DeviceBuf(n_used * hidden * 4), hip.DeviceBuf(hidden * 4)
    ns_h, ns_f = hidden // 32, ff // 32

    def token(t):
        runtime.moe_gate_up_swiglu(rein.Q4_K, gate, up, ids[t], dxq, act, hidden, ff, gate1.nbytes, ns_h, 0, n_used, 1, stream)
        runtime.quantize_q8(act, aq, ff, n_used, stream)
        runtime.moe_down(rein.Q6_K, down, ids[t], aq, eo, ff, hidden, down1.nbytes, n_used * ns_f, ns_f, n_used, 1, stream)
        runtime.moe_combine(eo, ids[t], wts, ones, out, 1, hidden, n_used, stream)

    def token_fused(t):
        runtime.moe_gate_up_swiglu_q8(rein.Q4_K, gate, up, ids[t], dxq, aq, hidden, ff, gate1.nbytes, ns_h, 0, n_used, 1, stream)
        runtime.moe_down_combine(rein.Q6_K, down, ids[t], wts, ones, aq, out, ff, hidden, down1.nbytes, n_used * ns_f, ns_f,
                                 n_used, 1, stream)

    # the whole routed FFN of one token through rein_moe_ffn (router and quantizer included): the logits of token t
    # peak on its own eight experts, so the sixteen tokens of a graph stream disjoint experts as above
    shape = runtime.moe_shape(1, hidden, n_expert, n_used, ff, rein.Q4_K, rein.Q6_K)
    wsb = hip.DeviceBuf(runtime.moe_workspace_bytes(shape))
    dx = hip.DeviceBuf.from_host(x)
    lg = np.zeros((toks, n_expert), np.float32)
    for t in range(toks):
        lg[t, t * n_used:(t + 1) * n_used] = 4.0 + 0.1 * np.arange(n_used, dtype=np.float32)
    dlg = [hip.DeviceBuf.from_host(lg[t:t + 1]) for t in range(toks)]

    def token_ffn(t):
        runtime.moe_ffn(shape, dx, dlg[t], gate, up, down, ones, wsb, out, stream)

    sec4 = time_graph(stream, lambda: [token(t) for t in range(toks)], toks)
    sec = time_graph(stream, lambda: [token_fused(t) for t in range(toks)], toks)
    sec_ffn = time_graph(stream, lambda: [token_ffn(t) for t in range(toks)], toks)
    res = {"workload": "MoE decode expert FFN, 1 token, 128 experts top-8, hidden 2048, ff 768: gate+up+SwiGLU+quantize "
                       "(Q4_K) -> down+combine (Q6_K), 2 launches",
           "us_per_token": round(sec * 1e6, 2), "us_per_token_4_launch_chain": round(sec4 * 1e6, 2),
           "us_per_token_rein_moe_ffn": round(sec_ffn * 1e6, 2),
           "rein_moe_ffn_note": "router + quantizer + the two launches above from fp32 x and logits: 2 launches per token",
           "expert_bytes_per_token": per_token,
           "GBs": round(per_token / sec / 1e9, 0), "frac_hbm_peak": round(per_token / sec / 1e9 / HBM_PEAK_GBS, 4)}
    log("moe decode", res)
    return res


def extras_ondisk(stream):
    """The matvec call sites outside the repacked path: the tied LM head in on-disk Q6_K blocks
    (5120 -> 151936, 638 MB) and the split-K Q8_0 matvec for a tiny projection (5120 -> 96)."""
    out = []
    k, n = 5120, 151936
    w = (np.random.default_rng(0).standard_normal((1024, k)) * 0.02).astype(np.float32)
    raw = np.tile(quant.quantize_weights(rein.Q6_K, w), n // 1024 + 1)[: n * (k // 256) * 210]
    dw = [hip.DeviceBuf.from_host(raw) for _ in range(2)]
    x = np.random.default_rng(1).standard_normal((1, k)).astype(np.float32)
    dq = hip.DeviceBuf(k // 32 * 40)
    runtime.quantize_q8(hip.DeviceBuf.from_host(x), dq, k, 1, stream)
    dy = hip.DeviceBuf(n * 4)
    sec = time_graph(stream, lambda: [runtime.matvec_ondisk_xq8(rein.Q6_K, b, dq, dy, k, n, stream) for b in dw], 2)
    out.append({"op": "on-disk Q6_K matvec 5120 -> 151936 (tied LM head)", "us": round(sec * 1e6, 1),
                "GBs": round(raw.nbytes / sec / 1e9, 0), "frac_hbm_peak": round(raw.nbytes / sec / 1e9 / HBM_PEAK_GBS, 4)})
    packed = quant.repack_for_matvec(rein.Q6_K, raw, k, n)
    dp = [hip.DeviceBuf.from_host(packed) for _ in range(2)]
    sec = time_graph(stream, lambda: [runtime.matvec_xq8(rein.Q6_K, b, dq, dy, k, n, stream) for b in dp], 2)
    out.append({"op": "repacked Q6_K matvec, same matrix", "us": round(sec * 1e6, 1),
                "GBs": round(packed.nbytes / sec / 1e9, 0), "frac_hbm_peak": round(packed.nbytes / sec / 1e9 / HBM_PEAK_GBS, 4)})
    del dw, dp
    # the decode kernel away from the launch ramp: the same K = 5120 contraction, Q4_K, at the
    # vocabulary-sized N (450 MB per launch)
    p4 = tiled_weights(rein.Q4_K, k, n, seed=4)
    d4 = [hip.DeviceBuf.from_host(p4) for _ in range(2)]
    sec = time_graph(stream, lambda: [runtime.matvec_xq8(rein.Q4_K, b, dq, dy, k, n, stream) for b in d4], 2)
    out.append({"op": "repacked Q4_K matvec 5120 -> 151936 (450 MB per launch)", "us": round(sec * 1e6, 1),
                "GBs": round(p4.nbytes / sec / 1e9, 0), "frac_hbm_peak": round(p4.nbytes / sec / 1e9 / HBM_PEAK_GBS, 4)})
    del d4
    n2 = 96
    w8 = quant.repack_for_matvec(rein.Q8_0, quant.quantize_weights(rein.Q8_0, w[:n2]), k, n2)
    d8 = hip.DeviceBuf.from_host(w8)
    yp = hip.DeviceBuf(16 * n2 * 4)
    reps = 32
    for ns in (1, 4, 8, 16):
        sec = time_graph(stream, lambda: [runtime.matvec_q8_0_splitk(d8, dq, yp, k, n2, ns, stream) for _ in range(reps)], reps)
        out.append({"op": f"Q8_0 split-K matvec 5120 -> 96, n_split {ns}", "us": round(sec * 1e6, 2)})
    sec = time_graph(stream, lambda: [runtime.matvec_xq8(rein.Q8_0, d8, dq, yp, k, n2, stream) for _ in range(reps)], reps)
    out.append({"op": "Q8_0 matvec 5120 -> 96 without the split", "us": round(sec * 1e6, 2)})
    for r in out:
        log("ondisk", r)
    return out


def extras_decode_stream(stream):
    """BASELINE configs[4]: 64 layers x {QKV 5120->7168, O 5120->5120, gate+up 5120->34816, down 17408->5120},
    Q4_K with every fourth layer's down and the 5120->151936 LM head in Q6_K, batch 1, one hipGraph."""
    n_layers, hidden, ffn = 64, 5120, 17408
    shapes = [("qkv", hidden, 7168), ("o", hidden, hidden), ("gate_up", hidden, 2 * ffn), ("down", ffn, hidden)]
    uniq = {}
    for name, k, n in shapes:
        for f in ((rein.Q4_K, rein.Q6_K) if name == "down" else (rein.Q4_K,)):
            uniq[(name, f)] = tiled_weights(f, k, n, seed=len(uniq))
    head = tiled_weights(rein.Q6_K, hidden, 151936, seed=99)
    layers, total = [], 0
    for layer in range(n_layers):
        for name, k, n in shapes:
            f = rein.Q6_K if (name == "down" and layer % 4 == 3) else rein.Q4_K
            buf = hip.DeviceBuf.from_host(uniq[(name, f)])                  # every layer its own copy in HBM
            layers.append((f, buf, k, n))
            total += uniq[(name, f)].nbytes
    dhead = hip.DeviceBuf.from_host(head)
    total += head.nbytes
    xs = {k: np.random.default_rng(k).standard_normal((1, k)).astype(np.float32) for k in (hidden, ffn)}
    dq = {}
    for k, x in xs.items():
        dx = hip.DeviceBuf.from_host(x)
        dq[k] = hip.DeviceBuf((k // 32) * 40)
        runtime.quantize_q8(dx, dq[k], k, 1, stream)
    dy = hip.DeviceBuf(151936 * 4)

    def step():
        for f, buf, k, n in layers:
            runtime.matvec_xq8(f, buf, dq[k], dy, k, n, stream)
        runtime.matvec_xq8(rein.Q6_K, dhead, dq[hidden], dy, hidden, 151936, stream)

    sec = time_graph(stream, step, 1, steps=5)
    res = {"workload": "decode weight stream, 64 layers (QKV, O, gate+up, down) + LM head, batch 1, one hipGraph of "
                       f"{len(layers) + 1} matvecs (Q4_K; every 4th down and the head Q6_K)",
           "ms_per_token": round(sec * 1e3, 3), "tokens_per_s": round(1.0 / sec, 1), "weight_GB": round(total / 1e9, 2),
           "GBs": round(total / sec / 1e9, 0), "frac_hbm_peak": round(total / sec / 1e9 / HBM_PEAK_GBS, 4)}
    log("decode stream", res)
    return res


def extras_decode_layer_separate(stream):
    """One decoder layer's matvecs at batch 1 when the model file keeps its projections as separate tensors, which is
    how the reference launches them (src/runtime/qwen35.rs:2670-2705): Q 5120->5120, K and V 5120->1024 (V in Q6_K),
    O 5120->5120, gate and up 5120->17408, down 17408->5120 -- seven launches -- against the same seven products in
    four launches with rein_matvec_multi_xq8 (Q+K+V, O, gate+up, down).  Eight layers with their own weights in one
    hipGraph, so every matvec streams from HBM."""
    n_layers, hidden, ffn, kv = 8, 5120, 17408, 1024
    spec = [("q", rein.Q4_K, hidden, hidden), ("k", rein.Q4_K, hidden, kv), ("v", rein.Q6_K, hidden, kv),
            ("o", rein.Q4_K, hidden, hidden), ("gate", rein.Q4_K, hidden, ffn), ("up", rein.Q4_K, hidden, ffn),
            ("down", rein.Q4_K, ffn, hidden)]
    host = {nm: tiled_weights(f, k, n, seed=i) for i, (nm, f, k, n) in enumerate(spec)}
    layers = [{nm: hip.DeviceBuf.from_host(host[nm]) for nm, _, _, _ in spec} for _ in range(n_layers)]
    total = sum(h.nbytes for h in host.values())
    fm = {nm: f for nm, f, _, _ in spec}
    dq = {}
    for k in (hidden, ffn):
        dx = hip.DeviceBuf.from_host(np.random.default_rng(k).standard_normal((1, k)).astype(np.float32))
        dq[k] = hip.DeviceBuf((k // 32) * 40)
        runtime.quantize_q8(dx, dq[k], k, 1, stream)
    ys = {nm: hip.DeviceBuf(n * 4) for nm, _, _, n in spec}

    def seven():
        for w in layers:
            for nm, f, k, n in spec:
                runtime.matvec_xq8(f, w[nm], dq[k], ys[nm], k, n, stream)

    def four():
        for w in layers:
            runtime.matvec_multi_xq8([fm["q"], fm["k"], fm["v"]], [w["q"], w["k"], w["v"]], [ys["q"], ys["k"], ys["v"]],
                                     [hidden, kv, kv], dq[hidden], hidden, 1, stream)
            runtime.matvec_xq8(fm["o"], w["o"], dq[hidden], ys["o"], hidden, hidden, stream)
            runtime.matvec_multi_xq8([fm["gate"], fm["up"]], [w["gate"], w["up"]], [ys["gate"], ys["up"]], [ffn, ffn],
                                     dq[hidden], hidden, 1, stream)
            runtime.matvec_xq8(fm["down"], w["down"], dq[ffn], ys["down"], ffn, hidden, stream)

    a = time_graph(stream, seven, n_layers)
    b = time_graph(stream, four, n_layers)
    res = {"workload": "one decoder layer, projections kept as separate tensors (Q, K, V, O, gate, up, down; Q4_K, V in Q6_K), "
                       "batch 1, 8 layers in one hipGraph",
           "us_per_layer_7_launches": round(a * 1e6, 2), "us_per_layer_4_launches_multi": round(b * 1e6, 2),
           "weight_MB_per_layer": round(total / 1e6, 1), "GBs_7_launches": round(total / a / 1e9, 0),
           "GBs_4_launches_multi": round(total / b / 1e9, 0), "frac_hbm_peak_multi": round(total / b / 1e9 / HBM_PEAK_GBS, 4)}
    log("decode layer, separate tensors", res)
    return res


def extras_decode_ffn(stream):
    """The FFN half of a dense decoder layer at batch 1 with the fused producers in place
    (hidden 5120, FFN 17408, Q4_K): add_rmsnorm_q8 -> gate+up matvec -> swiglu_q8 -> down matvec,
    four launches, against the six-launch chain without the fusion (norm, quantize, matvec,
    swiglu, quantize, matvec).  Eight layers with their own weights in one hipGraph, so every
    matvec streams from HBM."""
    n_layers, hidden, ffn = 8, 5120, 17408
    wgu = tiled_weights(rein.Q4_K, hidden, 2 * ffn, seed=1)
    wdn = tiled_weights(rein.Q4_K, ffn, hidden, seed=2)
    gu_w = [hip.DeviceBuf.from_host(wgu) for _ in range(n_layers)]
    dn_w = [hip.DeviceBuf.from_host(wdn) for _ in range(n_layers)]
    rng = np.random.default_rng(3)
    dev = hip.DeviceBuf.from_host
    h = dev(rng.standard_normal(hidden).astype(np.float32))
    attn = dev((rng.standard_normal(hidden) * 0.1).astype(np.float32))
    wn = dev(np.ones(hidden, np.float32))
    yn, q1 = hip.DeviceBuf(hidden * 4), hip.DeviceBuf(hidden // 32 * 40)
    gu = hip.DeviceBuf(2 * ffn * 4)
    up = gu.ptr + ffn * 4                               # the up half of the fused gate+up output
    act, q2 = hip.DeviceBuf(ffn * 4), hip.DeviceBuf(ffn // 32 * 40)
    out = hip.DeviceBuf(hidden * 4)

    def fused():
        for layer in range(n_layers):
            runtime.add_rmsnorm_q8(h, attn, wn, None, q1, hidden, 1, 1e-6, stream)
            runtime.matvec_xq8(rein.Q4_K, gu_w[layer], q1, gu, hidden, 2 * ffn, stream)
            runtime.swiglu_q8(gu, up, None, q2, ffn, stream)
            runtime.matvec_xq8(rein.Q4_K, dn_w[layer], q2, out, ffn, hidden, stream)

    def chain():
        for layer in range(n_layers):
            runtime.add_rmsnorm_q8(h, attn, wn, yn, q1, hidden, 1, 1e-6, stream)     # stands in for the fp32-only norm
            runtime.quantize_q8(yn, q1, hidden, 1, stream)
            runtime.matvec_xq8(rein.Q4_K, gu_w[layer], q1, gu, hidden, 2 * ffn, stream)
            runtime.swiglu_mul(gu, up, act, ffn, stream)
            runtime.quantize_q8(act, q2, ffn, 1, stream)
            runtime.matvec_xq8(rein.Q4_K, dn_w[layer], q2, out, ffn, hidden, stream)

    t_fused = time_graph(stream, fused, n_layers, steps=5)
    t_chain = time_graph(stream, chain, n_layers, steps=5)
    nbytes = wgu.nbytes + wdn.nbytes
    res = {"workload": "dense decoder FFN half-layer, batch 1, hidden 5120, FFN 17408, Q4_K, 8 layers per hipGraph",
           "us_per_layer_fused_4_launches": round(t_fused * 1e6, 2), "us_per_layer_unfused_6_launches": round(t_chain * 1e6, 2),
           "weight_bytes_per_layer": nbytes, "GBs_fused": round(nbytes / t_fused / 1e9, 0),
           "frac_hbm_peak_fused": round(nbytes / t_fused / 1e9 / HBM_PEAK_GBS, 4)}
    log("decode ffn", res)
    return res


def extras_fused(stream):
    """The producers in front of the matvecs: fused (one launch writes the BlockQ8 blocks) against the
    two-launch chain they replace, at the decode shapes (hidden 5120, FFN 17408) and the MoE
    intermediate (4096 expert rows x 768).  Launch-bound: microseconds per launch from a hipGraph."""
    out = []
    rng = np.random.default_rng(0)
    n, ffn, rows, ff = 5120, 17408, 4096, 768
    dev = hip.DeviceBuf.from_host
    h, a, w = (dev(rng.standard_normal(n).astype(np.float32)) for _ in range(3))
    y, q = hip.DeviceBuf(n * 4), hip.DeviceBuf(n // 32 * 40)
    reps = 32

    def t(fn):
        return time_graph(stream, lambda: [fn() for _ in range(reps)], reps) * 1e6

    out.append({"op": "add_rmsnorm_q8 n=5120 (hidden += add, norm, fp32 + BlockQ8)",
                "us": round(t(lambda: runtime.add_rmsnorm_q8(h, a, w, y, q, n, 1, 1e-6, stream)), 2)})
    out.append({"op": "rmsnorm_q8 n=5120", "us": round(t(lambda: runtime.rmsnorm_q8(h, w, q, n, 1, 1e-6, stream)), 2)})
    out.append({"op": "quantize_q8 n=5120 alone", "us": round(t(lambda: runtime.quantize_q8(h, q, n, 1, stream)), 2)})
    g, u = (dev(rng.standard_normal(ffn).astype(np.float32)) for _ in range(2))
    o, q2 = hip.DeviceBuf(ffn * 4), hip.DeviceBuf(ffn // 32 * 40)
    out.append({"op": "swiglu_q8 n=17408 fused", "us": round(t(lambda: runtime.swiglu_q8(g, u, o, q2, ffn, stream)), 2)})
    out.append({"op": "swiglu_mul + quantize_q8 n=17408 (two launches)",
                "us": round(t(lambda: (runtime.swiglu_mul(g, u, o, ffn, stream), runtime.quantize_q8(o, q2, ffn, 1, stream))), 2)})
    big = rows * ff
    g, u = (dev(rng.standard_normal(big).astype(np.float32)) for _ in range(2))
    o, q3 = hip.DeviceBuf(big * 4), hip.DeviceBuf(big // 32 * 40)
    fused = t(lambda: runtime.swiglu_q8(g, u, None, q3, big, stream))
    chain = t(lambda: (runtime.swiglu_mul(g, u, o, big, stream), runtime.quantize_q8(o, q3, ff, rows, stream)))
    out.append({"op": "swiglu_q8 4096 x 768 fused (MoE intermediate)", "us": round(fused, 2),
                "GBs": round((2 * big * 4 + big // 32 * 40) / fused / 1e3, 0)})
    out.append({"op": "swiglu_mul + quantize_q8 4096 x 768 (two launches)", "us": round(chain, 2),
                "GBs": round((4 * big * 4 + big // 32 * 40) / chain / 1e3, 0)})
    gu = dev(rng.standard_normal((rows, 2 * ff)).astype(np.float32))
    out.append({"op": "moe_geglu_q8 4096 x 768", "us": round(t(lambda: runtime.moe_geglu_q8(gu, q3, ff, rows, stream)), 2)})
    for r in out:
        log("fused", r)
    return out


HEADLINE_SHAPES = ((5120, 5120), (5120, 34816), (17408, 5120))      # (K, N) of configs[1]
# HBM bytes per launch of the three Q4_K batch-1 launches from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this file, each scaled by the same counter's reading for the set-up
# device-to-device copies of known size (fetch x1.9992, write x1.0).  Counters cannot be read
# live from inside the process, so these are the recorded figures of
# profiles/rein_mv_q4k_b1_decode_shapes.txt, reported only for the configuration they were taken on.
RECORDED_TRAFFIC_BYTES = {(5120, 5120): 15259700, (5120, 34816): 109573400, (17408, 5120): 52919800}
# the kernel each shape runs (rows per wavefront chosen by the library)
HEADLINE_KERNELS = {(5120, 5120): "rein_mv_q4k_r2_b1", (5120, 34816): "rein_mv_q4k_r4_b1", (17408, 5120): "rein_mv_q4k_r2_b1"}


def read_ceiling_us(stream, weights, nbytes):
    """Microseconds per launch of the plain read-only kernel (16 B per lane, nothing else) over the same
    rotation of buffers, in a graph of back-to-back launches like the matvecs: what a read of these bytes
    takes on this machine.  Best of three grid sizes."""
    import ctypes as C
    f = hip.Module.builtin().function("rein_measure_read16")
    sink = hip.DeviceBuf(16)
    best = None
    for grid in (2048, 4096, 8192):
        sec = time_graph(stream, lambda: [f.launch((grid, 1, 1), (256, 1, 1), 0, stream,
                                                   [C.c_void_p(b.ptr), C.c_size_t(nbytes // 16), C.c_void_p(sink.ptr)])
                                          for b in weights], len(weights))
        best = sec if best is None else min(best, sec)
    return best * 1e6


def extras_mmq_launch_forms(stream):
    """rein_mmq_xq8_ws picks one of four launches (rein_mmq_form_ws: 0 plain int8, 1 fp6 one token group per workgroup,
    2 fp6 split-tail, 3 int8 split-tail).  Here each is forced through the library's options on model shapes other
    than BASELINE's and timed beside the library's own choice: `lib_over_best` is what the choice leaves behind.
    Forced options fall back where a form is not valid for the token count (a ragged last token group), so every
    entry carries the form that actually ran."""
    from reinstinct_amd import _lib
    forms = {"int8": {"REIN_MMQ6": "0", "REIN_MMQ_SK": "0"}, "int8_split_tail": {"REIN_MMQ6": "0", "REIN_MMQ_SK": "2"},
             "fp6_mixed": {"REIN_MMQ6_FROM": "1", "REIN_MMQ6_SK": "0"}, "fp6_split_tail": {"REIN_MMQ6_FROM": "1", "REIN_MMQ6_SK": "2"}}
    names = sorted({k for f in forms.values() for k in f})
    shapes = {rein.Q4_K: [(5120, 17408), (17408, 5120), (4096, 14336), (14336, 4096), (8192, 28672), (8192, 10240), (4096, 6144), (5120, 13824)],
              rein.Q6_K: [(5120, 17408), (17408, 5120), (4096, 14336), (8192, 10240)],
              rein.Q8_0: [(5120, 17408), (17408, 5120), (4096, 14336), (8192, 10240)]}
    out = []
    for f, shape_list in shapes.items():
        for k, n in shape_list:
            packed = tiled_weights(f, k, n, seed=5)
            ws = [hip.DeviceBuf.from_host(packed) for _ in range(max(3, min(12, (400 << 20) // packed.nbytes + 1)))]
            for m in (128, 256, 384, 512, 768, 1024, 2048):
                x = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
                dx, dq, dy = hip.DeviceBuf.from_host(x), hip.DeviceBuf(m * (k // 32) * 40), hip.DeviceBuf(m * n * 4)
                runtime.quantize_q8(dx, dq, k, m, stream)

                def timed():
                    wsb = runtime.mmq_workspace_bytes(f, k, m)
                    wsp = hip.DeviceBuf(wsb) if wsb else None
                    form = runtime.mmq_form_ws(f, k, n, m, wsb)
                    sec = time_graph(stream, lambda: [runtime.mmq_xq8_ws(f, w_, dq, dy, k, n, m, wsp, wsb, stream) for w_ in ws], len(ws), steps=3)
                    return round(sec * 1e6, 1), form

                timed()
                entry = {"fmt": FMT_NAME[f], "K": k, "N": n, "M": m}
                entry["lib_us"], entry["lib_form"] = timed()
                by_form = {}
                try:
                    for name, opts in forms.items():
                        if name.startswith("fp6") and f != rein.Q4_K:
                            continue
                        for o in names:
                            _lib.set_option(o, opts.get(o))
                        us, form = timed()
                        by_form[form] = min(us, by_form.get(form, us))
                finally:
                    for o in names:
                        _lib.set_option(o, None)
                entry["us_by_form"] = {str(a): b for a, b in sorted(by_form.items())}
                entry["lib_over_best"] = round(by_form.get(entry["lib_form"], entry["lib_us"]) / min(by_form.values()), 3)
                out.append(entry)
                log("mmq forms", entry)
                del dx, dq, dy
            del ws
    return out


def extras_barrier_cost(stream):
    """What a barrier across the workgroups of one launch costs through device memory (rein_measure_barrier, a
    measurement kernel in the code object: one workgroup per CU, nothing but the barrier, every wait bounded),
    per launch in a graph of 32 launches, beside an empty launch of the same shape: the price a persistent
    kernel would pay where the graph pays a launch boundary."""
    import ctypes as C
    f = hip.Module.builtin().function("rein_measure_barrier")
    out = hip.DeviceBuf.from_host(np.zeros(2, np.uint32))
    res = {}
    for grid, block in ((256, 1024), (256, 64), (64, 1024)):
        for mode, name in ((0, "empty"), (1, "every_workgroup_polls_every_flag"), (2, "one_gathers_the_others_poll_a_word"),
                           (3, "the_same_without_the_l2_write_back")):
            sec = time_graph(stream, lambda: [f.launch((grid, 1, 1), (block, 1, 1), 0, stream,
                                                       [C.c_uint(mode), C.c_uint(1 << 16), C.c_void_p(out.ptr)]) for _ in range(32)], 32)
            res[f"{grid}x{block}_{name}_us"] = round(sec * 1e6, 2)
    gave_up = int(out.to_host(np.uint32)[1])
    res["a_wait_gave_up"] = bool(gave_up)
    log("barrier cost", res)
    return res


def decode_sweep(stream, steps):
    """BASELINE configs[1] as a sweep: Q4_K and Q6_K over the three decode shapes at batch 1, 2, 4, 8, the
    other four formats at the gate+up shape; every cell over its own rotation of > 512 MB of weights.
    `vs_batch1` is the cell's time over the batch-1 time of the same format and shape."""
    plan = [(f, HEADLINE_SHAPES) for f in (rein.Q4_K, rein.Q6_K)]
    plan += [(f, ((5120, 34816),)) for f in (rein.Q4_0, rein.Q5_K, rein.Q8_0, rein.IQ4_XS)]
    out = []
    for f, shapes in plan:
        for (k, n) in shapes:
            rot = weight_rotation(tiled_weights(f, k, n, seed=5))
            base = None
            for b in (1, 2, 4, 8):
                c = MatvecCase(f, k, n, b, stream, seed=5, weights=rot)
                _, sl = c.time(max(3, steps // 4), 1)
                base = sl if base is None else base
                g = c.bytes_per_launch / sl / 1e9
                out.append({"fmt": FMT_NAME[f], "K": k, "N": n, "batch": b, "us": round(sl * 1e6, 2), "GBs": round(g, 0),
                            "frac_of_hbm_peak": round(g / HBM_PEAK_GBS, 3), "vs_batch1": round(sl / base, 3),
                            "kernel": runtime.matvec_kernel_name(f, k, n, b)})
                log("decode sweep", out[-1])
                del c
            del rot
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--sweep", action="store_true", help="also time the format x shape x batch sweep of configs[1]")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-mmq", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the objects of BASELINE configs[2..4] (MMQ formats x M, MoE expert FFN, decode weight stream)")
    ap.add_argument("--configs", default="",
                    help="comma-separated names of the `configs` objects to run instead of all of them (a profiler run that "
                         "wants one leg: rocprofv3 cannot follow the whole line, see settle())")
    ap.add_argument("--extras", nargs="?", const="all", default="",
                    help="also time the fused producers, the remaining matvec sites, the decode FFN chain, the barrier cost and "
                         "the launch forms of the prefill GEMM; with a comma-separated list of their names, only those")
    ap.add_argument("--fmt", default="q4_k")
    ap.add_argument("--batch", type=int, default=1)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); the path has no collectives",
              file=sys.stderr)
        sys.exit(2)

    init()
    hip.set_device(0)
    stream = hip.Stream()
    fmt = rein.FORMATS[args.fmt]

    cases = [MatvecCase(fmt, k, n, args.batch, stream, seed=1234 + i) for i, (k, n) in enumerate(HEADLINE_SHAPES)]
    settle(lambda: [c.launch(w) for c in cases for w in c.weights], stream)
    for c in cases:
        for _ in range(args.warmup):
            c.step()
    stream.synchronize()
    # K steps, each = one pass of every shape; one event pair per shape and step so
    # the per-kernel launch time is measured on the launch stream itself
    marks = [[(hip.Event(), hip.Event()) for _ in cases] for _ in range(args.steps)]
    t0, t1 = hip.Event(), hip.Event()
    t0.record(stream)
    for k in range(args.steps):
        for c, (e0, e1) in zip(cases, marks[k]):
            e0.record(stream)
            c.step()
            e1.record(stream)
    t1.record(stream)
    t1.synchronize()
    total_s = t0.elapsed_ms(t1) * 1e-3
    shapes = []
    for i, c in enumerate(cases):
        sec = sum(marks[k][i][0].elapsed_ms(marks[k][i][1]) for k in range(args.steps)) * 1e-3
        per_launch = sec / (args.steps * c.n_buf)
        gbs = c.bytes_per_launch / per_launch / 1e9
        shapes.append({"K": c.in_dim, "N": c.out_dim, "us_per_launch": round(per_launch * 1e6, 3),
                       "GBs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                       "bytes_per_launch": c.bytes_per_launch, "launches_per_step": c.n_buf})
        log(f"matvec {args.fmt} {c.in_dim}->{c.out_dim} b{args.batch}: {per_launch * 1e6:.2f} us/launch, {gbs:.0f} GB/s "
            f"({c.n_buf} buffers/step)")
    step_bytes = sum(c.bytes_per_launch * c.n_buf for c in cases)
    value = step_bytes * args.steps / total_s / 1e9
    is_headline = fmt == rein.Q4_K and args.batch == 1
    # the roofline object describes the launch the target is quoted on: K = 5120 -> N = 5120 (it is also the
    # launch furthest from the roof); the other two shapes and the step aggregate are in config.shapes / value
    dom = shapes[0]
    for sh, c in zip(shapes, cases):
        sh["read_only_ceiling_us"] = round(read_ceiling_us(stream, c.weights, c.bytes_per_launch), 3)
        sh["frac_of_read_only_ceiling"] = round(sh["read_only_ceiling_us"] / sh["us_per_launch"], 3)
        if is_headline:
            sh["kernel"] = HEADLINE_KERNELS[(sh["K"], sh["N"])]
            sh["traffic_recorded"] = RECORDED_TRAFFIC_BYTES[(sh["K"], sh["N"])]
        log(f"read-only kernel over the same {sh['bytes_per_launch']} bytes: {sh['read_only_ceiling_us']} us")

    out = {
        "metric": "Q4_K decode matvec HBM GB/s (% of peak) + MMQ pp512 int8 TOPS, 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "clock_settle_ms": round(CLOCK_SETTLE_S * 1e3), "ms_per_step": round(total_s / args.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8 (int8 dot4, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"{args.fmt} repacked-v2 decode matvec, batch {args.batch}, BASELINE configs[1] shapes "
                               "5120->5120, 5120->34816 (fused gate+up), 17408->5120; value = total algorithmic bytes "
                               "/ total time; step = one pass of each shape over its rotation of distinct weight buffers",
                   "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2), "shapes": shapes},
        "roofline": {"bound": "hbm", "achieved": dom["GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom["frac_of_hbm_peak"], "traffic": dom.get("traffic_recorded"),
                     "traffic_source": "recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file "
                                       "(profiles/rein_mv_q4k_b1_decode_shapes.txt), not read in this run; the other two "
                                       "shapes in config.shapes[].traffic_recorded" if is_headline else None,
                     "kernel": f"{HEADLINE_KERNELS[(dom['K'], dom['N'])] if is_headline else 'decode matvec'} "
                               f"(K={dom['K']} -> N={dom['N']}, the shape the 70 % target is quoted on)",
                     "us_per_launch": dom["us_per_launch"], "algorithmic_bytes_per_launch": dom["bytes_per_launch"],
                     "read_only_ceiling_us": dom["read_only_ceiling_us"],
                     "step_aggregate_frac": round(value / HBM_PEAK_GBS, 4)},
    }

    if is_headline:
        # the same kernel and contraction (Q4_K, K = 5120) where one launch is long enough for the
        # launch / ramp time not to matter: the vocabulary-sized N = 151936, 450 MB per launch
        k, n = 5120, 151936
        p4 = tiled_weights(rein.Q4_K, k, n, seed=4)
        d4 = [hip.DeviceBuf.from_host(p4) for _ in range(2)]
        xq = hip.DeviceBuf(k // 32 * 40)
        runtime.quantize_q8(hip.DeviceBuf.from_host(np.random.default_rng(1).standard_normal((1, k)).astype(np.float32)),
                            xq, k, 1, stream)
        dy = hip.DeviceBuf(n * 4)
        sec = time_graph(stream, lambda: [runtime.matvec_xq8(rein.Q4_K, b, xq, dy, k, n, stream) for b in d4], 2)
        nbytes = p4.nbytes + k // 32 * 40 + n * 4
        out["large_n"] = {"workload": "Q4_K decode matvec K=5120 -> N=151936, batch 1 (same kernel, 450 MB per launch)",
                          "us_per_launch": round(sec * 1e6, 1), "GBs": round(nbytes / sec / 1e9, 0),
                          "frac_of_hbm_peak": round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 4)}
        log("large N:", out["large_n"])
        del d4, p4

    if not args.no_mmq:
        mm = MmqCase(rein.Q4_K, 512, 5120, 17408, stream, seed=77)
        sec = mm.time(max(4, min(args.steps, 20)), 2)
        tops = mm.ops / sec / 1e12
        log(f"mmq q4_k 512x5120x17408: {sec * 1e6:.1f} us, {tops:.1f} TOPS")
        out["mmq"] = {"workload": "Q4_K MMQ prefill GEMM 512x5120x17408 (BASELINE configs[2])",
                      "us_per_launch": round(sec * 1e6, 2), "value": round(tops, 2), "unit": "int8 TOPS",
                      "roofline": {"bound": "mfma", "achieved": round(tops, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                   "frac": round(tops / INT8_PEAK_TOPS, 4),
                                   "kernel": mmq_kernel_name(rein.Q4_K, 5120, 17408, 512),
                                   "counters_recorded": {"mfma_busy_frac_of_simd_cycles": 0.331, "valu_issue_frac": 0.479,
                                                         "hbm_fetch_bytes": 148.6e6, "input_bytes": 57.1e6,
                                                         "source": "rocprofv3 --pmc runs of this file, profiles/rein_mmq6_q4k_sk_pp512.txt; "
                                                                   "not read in this run"}}}
        del mm

    if not args.no_configs:
        legs = {"decode_sweep_configs1": lambda: decode_sweep(stream, args.steps), "mmq_configs2": lambda: extras_mmq(stream),
                "mmq_short_prompts": lambda: extras_mmq_small(stream),
                "moe_configs3": lambda: extras_moe(stream), "moe_configs3_one_token": lambda: extras_moe_decode(stream),
                "decode_stream_configs4": lambda: extras_decode_stream(stream),
                "decode_layer_separate_tensors": lambda: extras_decode_layer_separate(stream)}
        wanted = [n for n in args.configs.split(",") if n] if args.configs else list(legs)
        unknown = [n for n in wanted if n not in legs]
        if unknown:
            print(f"bench.py: --configs knows {', '.join(legs)}; got {', '.join(unknown)}", file=sys.stderr)
            sys.exit(2)
        out["configs"] = {n: legs[n]() for n in legs if n in wanted}

    if args.sweep:
        sweep = []
        for f in (rein.Q4_0, rein.Q4_K, rein.Q5_K, rein.Q6_K, rein.Q8_0, rein.IQ4_XS, rein.IQ3_S):
            for (k, n) in HEADLINE_SHAPES:
                _, packed = synth_weights(f, k, n, seed=5)
                for b in (1, 2, 4, 8):
                    c = MatvecCase(f, k, n, b, stream, seed=5, packed=packed)
                    _, sl = c.time(max(3, args.steps // 4), 1)
                    g = c.bytes_per_launch / sl / 1e9
                    sweep.append({"fmt": FMT_NAME[f], "K": k, "N": n, "batch": b, "us": round(sl * 1e6, 2),
                                  "GBs": round(g, 0), "frac": round(g / HBM_PEAK_GBS, 3)})
                    log(sweep[-1])
                    del c
        out["sweep"] = sweep

    if args.extras:
        legs = {"fused_producers": extras_fused, "other_matvec_sites": extras_ondisk, "decode_ffn_chain": extras_decode_ffn,
                "barrier_cost": extras_barrier_cost, "mmq_launch_forms": extras_mmq_launch_forms}
        wanted = list(legs) if args.extras == "all" else [n for n in args.extras.split(",") if n]
        unknown = [n for n in wanted if n not in legs]
        if unknown:
            print(f"bench.py: --extras knows {', '.join(legs)}; got {', '.join(unknown)}", file=sys.stderr)
            sys.exit(2)
        out["extras"] = {n: legs[n](stream) for n in legs if n in wanted}

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(fmt, 5120, 5120, seed=1234)
        log("cpu baseline:", out["cpu_baseline"])
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
