#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only a,b,...] [--no-cpu]

Headline (`value`): Q4 qmv at M=1, K=N=4096 (group 64, f16) in GB/s of algorithmic bytes.  A step is a
train of TRAIN (200) back-to-back launches of the kernel on one stream; the weights are cycled over enough
distinct sets (> 1 GiB) that every launch streams from HBM instead of the L2 / Infinity Cache.  W warm-up
steps and an untimed settle phase come first, then exactly K steps are timed with HIP events on that stream.
All inputs are resident in HBM before the timed region.  The other benchmark configurations (qmv at N=9216,
Q4 qmm at M=128/512, Q8 bf16 qmm, gather_qmm, the MoE block), the machine floors (empty launch, plain read,
MFMA-only loop) and the CPU baselines are reported under "extra" / "cpu_baseline".  One JSON line on stdout.
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
MFMA_F16_PEAK_TF = 2500.0  # dense f16 / bf16 MFMA
TRAIN = 200                # launches per step of the matmul sections
GEMM_MIN_LAUNCHES = 10000  # the clock needs tens of milliseconds of sustained matrix work to settle
SETTLE_S = 0.25            # untimed run of the workload in front of every timed region


def measured_profiles():
    """Figures that only a profiler run can give, read from the committed rocprofv3 summaries under profiles/
    (counters and traces cannot be read from inside the process): `traffic_bytes_per_launch <key> <bytes>` (FETCH_SIZE
    + WRITE_SIZE of two counter runs of this script, each scaled by what it reads for the plain copy this script also
    launches) and `kernel_trace_avg_us <key> <us>` (average kernel duration in a kernel trace of this script).  Every
    figure is returned with the file it came from and that file's `measured_at` line, so a stale figure can be told."""
    out = {"traffic": {}, "trace_us": {}}
    pdir = os.path.join(ROOT, "profiles")
    if os.path.isdir(pdir):
        for name in sorted(os.listdir(pdir)):
            if not name.endswith(".txt"):
                continue
            text = open(os.path.join(pdir, name)).read()
            at = re.search(r"^measured_at\s+(.+)$", text, re.M)
            src = {"file": f"profiles/{name}", "measured_at": at.group(1).strip() if at else None}
            for m in re.finditer(r"^traffic_bytes_per_launch\s+(\S+)\s+(\d+)", text, re.M):
                out["traffic"][m.group(1)] = dict(src, bytes=int(m.group(2)))
            for m in re.finditer(r"^kernel_trace_avg_us\s+(\S+)\s+([0-9.]+)", text, re.M):
                out["trace_us"][m.group(1)] = dict(src, us=float(m.group(2)))
    return out


def matmul_bytes(m, n, k, bits, gs=64, act_bytes=2):
    """Algorithmic bytes of one quantized matmul: packed weights + f16 scales and biases +
    activations in + f16 out."""
    return n * k * bits // 8 + 2 * (n * k // gs) * 2 + m * k * act_bytes + m * n * 2


def make_weight(rng, n, k, bits, lead=()):
    lo, hi = (0.005, 0.02) if bits <= 4 else (0.0005, 0.002)
    words = rng.integers(0, 2**32, size=tuple(lead) + (n, k * bits // 32), dtype=np.uint32)
    s = rng.uniform(lo, hi, size=tuple(lead) + (n, k // 64)).astype(np.float16)
    b = (-(2.0 ** (bits - 1)) * s.astype(np.float32)).astype(np.float16)
    return words, s, b


class Timer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self, rt):
        self.rt = rt
        self.stream = rt.Stream()
        self.e0, self.e1 = rt.Event(), rt.Event()
        self.cap = 0  # --max-launches: also bounds the trains of the settle phase

    def run(self, fn, launches, warmup, chunk=TRAIN, uncapped=False):
        """fn(c) enqueues c launches.  Warm-up, an untimed settle phase of about SETTLE_S, then `launches`
        launches between two events; returns milliseconds per launch."""
        if self.cap > 0 and not uncapped:
            launches, warmup, chunk = min(launches, self.cap), min(warmup, self.cap), min(chunk, self.cap)
        fn(max(1, warmup))
        self.stream.sync()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < (SETTLE_S if self.cap == 0 else 0.0):
            fn(chunk)
            self.stream.sync()
        self.e0.record(self.stream)
        done = 0
        while done < launches:  # enqueued train by train: the queue never runs dry, the host stays ahead
            c = min(chunk, launches - done)
            fn(c)
            done += c
        self.e1.record(self.stream)
        self.e1.sync()
        self.stream.sync()
        return self.e0.elapsed_ms(self.e1) / launches


def bench_matmul(ops, rt, timer, rng, m, n, k, bits, x_dtype, launches, warmup, min_total_bytes, check=True, kernel=0,
                 check_rows=None, graph=False, queued_trains=0, gemm_layout=False):
    from oracle import model
    wbytes = n * k * bits // 8 + 4 * (n * k // 64)
    n_sets = max(1, -(-min_total_bytes // wbytes))
    base = make_weight(rng, n, k, bits)
    qws = [ops.QuantizedWeight.from_numpy(*base, 64, bits)]
    for i in range(1, n_sets):  # distinct buffers; contents rolled so that sets differ
        qws.append(ops.QuantizedWeight.from_numpy(np.roll(base[0], i, axis=0), np.roll(base[1], i, axis=0),
                                                  np.roll(base[2], i, axis=0), 64, bits))
    if gemm_layout:  # every set also gets the tile-contiguous copy for the K-split GEMMs (a second buffer of the same size)
        for q in qws:
            if not q.use_gemm_layout(True):
                raise RuntimeError("no GEMM layout for this weight")
    xf = rng.standard_normal((m, k)).astype(np.float32)
    if x_dtype == "bf16":
        xh = model.f32_to_bf16_bits(xf)
        xd = rt.DeviceBuffer.from_numpy(xh, rt.BF16)
        x64 = model.bf16_bits_to_f32(xh).astype(np.float64)
    else:
        xh = xf.astype(np.float16)
        xd = rt.DeviceBuffer.from_numpy(xh)
        x64 = xh.astype(np.float64)
    outs = [rt.DeviceBuffer((m, n), rt.F16) for _ in range(min(n_sets, 8))]
    if queued_trains:
        # Every train is enqueued behind a stall kernel (a few milliseconds of matrix instructions on a quarter of the
        # CUs), so the whole train sits in the queue before its first kernel starts and runs back to back whatever a
        # launch costs the host - under a tracer too, where the host needs longer per launch than the kernel runs.
        L, sink = rt.lib(), rt.DeviceBuffer((64,), rt.U32)
        total_ms = 0.0
        for _ in range(queued_trains + 1):
            rt.check(L.rmlx_hip_measure_floor(rt.FLOOR_MFMA, None, 64, 0, 8000, sink.ptr, 1, timer.stream.handle))
            timer.e0.record(timer.stream)
            ops.qmm_encode_many(qws, xd, outs, TRAIN, stream=timer.stream, kernel=kernel)
            timer.e1.record(timer.stream)
            timer.e1.sync()
            total_ms += timer.e0.elapsed_ms(timer.e1)
            if _ == 0:
                total_ms = 0.0  # (the first train is warm-up)
        launches = queued_trains * TRAIN
        ms = total_ms / launches
    elif graph:  # the train is recorded once and replayed: no host work per launch (kernel nodes only)
        with rt.Graph.record(timer.stream) as g:
            ops.qmm_encode_many(qws, xd, outs, TRAIN, stream=timer.stream, kernel=kernel)

        def replay(c):
            for _ in range(max(1, c // TRAIN)):
                g.launch()
        launches = max(TRAIN, launches // TRAIN * TRAIN)
        if timer.cap > 0:
            launches = TRAIN
        ms = timer.run(replay, launches, warmup, chunk=TRAIN, uncapped=True)
    else:
        ms = timer.run(lambda c: ops.qmm_encode_many(qws, xd, outs, c, stream=timer.stream, kernel=kernel), launches, warmup)
    res = {"us": ms * 1e3, "launches": launches, "n_weight_sets": n_sets,
           "bytes": matmul_bytes(m, n, k, bits, act_bytes=2), "flops": 2 * m * n * k}
    res["gbs"] = res["bytes"] / (ms * 1e-3) / 1e9
    res["hbm_frac"] = res["gbs"] / HBM_PEAK_GBS
    res["tflops"] = res["flops"] / (ms * 1e-3) / 1e12
    if check:  # parity of the timed configuration against the oracle, on weight set 0
        ops.qmm_encode_many(qws[:1], xd, outs[:1], 1, stream=timer.stream, kernel=kernel)
        timer.stream.sync()
        rows = slice(None) if check_rows is None else slice(0, check_rows)  # (of very tall weights: the first rows)
        ref = model.qmm(x64, base[0][rows], base[1][rows], base[2][rows], 64, bits)
        err = float(np.abs(outs[0].numpy().astype(np.float64)[:, rows] - ref).max())
        res["max_err"], res["tol"] = err, model.tolerance(ref)
        res["pass"] = bool(err <= res["tol"])
    return res


def bench_moe(ops, rt, timer, rng, T, calls, experts, bits=4):
    from oracle import model
    gate_up, down, gh, dh = experts
    x = rng.standard_normal((T, 4096)).astype(np.float16)
    logits = rng.standard_normal((T, 128)).astype(np.float32)
    xd, ld = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer.from_numpy(logits)
    out = rt.DeviceBuffer((T, 4096), rt.F16)

    def run(c):
        for _ in range(c):
            ops.moe_forward(gh, None, dh, xd, ld, 8, stream=timer.stream, out=out)

    ms = timer.run(run, calls, 10, chunk=20)
    idx, w, _, _ = model.topk_route(logits, 8)
    distinct = len(np.unique(idx))
    nbytes = distinct * (18874368 * bits // 8 + 1179648) + T * 4096 * 2 * 2 + T * 128 * 4
    res = {"us": ms * 1e3, "calls": calls, "distinct_experts": distinct, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9,
           "flops": 2 * 8 * T * (4096 * 3072 + 1536 * 4096)}
    toks = np.arange(min(T, 2))
    sel = (toks[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    gate = tuple(a[:, :1536] for a in gate_up)
    up = tuple(a[:, 1536:] for a in gate_up)
    ref = model.moe_forward(x[toks], idx[sel], w[sel], gate, up, down, 64, 8, bits=bits)
    err = float(np.abs(out.numpy()[toks].astype(np.float64) - ref).max())
    res["max_err"], res["tol"], res["pass"] = err, model.tolerance(ref), bool(err <= model.tolerance(ref))
    return res


def bench_moe_shape(ops, rt, timer, rng, T, calls, gate_up, down, gh, dh, E, top_k, D, I):
    """The routed block over other expert shapes (E experts, top_k picks, hidden D, intermediate I; 4-bit, group 64): time
    per call, weight bandwidth over the distinct experts of the batch, the first token against the oracle."""
    from oracle import model
    x = rng.standard_normal((T, D)).astype(np.float16)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    xd, ld = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer.from_numpy(logits)
    out = rt.DeviceBuffer((T, D), rt.F16)

    def run(c):
        for _ in range(c):
            ops.moe_forward(gh, None, dh, xd, ld, top_k, stream=timer.stream, out=out)

    ms = timer.run(run, calls, 3, chunk=10)
    idx, w, _, _ = model.topk_route(logits, top_k)
    distinct = len(np.unique(idx))
    nbytes = distinct * (3 * I * D // 2 + 3 * (I * D // 64) * 4)
    gate, up = tuple(a[:, :I] for a in gate_up), tuple(a[:, I:] for a in gate_up)
    ref = model.moe_forward(x[:1], idx[:top_k], w[:top_k], gate, up, down, 64, top_k)
    err = float(np.abs(out.numpy()[:1].astype(np.float64) - ref).max())
    return {"us": ms * 1e3, "calls": calls, "distinct_experts": distinct, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9,
            "flops": 2 * top_k * T * 3 * I * D, "max_err": err, "tol": model.tolerance(ref), "pass": bool(err <= model.tolerance(ref))}


def bench_gather(ops, rt, timer, rng, batch, mpb, gh, gate_up, calls):
    """gather_qmm over the stacked gate/up weights of the MoE configuration (every batch entry names an expert)."""
    from oracle import model
    E, n, k = gh.n_experts, gh.out_features, gh.in_features
    idx = rng.integers(0, E, size=batch).astype(np.uint32)
    x = rng.standard_normal((batch, mpb, k)).astype(np.float16)
    xd, idxd = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer.from_numpy(idx)
    out = rt.DeviceBuffer((batch, mpb, n), rt.F16)

    def run(c):
        for _ in range(c):
            ops.gather_qmm(xd, gh.weights_buf, gh.scales_buf, gh.biases_buf, idxd, batch, mpb, n, k, E, 64,
                           stream=timer.stream, out=out)

    ms = timer.run(run, calls, 10, chunk=20)
    distinct = len(np.unique(idx))
    nbytes = distinct * (n * k // 2 + 4 * (n * k // 64)) + batch * mpb * (k + n) * 2
    res = {"us": ms * 1e3, "calls": calls, "distinct_experts": distinct, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9}
    e0 = int(idx[0])
    ref = model.qmm(x[0].astype(np.float64), gate_up[0][e0], gate_up[1][e0], gate_up[2][e0], 64, 4)
    err = float(np.abs(out.numpy()[0].astype(np.float64) - ref).max())
    res["max_err"], res["tol"], res["pass"] = err, model.tolerance(ref), bool(err <= model.tolerance(ref))
    return res


def bench_dequant(ops, rt, timer, rng, fmt, k, n, gs, launches):
    """AWQ / GPTQ INT4 -> f32 dequantisation of one [k, n] matrix (store-bound: 4 bytes out per element).
    Four input sets alternate; the packed inputs are an eighth of the traffic, the f32 output the rest."""
    from oracle import model
    groups = k // gs
    sets = []
    for _ in range(4):
        shape = (k, n // 8) if fmt == "awq" else (k // 8, n)
        qw = rng.integers(0, 2**32, size=shape, dtype=np.uint64).astype(np.uint32)
        qz = rng.integers(0, 2**32, size=(groups, n // 8), dtype=np.uint64).astype(np.uint32)
        sc = rng.uniform(0.001, 0.05, size=(groups, n)).astype(np.float32)
        sets.append((qw, qz, sc, [rt.DeviceBuffer.from_numpy(a) for a in (qw, qz, sc)]))
    out = rt.DeviceBuffer((k, n), rt.F32)

    def launch(i):
        d = sets[i % 4][3]
        if fmt == "awq":
            ops.awq_dequant(d[0], d[1], d[2], k, n, gs, stream=timer.stream, out=out)
        else:
            ops.gptq_dequant(d[0], d[1], d[2], None, k, n, gs, stream=timer.stream, out=out)

    def run(c):
        for i in range(c):
            launch(i)

    ms = timer.run(run, launches, 10, chunk=50)
    nbytes = k * n * 4 + k * n // 2 + groups * n // 2 + groups * n * 4
    launch(0)
    timer.stream.sync()
    qw, qz, sc, _ = sets[0]
    ref = model.awq_dequant(qw, qz, sc, gs) if fmt == "awq" else model.gptq_dequant(qw, qz, sc, None, gs)
    return {"us": ms * 1e3, "launches": launches, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9,
            "hbm_frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "pass": bool(np.array_equal(out.numpy(), ref))}


def bench_floors(rt, timer, launches):
    """What the machine does with nothing but the launch / the loads / the matrix instructions, timed with the same
    events on the same stream as everything else: the figures the achieved fractions are to be read against."""
    L = rt.lib()
    sink = rt.DeviceBuffer((64,), rt.U32)
    st = timer.stream.handle
    floors = {}

    def go(kind, src, nbytes, n_src, iters, count):
        rt.check(L.rmlx_hip_measure_floor(kind, src, nbytes, n_src, iters, sink.ptr, count, st))

    ms = timer.run(lambda c: go(rt.FLOOR_EMPTY, None, 0, 0, 0, c), launches, TRAIN)
    floors["empty_kernel_us"] = ms * 1e3
    for label, nbytes, total in (("9.45MB", 9453568, 1200 << 20), ("21.3MB", 21260288, 1300 << 20),
                                 ("75.5MB", 75505664, 1300 << 20), ("1GiB", 1 << 30, 1 << 30)):
        nbytes = -(-nbytes // 16) * 16
        n_src = max(1, total // nbytes)
        src = rt.DeviceBuffer((n_src * nbytes // 4,), rt.U32)
        rt.check(L.rmlx_hip_memset(src.ptr, 1, n_src * nbytes, None))
        n_launch = launches if nbytes < (64 << 20) else max(20, launches // 20)
        best = None
        for name, kind in (("u2", rt.FLOOR_READ2), ("u4", rt.FLOOR_READ4), ("u8", rt.FLOOR_READ8)):
            ms = timer.run(lambda c: go(kind, src.ptr, nbytes, n_src, 0, c), n_launch, min(TRAIN, n_launch),
                           chunk=min(TRAIN, n_launch))
            r = {"us": ms * 1e3, "gbs": nbytes / (ms * 1e-3) / 1e9, "loads_in_flight_per_lane": int(name[1:])}
            if best is None or r["us"] < best["us"]:
                best = r
            floors[f"read_{label}_{name}_us"] = r["us"]
        best["bytes"], best["copies_cycled"] = nbytes, n_src
        floors[f"read_{label}"] = best
        src.free()
    iters, blocks = 2048, 0
    info_blocks = 2 * rt.device_info()["compute_units"]
    n_mfma = max(20, launches // 20)
    ms = timer.run(lambda c: go(rt.FLOOR_MFMA, None, blocks, 0, iters, c), n_mfma, 5, chunk=20)
    flops = info_blocks * 8 * iters * 16 * 16384
    floors["mfma_loop"] = {"us": ms * 1e3, "tflops": flops / (ms * 1e-3) / 1e12, "workgroups": info_blocks,
                           "frac_of_peak": flops / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TF}
    # the matrix rate with and-or instructions of a 4-bit unpacking on the vector ALU of the same SIMD
    for v in (2, 4, 6, 8):
        ms = timer.run(lambda c: go(rt.FLOOR_MFMA_VALU, None, blocks, v, iters, c), n_mfma, 5, chunk=20)
        floors[f"mfma_loop_with_{v}_valu_per_mfma"] = {"us": ms * 1e3, "tflops": flops / (ms * 1e-3) / 1e12}
    # LDS operand reads: bytes per clock and CU at 8 and 16 waves per CU
    cus, clk = rt.device_info()["compute_units"], rt.device_info()["clock_khz"] * 1e3
    for waves in (8, 16):
        ms = timer.run(lambda c: go(rt.FLOOR_LDS, None, 0, waves, iters, c), n_mfma, 5, chunk=20)
        per_cu = waves * 64 * 128 * iters
        floors[f"lds_read_{waves}_waves"] = {"us": ms * 1e3, "bytes_per_clk_per_cu": per_cu / (ms * 1e-3 * clk),
                                             "tbs_all_cus": per_cu * cus / (ms * 1e-3) / 1e12}
    # reads that hit the L2 of every XCD (all workgroups walk one 2 MB source): the rate at which hits fill the CUs
    nbytes = 2 << 20
    src = rt.DeviceBuffer((nbytes // 4,), rt.U32)
    rt.check(L.rmlx_hip_memset(src.ptr, 1, nbytes, None))
    ms = timer.run(lambda c: go(rt.FLOOR_L2_READ, src.ptr, nbytes, 0, 256, c), n_mfma, 5, chunk=20)
    per_cu = 2 * 256 * 32768
    floors["l2_hit_read"] = {"us": ms * 1e3, "bytes_per_clk_per_cu": per_cu / (ms * 1e-3 * clk),
                             "tbs_all_cus": per_cu * cus / (ms * 1e-3) / 1e12}
    src.free()
    return floors


def _time_reps(fn, budget_s, max_reps=1000):
    fn()  # warm
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or reps >= max_reps:
            return el / reps, reps, el


def cpu_baseline(rng, budget_s, all_configs):
    """The C restatement of the reference's scalar `affine_qmm` / `affine_qmm_q8` (oracle/affine_qmm_ref.c) timed
    on this host: the headline configuration on one thread (the reference's CPU path is single-threaded) and with
    the output columns split over the host threads; beside it, one bounded run of every other configuration."""
    from oracle import model, refpath
    threads = min(16, os.cpu_count() or 1)

    def matmul_case(m, n, k, bits, nthreads, budget):
        words, s, b = make_weight(rng, n, k, bits)
        x = rng.standard_normal((m, k)).astype(np.float16).astype(np.float32)
        wb, s32, b32 = model.words_to_bytes(words), s.astype(np.float32), b.astype(np.float32)
        if nthreads == 1:
            per, reps, el = _time_reps(lambda: refpath.affine_qmm(x, wb, s32, b32, m, n, k, 64, bits), budget)
        else:
            per, reps, el = _time_reps(lambda: refpath.affine_qmm_threads(x, wb, s32, b32, m, n, k, 64, bits, threads=nthreads), budget)
        nb, fl = matmul_bytes(m, n, k, bits), 2 * m * n * k
        return {"ms": per * 1e3, "gbs": nb / per / 1e9, "gflops": fl / per / 1e9, "cores": nthreads,
                "sample": f"{reps} run(s) of the full M={m} N={n} K={k} Q{bits} matmul ({el:.1f} s)"}

    head = matmul_case(1, 4096, 4096, 4, 1, budget_s)
    out = {"value": head["gbs"], "unit": "GB/s", "cores": 1, "kind": "port", "sample": head["sample"],
           "us_per_matmul": head["ms"] * 1e3, "host_cores_available": os.cpu_count()}
    allc = matmul_case(1, 4096, 4096, 4, threads, budget_s / 4)
    out["all_cores"] = {"value": allc["gbs"], "unit": "GB/s", "cores": threads, "us_per_matmul": allc["ms"] * 1e3,
                        "sample": allc["sample"] + f", columns split over {threads} threads"}
    if not all_configs:
        return out
    cfg = {}
    cfg["config2_q4_qmv_m1_n9216"] = matmul_case(1, 9216, 4096, 4, 1, 2.0)
    cfg["config2_q4_qmv_m8_n9216"] = matmul_case(8, 9216, 4096, 4, 1, 2.0)
    cfg["config3_q4_qmm_m128_4096"] = matmul_case(128, 4096, 4096, 4, threads, 1.0)
    cfg["config3_q4_qmm_m512_4096"] = matmul_case(512, 4096, 4096, 4, threads, 1.0)
    cfg["config4_q8_qmm_m128_n12288"] = matmul_case(128, 12288, 4096, 8, threads, 1.0)
    # config 5: per-expert `affine_qmm` on the gathered rows + SwiGLU + weighted sum.  Only the experts the routing
    # touches are generated (same shapes and distributions as the GPU run); T = 4 on one thread, T = 32 on all.
    for T, nthreads in ((4, 1), (32, threads)):
        logits = rng.standard_normal((T, 128)).astype(np.float32)
        idx, w, _, _ = model.topk_route(logits, 8)
        x = rng.standard_normal((T, 4096)).astype(np.float16).astype(np.float32)
        order, offsets = model.moe_sort(idx, 128)
        used = [e for e in range(128) if offsets[e + 1] > offsets[e]]
        weights = {}
        for e in used:
            gu, dn = make_weight(rng, 3072, 4096, 4), make_weight(rng, 4096, 1536, 4)
            weights[e] = [(model.words_to_bytes(t[0]), t[1].astype(np.float32), t[2].astype(np.float32)) for t in (gu, dn)]

        def mm(xe, trip, n, k):
            if nthreads == 1:
                return refpath.affine_qmm(xe, *trip, xe.shape[0], n, k, 64, 4)
            return refpath.affine_qmm_threads(xe, *trip, xe.shape[0], n, k, 64, 4, threads=nthreads)

        def block():
            out_t = np.zeros((T, 4096), np.float32)
            for e in used:
                pos = order[offsets[e]:offsets[e + 1]]
                xe = np.ascontiguousarray(x[pos // 8])
                gu = mm(xe, weights[e][0], 3072, 4096)
                g, u = gu[:, :1536], gu[:, 1536:]
                h = np.ascontiguousarray((g / (1.0 + np.exp(-g)) * u).astype(np.float32))
                y = mm(h, weights[e][1], 4096, 1536)
                np.add.at(out_t, pos // 8, w[pos][:, None] * y)
            return out_t

        t0 = time.perf_counter()
        block()
        el = time.perf_counter() - t0
        nbytes = len(used) * (18874368 // 2 + 1179648)
        cfg[f"config5_moe_q4_T{T}"] = {"ms": el * 1e3, "gbs": nbytes / el / 1e9, "cores": nthreads,
                                       "sample": f"1 run of the routed block, {len(used)} distinct experts ({el:.1f} s)"}
    out["configs"] = cfg
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50, help=f"timed steps; a step is a train of {TRAIN} launches")
    ap.add_argument("--warmup", type=int, default=10, help="untimed warm-up steps")
    ap.add_argument("--only", default="", help="comma-separated sections: headline, floors, qmv, qmm, dequant, gather, moe, moe8, large; not in the default "
                                           "run: moevariants (the routed block at T = 96 / 128 / 160 under every choice of expert kernels), "
                                           "shapes (dimensions of models in the field that are no multiples of 512)")
    ap.add_argument("--quick", action="store_true", help="headline and floors only, short CPU baseline")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the second headline measurement that replays the train from a recorded graph")
    ap.add_argument("--max-launches", type=int, default=0,
                    help="cap on the launches of every timed run (for hardware-counter runs, where each dispatch is slow)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    sections = set(filter(None, args.only.split(","))) or ({"headline", "floors"} if args.quick else
                                                           {"headline", "floors", "qmv", "qmm", "dequant", "gather", "moe", "moe8", "large"})

    from rmlx_amd import ops, runtime as rt
    rt.init(0)
    info = rt.device_info()
    timer = Timer(rt)
    rng = np.random.default_rng(1001)
    GiB = 1 << 30
    launches, warm = args.steps * TRAIN, args.warmup * TRAIN
    gemm_launches = max(launches, GEMM_MIN_LAUNCHES)
    train_warm = TRAIN
    if args.max_launches > 0:
        launches, warm, gemm_launches = min(launches, args.max_launches), min(warm, args.max_launches), args.max_launches
        train_warm = min(TRAIN, args.max_launches)
        timer.cap = args.max_launches

    def progress(what):  # (a line per section on stderr: long profiler runs are not silent)
        print(f"[bench] {what}", file=sys.stderr, flush=True)
    prof = measured_profiles()

    # ---- headline: Q4 qmv M=1 K=N=4096, weights cycled through > 1 GiB ---------------------------------
    progress("headline")
    head = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "f16", launches, warm, GiB + GiB // 8)
    extra = {"device": info, "launches_per_step": TRAIN, "q4_qmv_m1_4096": head}
    # The same configuration in trains that are fully enqueued before they start (behind a stall kernel): what a kernel
    # trace of this command shows for these launches is the kernel's duration in a train, not that of a lone launch.
    progress("headline, trains enqueued behind a stall kernel")
    extra["q4_qmv_m1_4096_queued_trains"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "f16", launches, TRAIN,
                                                         GiB + GiB // 8, queued_trains=max(5, min(args.steps, 25)))
    if not args.no_graph:
        # The same train recorded once as a graph (kernel nodes only) and replayed: no host work per launch.  (Not under
        # rocprofv3 7.2, whose kernel tracing crashes in hipGraphLaunch: profile runs pass --no-graph.)
        progress("headline, graph replay")
        extra["q4_qmv_m1_4096_graph_replay"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "f16", launches, TRAIN,
                                                            GiB + GiB // 8, graph=True)
    # A plain copy of known size (identity `index_gather`, 128 MiB in, 128 MiB out) so that a counter
    # run of this same command can scale FETCH_SIZE / WRITE_SIZE by what they read for it.
    rows = 16384
    src = rt.DeviceBuffer((rows, 4096), rt.F16)
    ident = rt.DeviceBuffer.from_numpy(np.arange(rows, dtype=np.uint32))
    ops.index_gather(src, ident, stream=timer.stream)
    timer.stream.sync()
    extra["copy_calibration"] = {"kernel": "index_gather_kernel", "read_bytes": rows * 4096 * 2 + rows * 4,
                                 "write_bytes": rows * 4096 * 2}
    del src, ident
    if "floors" in sections:
        progress("floors")
        extra["floors"] = bench_floors(rt, timer, launches)
    if "qmv" in sections:
        progress("qmv")
        extra["q4_qmv_m1_4096_cache_resident"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "f16",
                                                              launches, warm, 0, check=False)
        for m in (1, 4, 8):
            extra[f"q4_qmv_m{m}_n9216"] = bench_matmul(ops, rt, timer, rng, m, 9216, 4096, 4, "f16", launches,
                                                       warm, GiB + GiB // 8, check=(m == 8))
        extra["q4_qmv_m2_4096"] = bench_matmul(ops, rt, timer, rng, 2, 4096, 4096, 4, "f16", launches, warm, GiB + GiB // 8)
        extra["q8_qmv_m1_4096"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 8, "f16", launches, warm, GiB + GiB // 8)
        extra["q2_qmv_m1_4096"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 2, "f16", launches, warm, GiB + GiB // 8)
        # long K, short N: the shapes the reference sends to its split-K GEMV (K > 8192 and N <= 2048)
        extra["q4_qmv_m1_n2048_k16384"] = bench_matmul(ops, rt, timer, rng, 1, 2048, 16384, 4, "f16", launches, warm, GiB + GiB // 8)
    if "large" in sections:
        progress("large")  # launches long enough that start-up cost no longer matters
        big = max(400, launches // 10)
        extra["q4_qmv_m1_n32768"] = bench_matmul(ops, rt, timer, rng, 1, 32768, 4096, 4, "f16", big, train_warm, GiB + GiB // 8)
        extra["q4_qmv_m1_n151936"] = bench_matmul(ops, rt, timer, rng, 1, 151936, 4096, 4, "f16", max(100, big // 4), 20,
                                                  GiB + GiB // 8, check_rows=4096)
    if "qmm" in sections:
        progress("qmm")
        for m in (128, 512, 4096):
            m_launches = gemm_launches if m <= 512 else max(50, gemm_launches // 10)
            r = bench_matmul(ops, rt, timer, rng, m, 4096, 4096, 4, "f16", m_launches, train_warm, GiB + GiB // 8)
            r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
            extra[f"q4_qmm_m{m}_4096"] = r
        # the same with the optional tile-contiguous copy of the weights (rmlx_hip_qweight_set_gemm_layout)
        r = bench_matmul(ops, rt, timer, rng, 128, 4096, 4096, 4, "f16", gemm_launches, train_warm, GiB + GiB // 8, gemm_layout=True)
        r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
        extra["q4_qmm_m128_4096_gemm_layout"] = r
        for name, kern in (("q8_qmm_bf16_m128_n12288", rt.KERNEL_AUTO), ("q8_qmm_bf16_m128_n12288_bf16_mfma", rt.KERNEL_QMM_BF16)):
            r = bench_matmul(ops, rt, timer, rng, 128, 12288, 4096, 8, "bf16", gemm_launches, train_warm, GiB + GiB // 8, kernel=kern)
            r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
            extra[name] = r
        r = bench_matmul(ops, rt, timer, rng, 128, 12288, 4096, 8, "bf16", gemm_launches, train_warm, GiB + GiB // 8, gemm_layout=True)
        r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
        extra["q8_qmm_bf16_m128_n12288_gemm_layout"] = r
    if "shapes" in sections:
        # Dimensions of models in the field that are no multiples of 512 (not BASELINE configurations): dense matmuls with K in
        # whole blocks of 128 / 64 and short rows of tall matrices, and the routed block over expert shapes with such an
        # intermediate size.  One line per (shape, rows) / (shape, tokens).
        progress("shapes")
        few = max(60, launches // 30)
        for n, k, ms in ((4096, 11008, (1, 8, 64, 512)), (9728, 896, (1, 2, 24)), (151936, 896, (1,)), (13824, 1152, (16, 512)),
                         (4096, 2880, (8, 64, 512))):
            for m in ms:
                extra[f"shape_q4_n{n}_k{k}_m{m}"] = bench_matmul(ops, rt, timer, rng, m, n, k, 4, "f16", few, 10, GiB // 4, check_rows=256)
        extra["shape_q4_n4096_k4096_m1_bf16_rows"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "bf16", launches, warm, GiB + GiB // 8)
        for name, E, top_k, D, I in (("e128_top8_d2048_i768", 128, 8, 2048, 768), ("e64_top6_d2048_i1408", 64, 6, 2048, 1408),
                                     ("e16_top2_d4096_i6400", 16, 2, 4096, 6400), ("e32_top4_d2880_i2880", 32, 4, 2880, 2880)):
            one_gu, one_dn = make_weight(rng, 2 * I, D, 4, lead=(1,)), make_weight(rng, D, I, 4, lead=(1,))
            gu = tuple(np.ascontiguousarray(np.broadcast_to(a, (E,) + a.shape[1:])) for a in one_gu)  # (one random expert repeated)
            dn = tuple(np.ascontiguousarray(np.broadcast_to(a, (E,) + a.shape[1:])) for a in one_dn)
            gq, dq = ops.QuantizedWeight.from_numpy(*gu, 64, 4), ops.QuantizedWeight.from_numpy(*dn, 64, 4)
            for T in (1, 4, 32, 128, 512, 2048):
                extra[f"shape_moe_q4_{name}_T{T}"] = bench_moe_shape(ops, rt, timer, np.random.default_rng(700 + T), T, 40 if T <= 128 else 12,
                                                                     gu, dn, gq, dq, E, top_k, D, I)
            del gq, dq, gu, dn
    if "dequant" in sections:
        progress("dequant")
        for fmt in ("awq", "gptq"):
            extra[f"{fmt}_dequant_4096x4096_gs128"] = bench_dequant(ops, rt, timer, rng, fmt, 4096, 4096, 128, max(200, launches // 10))
    if sections & {"gather", "moe", "moevariants"}:
        progress("gather / moe")
        gate_up = make_weight(rng, 3072, 4096, 4, lead=(128,))
        down = make_weight(rng, 4096, 1536, 4, lead=(128,))
        experts = (gate_up, down, ops.QuantizedWeight.from_numpy(*gate_up, 64, 4),
                   ops.QuantizedWeight.from_numpy(*down, 64, 4))
        calls = max(200, launches // 10)
        if "gather" in sections:
            for batch, mpb in ((32, 1), (32, 8), (32, 64)):
                r = bench_gather(ops, rt, timer, rng, batch, mpb, experts[2], gate_up, calls)
                r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
                extra[f"gather_qmm_q4_b{batch}_m{mpb}"] = r
        if "moe" in sections:
            for T in (1, 4, 8, 32, 128, 512, 2048):  # from 10 rows per expert on average on the grouped MFMA GEMM
                r = bench_moe(ops, rt, timer, rng, T, calls if T <= 128 else max(50, calls // 4), experts)
                r["tflops"] = r["flops"] / (r["us"] * 1e-6) / 1e12
                r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
                r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
                extra[f"moe_q4_T{T}"] = r
        if "moevariants" in sections:
            # The routed block at 6 / 8 / 10 rows per expert with every choice of expert kernels (for kernel traces:
            # which projection costs what under which kernel).  (label, GEMM threshold, streaming kernel selector)
            variants = (("kplit_8row_chunks", 0, 1), ("wave_per_tile_8row_chunks", 0, 2), ("wave_per_tile_16row_chunks", 0, 3),
                        ("hybrid_kplit_gate_up_wave_down", 0, 4), ("split_by_rows_kplit_and_16row", 0, 5), ("grouped_gemm", 1, 0),
                        ("library_choice", None, 0))
            for T in (96, 128, 160):
                for label, min_rows, kind in variants:
                    # (a threshold of 1 forces the GEMM; its tile height follows the average rows per expert: 16-row tiles
                    # at T = 96, 32-row tiles at T = 128 and 160)
                    # (an empty marker kernel in front of every measurement: a kernel trace is split at these)
                    rt.check(rt.lib().rmlx_hip_measure_floor(rt.FLOOR_EMPTY, None, 0, 0, 0, None, 1, timer.stream.handle))
                    prev_rows = experts[2].set_expert_gemm_min_rows(0)
                    experts[2].set_expert_gemm_min_rows(prev_rows if min_rows is None else min_rows)
                    prev_kind = experts[2].set_expert_stream_kernel(kind)
                    try:
                        r = bench_moe(ops, rt, timer, rng, T, max(100, calls // 2), experts)
                    finally:
                        experts[2].set_expert_gemm_min_rows(prev_rows)
                        experts[2].set_expert_stream_kernel(prev_kind)
                    r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
                    extra[f"moe_q4_T{T}_{label}"] = r
        del experts, gate_up, down
    if "moe8" in sections:
        progress("moe8")
        gate_up = make_weight(rng, 3072, 4096, 8, lead=(128,))
        down = make_weight(rng, 4096, 1536, 8, lead=(128,))
        experts = (gate_up, down, ops.QuantizedWeight.from_numpy(*gate_up, 64, 8),
                   ops.QuantizedWeight.from_numpy(*down, 64, 8))
        calls = max(200, launches // 10)
        for T in (4, 32, 512):
            r = bench_moe(ops, rt, timer, rng, T, calls if T <= 128 else max(50, calls // 4), experts, bits=8)
            r["tflops"] = r["flops"] / (r["us"] * 1e-6) / 1e12
            r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
            extra[f"moe_q8_T{T}"] = r
        del experts, gate_up, down

    step_ms = head["us"] * TRAIN / 1e3
    line = {
        "metric": "Q4 qmv HBM GB/s (M=1, K=N=4096)",
        "value": head["gbs"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"Q4 qmv M=1 K=4096 N=4096 group_size=64 f16 activations; one step = {TRAIN} back-to-back launches, "
                               f"{head['n_weight_sets']} distinct weight sets cycled (HBM-resident, > 1 GiB)",
                   "launches_per_step": TRAIN, "parity_max_err": head.get("max_err"), "parity_tol": head.get("tol")},
        "roofline": {"bound": "hbm", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["gbs"] / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "qmv_m1_kernel", "bytes_per_launch": head["bytes"], "avg_launch_us": head["us"]},
    }

    def annotate(roof, key, algorithmic, peak_per_us):
        """Adds what the committed profiler summaries hold for this kernel: HBM traffic per launch and the average
        kernel duration of a kernel trace (with the fraction it gives), each with its source file."""
        t = prof["traffic"].get(key)
        if t is not None:
            roof["traffic"], roof["traffic_source"] = t["bytes"], {k: t[k] for k in ("file", "measured_at")}
        k = prof["trace_us"].get(key)
        if k is not None:
            roof["kernel_trace_avg_us"] = k["us"]
            roof["frac_kernel_trace"] = algorithmic / k["us"] / peak_per_us
            roof["kernel_trace_source"] = {x: k[x] for x in ("file", "measured_at")}

    annotate(line["roofline"], "qmv_q4_m1_4096", head["bytes"], HBM_PEAK_GBS * 1e3)
    g = extra.get("q4_qmv_m1_4096_graph_replay")
    if g is not None:
        line["roofline"]["graph_replay_launch_us"] = g["us"]
        line["roofline"]["frac_graph_replay"] = g["gbs"] / HBM_PEAK_GBS
    qd = extra.get("q4_qmv_m1_4096_queued_trains")
    if qd is not None:
        line["roofline"]["queued_train_launch_us"] = qd["us"]
    fl = extra.get("floors", {}).get("read_9.45MB")
    if fl is not None:
        # what a kernel that only reads the same bytes reaches in the same train: the ceiling of `frac` at this size
        line["roofline"]["floor_frac"] = fl["gbs"] / HBM_PEAK_GBS
        line["roofline"]["floor_us"] = fl["us"]
    if "q4_qmm_m512_4096" in extra:
        q = extra["q4_qmm_m512_4096"]
        roof = {"bound": "mfma", "achieved": q["tflops"], "peak": MFMA_F16_PEAK_TF, "unit": "TFLOP/s", "frac": q["mfma_frac"],
                "traffic": None, "kernel": "qmm_k2_kernel", "avg_launch_us": q["us"], "flops_per_launch": q["flops"]}
        annotate(roof, "qmm_q4_m512_4096", q["flops"], MFMA_F16_PEAK_TF * 1e6)
        ml = extra.get("floors", {}).get("mfma_loop")
        if ml is not None:  # the matrix instructions alone, no loads and no unpacking
            roof["floor_frac"] = ml["frac_of_peak"]
        line["secondary"] = {"metric": "Q4 qmm TFLOPS (M=512, K=N=4096)", "value": q["tflops"], "unit": "TFLOP/s",
                             "roofline": roof, "launches": q["launches"]}
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(np.random.default_rng(1001), 3.0 if args.quick else 10.0,
                                            all_configs=not args.quick and not args.only)
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
