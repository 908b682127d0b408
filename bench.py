#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

Headline (`value`): Q4 qmv at M=1, K=N=4096 (group 64, f16) in GB/s of algorithmic bytes.  A step
is one launch of the qmv kernel; weights are cycled over enough distinct sets (> 1 GiB) that
every launch streams from HBM instead of the L2 / Infinity Cache.  All inputs are resident in
HBM before the timed region.  The other benchmark configurations (qmv at N=9216, Q4 qmm at
M=128/512, Q8 bf16 qmm, the MoE block) are timed the same way and reported under "extra".
One JSON line is printed on stdout.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
MFMA_F16_PEAK_TF = 2500.0  # dense f16 / bf16 MFMA

# HBM-side bytes per launch of the two roofline kernels, from rocprofv3 counter runs of this script
# (FETCH_SIZE and WRITE_SIZE, each scaled by what it reads for the plain copy below); the runs and
# the scaling are recorded in profiles/bench_all_configs_hbm_traffic_pmc.txt.  Counters cannot be
# read from inside this process, so the figures are carried here and re-measured with the kernels.
MEASURED_TRAFFIC_BYTES = {"qmv_q4_m1_4096": 9541139, "qmm_q4_m512_4096": 39722504}


def matmul_bytes(m, n, k, bits, gs=64, act_bytes=2):
    """Algorithmic bytes of one quantized matmul: packed weights + f16 scales and biases +
    activations in + f16 out."""
    return n * k * bits // 8 + 2 * (n * k // gs) * 2 + m * k * act_bytes + m * n * 2


def make_weight(rng, n, k, bits, lead=()):
    lo, hi = (0.005, 0.02) if bits == 4 else (0.0005, 0.002)
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

    def run(self, fn, steps, warmup):
        fn(warmup)
        self.stream.sync()
        self.e0.record(self.stream)
        fn(steps)
        self.e1.record(self.stream)
        self.e1.sync()
        self.stream.sync()
        return self.e0.elapsed_ms(self.e1) / steps  # ms per step


def bench_matmul(ops, rt, timer, rng, m, n, k, bits, x_dtype, steps, warmup, min_total_bytes, check=True, kernel=0):
    from oracle import model
    wbytes = n * k * bits // 8 + 4 * (n * k // 64)
    n_sets = max(1, -(-min_total_bytes // wbytes))
    base = make_weight(rng, n, k, bits)
    qws = [ops.QuantizedWeight.from_numpy(*base, 64, bits)]
    for i in range(1, n_sets):  # distinct buffers; contents rolled so that sets differ
        qws.append(ops.QuantizedWeight.from_numpy(np.roll(base[0], i, axis=0), np.roll(base[1], i, axis=0),
                                                  np.roll(base[2], i, axis=0), 64, bits))
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
    ms = timer.run(lambda c: ops.qmm_encode_many(qws, xd, outs, c, stream=timer.stream, kernel=kernel), steps, warmup)
    res = {"us": ms * 1e3, "steps": steps, "n_weight_sets": n_sets,
           "bytes": matmul_bytes(m, n, k, bits, act_bytes=2), "flops": 2 * m * n * k}
    res["gbs"] = res["bytes"] / (ms * 1e-3) / 1e9
    res["tflops"] = res["flops"] / (ms * 1e-3) / 1e12
    if check:  # parity of the timed configuration against the oracle, on weight set 0
        ops.qmm_encode_many(qws[:1], xd, outs[:1], 1, stream=timer.stream, kernel=kernel)
        timer.stream.sync()
        ref = model.qmm(x64, *base, 64, bits)
        err = float(np.abs(outs[0].numpy().astype(np.float64) - ref).max())
        res["max_err"], res["tol"] = err, model.tolerance(ref)
        res["pass"] = bool(err <= res["tol"])
    return res


def bench_moe(ops, rt, timer, rng, T, steps, warmup, experts, bits=4):
    from oracle import model
    gate_up, down, gh, dh = experts
    x = rng.standard_normal((T, 4096)).astype(np.float16)
    logits = rng.standard_normal((T, 128)).astype(np.float32)
    xd, ld = rt.DeviceBuffer.from_numpy(x), rt.DeviceBuffer.from_numpy(logits)
    out = rt.DeviceBuffer((T, 4096), rt.F16)

    def run(c):
        for _ in range(c):
            ops.moe_forward(gh, None, dh, xd, ld, 8, stream=timer.stream, out=out)

    ms = timer.run(run, steps, warmup)
    idx, w, _, _ = model.topk_route(logits, 8)
    distinct = len(np.unique(idx))
    nbytes = distinct * (18874368 * bits // 8 + 1179648) + T * 4096 * 2 * 2 + T * 128 * 4
    res = {"us": ms * 1e3, "distinct_experts": distinct, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9,
           "flops": 2 * 8 * T * (4096 * 3072 + 1536 * 4096)}
    toks = np.arange(min(T, 2))
    sel = (toks[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    gate = tuple(a[:, :1536] for a in gate_up)
    up = tuple(a[:, 1536:] for a in gate_up)
    ref = model.moe_forward(x[toks], idx[sel], w[sel], gate, up, down, 64, 8, bits=bits)
    err = float(np.abs(out.numpy()[toks].astype(np.float64) - ref).max())
    res["max_err"], res["tol"], res["pass"] = err, model.tolerance(ref), bool(err <= model.tolerance(ref))
    return res


def bench_gather(ops, rt, timer, rng, batch, mpb, gh, gate_up, steps, warmup):
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

    ms = timer.run(run, steps, warmup)
    distinct = len(np.unique(idx))
    nbytes = distinct * (n * k // 2 + 4 * (n * k // 64)) + batch * mpb * (k + n) * 2
    res = {"us": ms * 1e3, "distinct_experts": distinct, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9}
    e0 = int(idx[0])
    ref = model.qmm(x[0].astype(np.float64), gate_up[0][e0], gate_up[1][e0], gate_up[2][e0], 64, 4)
    err = float(np.abs(out.numpy()[0].astype(np.float64) - ref).max())
    res["max_err"], res["tol"], res["pass"] = err, model.tolerance(ref), bool(err <= model.tolerance(ref))
    return res


def bench_dequant(ops, rt, timer, rng, fmt, k, n, gs, steps, warmup):
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

    ms = timer.run(run, steps, warmup)
    nbytes = k * n * 4 + k * n // 2 + groups * n // 2 + groups * n * 4
    launch(0)
    timer.stream.sync()
    qw, qz, sc, _ = sets[0]
    ref = model.awq_dequant(qw, qz, sc, gs) if fmt == "awq" else model.gptq_dequant(qw, qz, sc, None, gs)
    return {"us": ms * 1e3, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9,
            "hbm_frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "pass": bool(np.array_equal(out.numpy(), ref))}


def cpu_baseline(rng, budget_s=10.0):
    """The C restatement of the reference's scalar `affine_qmm` (oracle/affine_qmm_ref.c) on the
    headline configuration (M=1, K=N=4096), one host thread, repeated for about `budget_s`."""
    from oracle import model, refpath
    n = k = 4096
    words, s, b = make_weight(rng, n, k, 4)
    x = rng.standard_normal((1, k)).astype(np.float16).astype(np.float32)
    wb, s32, b32 = model.words_to_bytes(words), s.astype(np.float32), b.astype(np.float32)
    refpath.affine_qmm(x, wb, s32, b32, 1, n, k, 64)  # warm
    reps, t0 = 0, time.perf_counter()
    while True:
        refpath.affine_qmm(x, wb, s32, b32, 1, n, k, 64)
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s:
            break
    per = el / reps
    # the same loop nest with the output columns split over the host cores this job may use
    threads = min(16, os.cpu_count() or 1)
    treps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s / 4:
        refpath.affine_qmm_threads(x, wb, s32, b32, 1, n, k, 64, threads=threads)
        treps += 1
    tper = (time.perf_counter() - t0) / treps
    return {"value": matmul_bytes(1, n, k, 4) / per / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} repetitions of the full M=1 K=N=4096 Q4 matmul ({el:.1f} s, {per * 1e3:.2f} ms each)",
            "us_per_matmul": per * 1e6, "host_cores_available": os.cpu_count(),
            "all_cores": {"value": matmul_bytes(1, n, k, 4) / tper / 1e9, "unit": "GB/s", "cores": threads,
                          "us_per_matmul": tper * 1e6, "sample": f"{treps} repetitions, columns split over {threads} threads"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20000)
    ap.add_argument("--warmup", type=int, default=2000)
    ap.add_argument("--quick", action="store_true", help="headline configuration only, short CPU baseline")
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    from rmlx_amd import ops, runtime as rt
    rt.init(0)
    info = rt.device_info()
    timer = Timer(rt)
    rng = np.random.default_rng(1001)
    GiB = 1 << 30

    # ---- headline: Q4 qmv M=1 K=N=4096, weights cycled through > 1 GiB ---------------------------------
    head = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "f16", args.steps, args.warmup, GiB + GiB // 8)
    extra = {"device": info, "q4_qmv_m1_4096": head}
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
    if not args.quick:
        extra["q4_qmv_m1_4096_cache_resident"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 4, "f16",
                                                              args.steps, args.warmup, 0, check=False)
        for m in (1, 4, 8):
            extra[f"q4_qmv_m{m}_n9216"] = bench_matmul(ops, rt, timer, rng, m, 9216, 4096, 4, "f16", args.steps,
                                                       args.warmup, GiB + GiB // 8, check=(m == 8))
        extra["q4_qmv_m2_4096"] = bench_matmul(ops, rt, timer, rng, 2, 4096, 4096, 4, "f16", args.steps, args.warmup,
                                               GiB + GiB // 8)
        extra["q8_qmv_m1_4096"] = bench_matmul(ops, rt, timer, rng, 1, 4096, 4096, 8, "f16", args.steps, args.warmup,
                                               GiB + GiB // 8)
        # the GEMM sections run at least 10 000 steps: the GPU needs a few hundred milliseconds of sustained
        # matrix work before its clock settles (a 100-launch window reads 15 % slower, a 2 000-launch one 3 %)
        # (short runs, as under a counter pass, keep their own count)
        gemm_steps = max(args.steps, 10000) if args.steps >= 1000 else args.steps
        for m in (128, 512, 4096):
            m_steps = gemm_steps if m <= 512 else max(50, gemm_steps // 10)
            r = bench_matmul(ops, rt, timer, rng, m, 4096, 4096, 4, "f16", m_steps, min(args.warmup, m_steps), 4 * 9437184)
            r["steps"] = m_steps
            r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
            extra[f"q4_qmm_m{m}_4096"] = r
        for name, kern in (("q8_qmm_bf16_m128_n12288", rt.KERNEL_AUTO), ("q8_qmm_bf16_m128_n12288_bf16_mfma", rt.KERNEL_QMM_BF16)):
            r = bench_matmul(ops, rt, timer, rng, 128, 12288, 4096, 8, "bf16", gemm_steps, args.warmup, 4 * 53477376, kernel=kern)
            r["steps"] = gemm_steps
            r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
            r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
            extra[name] = r
        for fmt in ("awq", "gptq"):
            extra[f"{fmt}_dequant_4096x4096_gs128"] = bench_dequant(ops, rt, timer, rng, fmt, 4096, 4096, 128,
                                                                    max(50, args.steps // 10), 10)
        gate_up = make_weight(rng, 3072, 4096, 4, lead=(128,))
        down = make_weight(rng, 4096, 1536, 4, lead=(128,))
        experts = (gate_up, down, ops.QuantizedWeight.from_numpy(*gate_up, 64, 4),
                   ops.QuantizedWeight.from_numpy(*down, 64, 4))
        for batch, mpb in ((32, 1), (32, 8), (32, 64)):
            r = bench_gather(ops, rt, timer, rng, batch, mpb, experts[2], gate_up, max(50, args.steps // 10), 10)
            r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
            extra[f"gather_qmm_q4_b{batch}_m{mpb}"] = r
        for T in (4, 32, 128, 512, 2048):  # from 8 rows per expert on average (T = 128) on the grouped MFMA GEMM
            r = bench_moe(ops, rt, timer, rng, T, max(50, args.steps // (10 if T <= 128 else 40)), 10, experts)
            r["tflops"] = r["flops"] / (r["us"] * 1e-6) / 1e12
            r["mfma_frac"] = r["tflops"] / MFMA_F16_PEAK_TF
            r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
            extra[f"moe_q4_T{T}"] = r
        del experts, gate_up, down
        gate_up = make_weight(rng, 3072, 4096, 8, lead=(128,))
        down = make_weight(rng, 4096, 1536, 8, lead=(128,))
        experts = (gate_up, down, ops.QuantizedWeight.from_numpy(*gate_up, 64, 8),
                   ops.QuantizedWeight.from_numpy(*down, 64, 8))
        for T in (4, 32, 512):
            r = bench_moe(ops, rt, timer, rng, T, max(50, args.steps // (10 if T <= 128 else 40)), 10, experts, bits=8)
            r["tflops"] = r["flops"] / (r["us"] * 1e-6) / 1e12
            r["hbm_frac"] = r["gbs"] / HBM_PEAK_GBS
            extra[f"moe_q8_T{T}"] = r

    line = {
        "metric": "Q4 qmv HBM GB/s (M=1, K=N=4096)",
        "value": head["gbs"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["us"] / 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "Q4 qmv M=1 K=4096 N=4096 group_size=64 f16 activations, "
                               f"{head['n_weight_sets']} distinct weight sets cycled (HBM-resident, > 1 GiB)",
                   "parity_max_err": head.get("max_err"), "parity_tol": head.get("tol")},
        "roofline": {"bound": "hbm", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["gbs"] / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES["qmv_q4_m1_4096"],
                     "kernel": "qmv_m1_kernel<4,64,1,true,1,false>", "bytes_per_launch": head["bytes"],
                     "avg_launch_us": head["us"]},
    }
    if not args.quick and "q4_qmm_m512_4096" in extra:
        q = extra["q4_qmm_m512_4096"]
        line["secondary"] = {"metric": "Q4 qmm TFLOPS (M=512, K=N=4096)", "value": q["tflops"], "unit": "TFLOP/s",
                             "roofline": {"bound": "mfma", "achieved": q["tflops"], "peak": MFMA_F16_PEAK_TF,
                                          "unit": "TFLOP/s", "frac": q["mfma_frac"],
                                          "traffic": MEASURED_TRAFFIC_BYTES["qmm_q4_m512_4096"],
                                          "kernel": "qmm_rw_kernel<4,1,4,8,false,64>", "avg_launch_us": q["us"]},
                             "steps": q["steps"]}
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(np.random.default_rng(1001), 3.0 if args.quick else 10.0)
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
