#!/usr/bin/env python3
"""Writes the committed golden vectors of the quantized-matmul path (tests/golden/*.npz).

The reference's own CPU tests build their data in-process from a tiny LCG and a min/max quantiser
(crates/rmlx-core/src/ops/quantized.rs:10638-10676, 10743-10753, 11605-11636) and assert the CPU
`affine_qmm` against a naive dequantize-then-matmul.  This script reproduces exactly those cases
(same seeds, shapes and draw order) with the restatement in oracle/, and stores inputs and outputs
so that every later change of the oracle or of the HIP kernels is checked against fixed numbers:

  lcg_<M>x<N>x<K>_gs<G>_q<bits>_seed<S>.npz
      x f32 [M,K], w_packed u8 [N,K/2 | K], scales/biases f32 [N,K/G]   (the reference's CPU layout)
      words u32 [N,K*bits/32]                                           (the same weights, MLX layout)
      out_tiled f32 [M,N]   (`affine_qmm` / `affine_qmm_q8` loop nest, quantized.rs:2649-2836)
      out_naive f32 [M,N]   (`naive_matmul_with_dequant`, :10678-10719)
      out_f64  f64 [M,N]    (float64 matmul of the f32-dequantized weights)
  route_T<T>_E<E>_K<K>_seed<S>[_wide].npz
      logits f32 [T,E]; expert_indices u32 [T*K]; expert_weights f32 [T*K]; expert_counts u32 [E];
      dispatch_offsets u32 [E+1]; sorted_assignments u32 [T*K]   (topk_route.rs:212-388, moe.rs:1439-1447)

  dequant_<awq|gptq>_<R>x<C>_gs<G>_seed<S>[_gidx].npz
      qweight / qzeros u32, scales f32, g_idx i32 (GPTQ with act-order only), out f32 [R,C]
      (`awq_dequant_f32` / `gptq_dequant_f32`, quantized.rs:707-783)

Run from the repository root:  python tests/golden/make_fixtures.py
Nothing here reads the reference tree; the fixtures are data only.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import model, refpath  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# (M, N, K, group_size, seed): the reference's test cases; each at 4 and 8 bits
LCG_CASES = [
    (8, 4, 128, 32, 42), (8, 4, 128, 64, 42), (8, 4, 128, 128, 42),   # quantized.rs:10721-10809, 11671-11750
    (4, 2, 64, 32, 123),                                              # :10815-10889, 11868-11939
    (32, 8, 64, 32, 7),                                               # :10933-10998, 11802-11866
    (16, 64, 512, 64, 42),                                            # kernel-sized twin (qmv / qmm shapes)
]
# (T, E, K, seed, logit scale); the last case is so wide that most of a row underflows after exp: its picks past the
# first few are ties at 0.0 that go to the lowest free index
ROUTE_CASES = [(4, 8, 2, 11, 4.0), (32, 128, 8, 12, 4.0), (7, 200, 3, 13, 4.0), (8, 16, 8, 14, 400.0)]
# (format, rows, cols, group_size, seed, with g_idx)
DEQUANT_CASES = [("awq", 16, 24, 4, 21, False), ("awq", 64, 128, 32, 24, False), ("gptq", 32, 16, 8, 22, False),
                 ("gptq", 32, 16, 8, 23, True), ("gptq", 128, 64, 32, 25, True)]


def lcg_case(m, n, k, gs, seed, bits):
    g = refpath.Lcg(seed)
    w = g.fill(n * k).reshape(n, k)  # weights first, then activations (quantized.rs:10750-10753)
    x = g.fill(m * k).reshape(m, k)
    packed, sc, bi = refpath.quantize_rows(w, gs, bits)
    words = model.bytes_to_words(packed)
    return dict(
        x=x, w_packed=packed, scales=sc, biases=bi, words=words,
        out_tiled=refpath.affine_qmm(x, packed, sc, bi, m, n, k, gs, bits),
        out_naive=refpath.naive_matmul_with_dequant(x, packed, sc, bi, m, n, k, gs, bits),
        out_f64=model.qmm(x, words, sc, bi, gs, bits),
    )


def route_case(t, e, k, seed, scale):
    g = refpath.Lcg(seed)
    logits = (scale * g.fill(t * e)).reshape(t, e).astype(np.float32)
    idx, w, counts, offsets = model.topk_route(logits, k)
    sorted_assign, _ = model.moe_sort(idx, e)
    return dict(logits=logits, expert_indices=idx, expert_weights=w.astype(np.float32), expert_counts=counts,
                dispatch_offsets=offsets, sorted_assignments=sorted_assign)


def dequant_case(fmt, rows, cols, gs, seed, with_gidx):
    rng = np.random.default_rng(seed)
    groups = rows // gs
    shape = (rows, cols // 8) if fmt == "awq" else (rows // 8, cols)
    qweight = rng.integers(0, 2**32, size=shape, dtype=np.uint64).astype(np.uint32)
    qzeros = rng.integers(0, 2**32, size=(groups, cols // 8), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.001, 0.05, size=(groups, cols)).astype(np.float32)
    d = dict(qweight=qweight, qzeros=qzeros, scales=scales)
    if fmt == "awq":
        d["out"] = model.awq_dequant(qweight, qzeros, scales, gs)
    else:
        g_idx = rng.integers(0, groups, size=rows).astype(np.int32) if with_gidx else None
        if with_gidx:
            d["g_idx"] = g_idx
        d["out"] = model.gptq_dequant(qweight, qzeros, scales, g_idx, gs)
    return d


def main():
    refpath.build()
    for (fmt, rows, cols, gs, seed, with_gidx) in DEQUANT_CASES:
        name = f"dequant_{fmt}_{rows}x{cols}_gs{gs}_seed{seed}{'_gidx' if with_gidx else ''}.npz"
        np.savez_compressed(os.path.join(HERE, name), **dequant_case(fmt, rows, cols, gs, seed, with_gidx))
    for (m, n, k, gs, seed) in LCG_CASES:
        for bits in (4, 8):
            np.savez_compressed(os.path.join(HERE, f"lcg_{m}x{n}x{k}_gs{gs}_q{bits}_seed{seed}.npz"),
                                **lcg_case(m, n, k, gs, seed, bits))
    for (t, e, k, seed, scale) in ROUTE_CASES:
        name = f"route_T{t}_E{e}_K{k}_seed{seed}{'_wide' if scale > 100 else ''}.npz"
        np.savez_compressed(os.path.join(HERE, name), **route_case(t, e, k, seed, scale))
    print("wrote", len([f for f in os.listdir(HERE) if f.endswith(".npz")]), "fixtures")


if __name__ == "__main__":
    main()
