"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU part: today's oracle reproduces every stored number bit for bit (so an edit of the oracle that
changes results is caught), and the stored numbers satisfy the reference's own assertions.
GPU part: the HIP path, through the C ABI, lands on the stored outputs within the acceptance bar;
routing and sorting are bit-exact.
"""
import glob
import os
import re

import numpy as np
import pytest

from oracle import model, refpath
from tests.helpers import assert_close

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LCG_FILES = sorted(glob.glob(os.path.join(GOLDEN, "lcg_*.npz")))
ROUTE_FILES = sorted(glob.glob(os.path.join(GOLDEN, "route_*.npz")))
DEQUANT_FILES = sorted(glob.glob(os.path.join(GOLDEN, "dequant_*.npz")))


def _lcg_meta(path):
    m, n, k, gs, bits, seed = map(int, re.match(r"lcg_(\d+)x(\d+)x(\d+)_gs(\d+)_q(\d+)_seed(\d+)\.npz",
                                                os.path.basename(path)).groups())
    return m, n, k, gs, bits, seed


def test_fixture_inventory():
    assert len(LCG_FILES) == 12 and len(ROUTE_FILES) == 4 and len(DEQUANT_FILES) == 5


def _dequant_meta(path):
    fmt, rows, cols, gs = re.match(r"dequant_(awq|gptq)_(\d+)x(\d+)_gs(\d+)_", os.path.basename(path)).groups()
    return fmt, int(rows), int(cols), int(gs)


def _dequant_oracle(path):
    fmt, rows, cols, gs = _dequant_meta(path)
    f = np.load(path)
    if fmt == "awq":
        return f, model.awq_dequant(f["qweight"], f["qzeros"], f["scales"], gs)
    return f, model.gptq_dequant(f["qweight"], f["qzeros"], f["scales"], f["g_idx"] if "g_idx" in f else None, gs)


@pytest.mark.parametrize("path", DEQUANT_FILES, ids=os.path.basename)
def test_oracle_reproduces_dequant_fixture(path):
    f, out = _dequant_oracle(path)
    assert out.dtype == np.float32 and np.array_equal(out, f["out"])


@pytest.mark.gpu
@pytest.mark.parametrize("path", DEQUANT_FILES, ids=os.path.basename)
def test_gpu_matches_dequant_fixture(hip, path):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    fmt, rows, cols, gs = _dequant_meta(path)
    f = np.load(path)
    dev = [DeviceBuffer.from_numpy(f[k]) for k in ("qweight", "qzeros", "scales")]
    if fmt == "awq":
        got = ops.awq_dequant(*dev, rows, cols, gs).numpy()
    else:
        g_idx = DeviceBuffer.from_numpy(f["g_idx"].view(np.uint32)) if "g_idx" in f else None
        got = ops.gptq_dequant(*dev, g_idx, rows, cols, gs).numpy()
    assert np.array_equal(got, f["out"])


@pytest.mark.parametrize("path", LCG_FILES, ids=os.path.basename)
def test_oracle_reproduces_lcg_fixture(path):
    m, n, k, gs, bits, seed = _lcg_meta(path)
    f = np.load(path)
    g = refpath.Lcg(seed)
    w = g.fill(n * k).reshape(n, k)
    x = g.fill(m * k).reshape(m, k)
    assert np.array_equal(x, f["x"])
    packed, sc, bi = refpath.quantize_rows(w, gs, bits)
    assert np.array_equal(packed, f["w_packed"]) and np.array_equal(sc, f["scales"]) and np.array_equal(bi, f["biases"])
    assert np.array_equal(model.bytes_to_words(packed), f["words"])
    assert np.array_equal(model.words_to_bytes(f["words"]), f["w_packed"])
    tiled = refpath.affine_qmm(x, packed, sc, bi, m, n, k, gs, bits)
    naive = refpath.naive_matmul_with_dequant(x, packed, sc, bi, m, n, k, gs, bits)
    assert np.array_equal(tiled, f["out_tiled"]) and np.array_equal(naive, f["out_naive"])
    # the reference's assertion on this data: tiled vs naive within 1e-4 relative (quantized.rs:10794-10808)
    assert np.all(np.abs(f["out_tiled"] - f["out_naive"]) / np.maximum(np.abs(f["out_naive"]), 1.0) < 1e-4)
    assert np.all(np.abs(f["out_tiled"] - f["out_f64"]) / np.maximum(np.abs(f["out_f64"]), 1.0) < 1e-4)
    assert np.array_equal(model.qmm(x, f["words"], sc, bi, gs, bits), f["out_f64"])


@pytest.mark.parametrize("path", ROUTE_FILES, ids=os.path.basename)
def test_oracle_reproduces_route_fixture(path):
    f = np.load(path)
    t, e = f["logits"].shape
    k = f["expert_indices"].size // t
    idx, w, counts, offsets = model.topk_route(f["logits"], k)
    assert np.array_equal(idx, f["expert_indices"]) and np.array_equal(counts, f["expert_counts"])
    assert np.array_equal(offsets, f["dispatch_offsets"])
    assert np.array_equal(w, f["expert_weights"])
    # brute force: stable argsort of exp(l - max) in float64, with what lies more than 80 below the row maximum
    # counted as 0 (the f32 softmax value underflows there, so those experts tie and go in index order)
    d = f["logits"].astype(np.float64) - f["logits"].max(axis=1, keepdims=True)
    brute = np.argsort(-np.where(d < -80.0, 0.0, np.exp(d)), axis=1, kind="stable")[:, :k].reshape(-1)
    assert np.array_equal(brute.astype(np.uint32), f["expert_indices"])
    if "_wide" in path:  # the case exists for the ties: ranking the logits must give other picks
        assert not np.array_equal(np.argsort(-f["logits"], axis=1, kind="stable")[:, :k].reshape(-1), f["expert_indices"])
    assert np.array_equal(np.argsort(f["expert_indices"], kind="stable").astype(np.uint32), f["sorted_assignments"])
    assert np.array_equal(np.bincount(f["expert_indices"], minlength=e), f["expert_counts"])


# ---- GPU -------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("path", LCG_FILES, ids=os.path.basename)
def test_gpu_matches_lcg_fixture(hip, path):
    from rmlx_amd import ops, runtime as rt
    m, n, k, gs, bits, seed = _lcg_meta(path)
    f = np.load(path)
    qw = ops.QuantizedWeight.from_numpy(f["words"], f["scales"].astype(np.float16), f["biases"].astype(np.float16), gs, bits)
    xd = rt.DeviceBuffer.from_numpy(f["x"])  # f32 activations: the cast is part of the path
    kernels = [rt.KERNEL_AUTO, rt.KERNEL_GENERIC]
    if n % 64 == 0 and k % 512 == 0 and gs == 64:
        kernels += [rt.KERNEL_QMM, rt.KERNEL_QMM_LDS] + ([rt.KERNEL_QMV] if bits == 4 else [])
    for kernel in kernels:
        out = ops.affine_quantized_matmul_batched(xd, qw, kernel=kernel).numpy()
        assert_close(out, f["out_f64"], f"{os.path.basename(path)} kernel={kernel}")


@pytest.mark.gpu
@pytest.mark.parametrize("path", ROUTE_FILES, ids=os.path.basename)
def test_gpu_matches_route_fixture(hip, path):
    from rmlx_amd import ops, runtime as rt
    f = np.load(path)
    t, e = f["logits"].shape
    k = f["expert_indices"].size // t
    r = ops.gpu_topk_route(rt.DeviceBuffer.from_numpy(f["logits"]), k)
    assert np.array_equal(r.expert_indices.numpy(), f["expert_indices"])
    assert np.array_equal(r.expert_counts.numpy(), f["expert_counts"])
    assert np.array_equal(r.dispatch_offsets.numpy(), f["dispatch_offsets"])
    # the routing kernel evaluates the softmax with the same sequence of f32 operations as the oracle
    assert np.array_equal(r.expert_weights.numpy(), f["expert_weights"])
    s, off = ops.moe_sort(r.expert_indices, e)
    assert np.array_equal(s.numpy(), f["sorted_assignments"]) and np.array_equal(off.numpy(), f["dispatch_offsets"])
