"""Pins the MoE half of the CPU oracle (routing weights, gather_qmm, SwiGLU, expert FFN, weighted combine)
against the reference's own known answers, float64 closed forms and brute-force loops that share no code with
the functions they check.  No GPU needed.
"""
import math

import numpy as np
import pytest

from oracle import model, refpath
from tests.helpers import make_weight


# ---- exp used by the routing -------------------------------------------------------------------------------

def test_exp_neg_exact_against_float64():
    rng = np.random.default_rng(0)
    x = np.concatenate([-rng.uniform(0, 80, 100_000), [0.0, -0.0, -80.0, -1e-8, -math.log(2), -10 * math.log(2)]])
    x = x.astype(np.float32)
    got = model.exp_neg_exact(x)
    ref = np.exp(x.astype(np.float64))
    assert np.all(np.abs(got - ref) <= 1.5 * np.spacing(ref.astype(np.float32)))
    assert got[100_000] == 1.0 and got[100_001] == 1.0
    xs = np.sort(x)
    assert np.all(np.diff(model.exp_neg_exact(xs)) >= 0)  # monotone: ranking by it never inverts the logits' order
    # below the cut-off the value is exactly zero and nothing is subnormal above it
    assert np.all(model.exp_neg_exact(np.array([-80.001, -200.0, -1e30, -np.inf], np.float32)) == 0.0)
    assert model.exp_neg_exact(np.array([-80.0], np.float32))[0] / 256 > np.finfo(np.float32).tiny


# ---- routing weights -----------------------------------------------------------------------------------------

def _softmax64(rows):
    rows = np.asarray(rows, dtype=np.float64)
    e = np.exp(rows - rows.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


@pytest.mark.parametrize("T,E,K,seed", [(16, 128, 8, 1), (5, 8, 2, 2), (3, 256, 8, 3), (9, 60, 1, 4), (4, 200, 5, 5)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_topk_route_weights_closed_form(T, E, K, seed, with_bias):
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((T, E)) * 2).astype(np.float32)
    bias = rng.standard_normal(E).astype(np.float32) if with_bias else None
    biased = logits if bias is None else (logits + bias[None, :]).astype(np.float32)
    idx, w, counts, offsets = model.topk_route(logits, K, bias=bias)
    idx2 = idx.reshape(T, K).astype(np.int64)
    # indices: brute-force stable argsort of the float64 softmax (no ties in continuous random data)
    assert np.array_equal(idx2, np.argsort(-_softmax64(biased), axis=1, kind="stable")[:, :K])
    # renormalised top-k softmax == softmax over the selected logits only
    sel = np.take_along_axis(biased.astype(np.float64), idx2, axis=1)
    assert np.allclose(w.reshape(T, K), _softmax64(sel), rtol=0, atol=1e-6)
    assert np.allclose(w.reshape(T, K).sum(axis=1), 1.0, atol=1e-6)
    # without renormalisation: the plain float64 softmax at the picks
    idx_p, w_p, _, _ = model.topk_route(logits, K, bias=bias, renormalize=False)
    assert np.array_equal(idx_p, idx)
    assert np.allclose(w_p.reshape(T, K), np.take_along_axis(_softmax64(biased), idx2, axis=1), rtol=0, atol=1e-6)
    assert np.array_equal(counts, np.bincount(idx, minlength=E)) and counts.sum() == T * K
    assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]))


def test_topk_route_ranks_softmax_values_with_ties_to_the_lower_index():
    # The reference ranks the f32 softmax value with strict > (topk_route.rs:283-300).  Expected picks by hand:
    # row 0: exp(-200) and exp(-150) are both 0 in f32 -> after expert 0 the tail ties at 0.0 -> experts 1, 2
    #        (ranking the logits would give 0, 2, 3: -150 and -160 beat -200)
    # row 1: everything but expert 5 underflows -> 5, then 0, 1
    # row 2: all equal -> 0, 1, 2
    # row 3: two exact ties at the top (3 and 6), then an underflowing tail -> 3, 6, 0
    logits = np.array([
        [0, -200, -150, -160, -170, -300, -120, -110],
        [-500, -400, -300, -200, -100, 0, -450, -350],
        [1, 1, 1, 1, 1, 1, 1, 1],
        [-100, -100, -100, 7, -100, -100, 7, -100],
    ], np.float32)
    want = np.array([[0, 1, 2], [5, 0, 1], [0, 1, 2], [3, 6, 0]], np.uint32)
    idx, w, _, _ = model.topk_route(logits, 3)
    assert np.array_equal(idx.reshape(4, 3), want)
    assert np.allclose(w.reshape(4, 3), [[1, 0, 0], [1, 0, 0], [1 / 3] * 3, [0.5, 0.5, 0]], atol=1e-6)
    # the same rows reached through a wide expert_bias on all-zero logits
    for r in range(4):
        idx_b, _, _, _ = model.topk_route(np.zeros((1, 8), np.float32), 3, bias=logits[r])
        assert np.array_equal(idx_b, want[r])
    # ranking the logits is a different order on row 0 -- the case the default must not follow
    idx_l, _, _, _ = model.topk_route(logits[:1], 3, rank_by="logit")
    assert list(idx_l) == [0, 7, 6]


# ---- gather_qmm ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("E,N,K,gs,batch,seed", [(4, 8, 64, 32, 6, 0), (3, 16, 128, 64, 5, 1), (5, 4, 256, 128, 9, 2)])
def test_gather_qmm_against_per_row_cpu_qmv(E, N, K, gs, batch, seed):
    # per row: the reference's test helper cpu_qmv_q4_reference (quantized.rs:12018-12049) on the picked expert
    rng = np.random.default_rng(seed)
    words, s, b = make_weight(rng, N, K, 4, gs, lead=(E,))
    x = rng.standard_normal((batch, K)).astype(np.float16)
    idx = rng.integers(0, E, batch).astype(np.uint32)
    idx[:2] = idx[0]  # a repeated expert
    got = model.gather_qmm(x, words, s, b, idx, gs)
    for r in range(batch):
        e = int(idx[r])
        ref = refpath.cpu_qmv_q4_reference(words[e], s[e].astype(np.float32), b[e].astype(np.float32),
                                           x[r].astype(np.float32), N, K, gs)
        assert np.allclose(got[r], ref, rtol=1e-4, atol=1e-4)
    # [batch, M_b, K] form: every row of an entry meets the same expert
    x3 = rng.standard_normal((batch, 3, K)).astype(np.float16)
    got3 = model.gather_qmm(x3, words, s, b, idx, gs)
    assert got3.shape == (batch, 3, N)
    for r in range(batch):
        assert np.array_equal(got3[r], model.qmm(x3[r], words[idx[r]], s[idx[r]], b[idx[r]], gs, 4))


# ---- SwiGLU ----------------------------------------------------------------------------------------------------

def test_silu_values():
    assert model.silu(0.0) == 0.0
    for v in (-20.0, -3.0, -0.5, 0.25, 1.0, 7.0):
        assert math.isclose(float(model.silu(v)), v / (1.0 + math.exp(-v)), rel_tol=1e-15)
        assert math.isclose(float(model.silu(v)) - float(model.silu(-v)), v, rel_tol=1e-12)  # silu(v) - silu(-v) = v
    assert math.isclose(float(model.silu(40.0)), 40.0, rel_tol=1e-15) and abs(float(model.silu(-40.0))) < 1e-15


# ---- weighted combine --------------------------------------------------------------------------------------------

def test_scatter_weighted_add_kat():
    # test_scatter_weighted_add_f32 (crates/rmlx-core/src/ops/moe_kernels.rs:420-450)
    src = [[10.0, 20.0], [30.0, 40.0], [50.0, 60.0]]
    out = model.scatter_weighted_add(src, [0, 1, 0], [0.5, 1.0, 0.25], 2)
    assert np.allclose(out, [[17.5, 25.0], [30.0, 40.0]], atol=1e-4)


def test_combine_cpu_kats():
    # test_moe_combine_cpu (crates/rmlx-distributed/tests/moe_tests.rs:115-135)
    out = model.combine_cpu([[1.0, 2, 3, 4, 5, 6], [10.0, 20, 30, 40, 50, 60]], [0.5, 0.7], [0, 1], 2, 1, 3)
    assert np.allclose(out, [[0.5, 1.0, 1.5], [28.0, 35.0, 42.0]], atol=1e-5)
    # zero weight (:660-672), top-2 (:674-687), out-of-range expert skipped (:689 ff.)
    assert np.allclose(model.combine_cpu([[10.0, 20, 30]], [0.0], [0], 1, 1, 3), 0.0)
    assert np.allclose(model.combine_cpu([[1.0, 2], [10.0, 20]], [0.6, 0.4], [0, 1], 1, 2, 2), [[4.6, 9.2]], atol=1e-5)
    assert np.allclose(model.combine_cpu([[1.0, 2]], [1.0], [7], 1, 1, 2), 0.0)


def test_scatter_weighted_add_equals_combine_cpu():
    # the two reference formulations of the combine agree: per-assignment rows against per-expert [T, D] outputs
    rng = np.random.default_rng(3)
    T, K, D, E = 5, 3, 4, 6
    per_expert = rng.standard_normal((E, T, D))
    idx = np.stack([rng.permutation(E)[:K] for _ in range(T)]).reshape(-1)
    w = rng.uniform(0, 1, T * K)
    rows = np.stack([per_expert[idx[a], a // K] for a in range(T * K)])
    a = model.scatter_weighted_add(rows, np.arange(T * K) // K, w, T)
    b = model.combine_cpu([per_expert[e].reshape(-1) for e in range(E)], w, idx, T, K, D)
    assert np.allclose(a, b, rtol=1e-13, atol=1e-13)


# ---- the whole block -----------------------------------------------------------------------------------------------

def _brute_moe(x, idx, w, gate, up, down, gs, K):
    """Per (token, k), nothing shared with model.moe_forward: rows dequantised by the C restatement of
    `dequantize_q4_row` from the byte image, Python-float dot products, math.exp, the hidden value rounded to f16."""
    T, D = x.shape
    inter = gate[0].shape[1]
    out = [[0.0] * D for _ in range(T)]

    def rows(trip, e):
        words, s, b = (t[e] for t in trip)
        n, k = words.shape[0], words.shape[1] * 8
        byts = model.words_to_bytes(words)
        return [refpath.dequantize_q4_row(byts[j], s[j].astype(np.float32), b[j].astype(np.float32), k, gs).astype(float)
                for j in range(n)]

    for t in range(T):
        xt = [float(v) for v in x[t]]
        for k in range(K):
            e = int(idx[t * K + k])
            wg, wu, wd = rows(gate, e), rows(up, e), rows(down, e)
            h = []
            for j in range(inter):
                g = sum(a * c for a, c in zip(xt, wg[j]))
                u = sum(a * c for a, c in zip(xt, wu[j]))
                h.append(float(np.float16(g / (1.0 + math.exp(-g)) * u)))
            for d in range(D):
                out[t][d] += float(w[t * K + k]) * sum(a * c for a, c in zip(h, wd[d]))
    return np.array(out)


@pytest.mark.parametrize("T,E,K,D,I,gs,seed", [(3, 4, 2, 64, 32, 32, 0), (4, 3, 3, 64, 64, 64, 1), (2, 5, 4, 128, 128, 128, 2)])
def test_moe_forward_against_brute_force(T, E, K, D, I, gs, seed):
    rng = np.random.default_rng(seed)
    gate, up, down = (make_weight(rng, n, k, 4, gs, lead=(E,)) for n, k in ((I, D), (I, D), (D, I)))
    x = rng.standard_normal((T, D)).astype(np.float16)
    # distinct experts per token as a router gives them, several tokens sharing an expert, and one token that
    # names the same expert twice (the flat interface allows it)
    idx = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint32)
    idx[-1, 1] = idx[-1, 0]
    w = rng.uniform(0.05, 1.0, (T, K)).astype(np.float32)
    got = model.moe_forward(x, idx.reshape(-1), w.reshape(-1), gate, up, down, gs, K)
    ref = _brute_moe(x, idx.reshape(-1), w.reshape(-1), gate, up, down, gs, K)
    assert np.allclose(got, ref, rtol=1e-9, atol=1e-9 * np.abs(ref).max())


def test_moe_forward_closed_forms():
    rng = np.random.default_rng(7)
    E, D, I, gs, T = 3, 64, 64, 64, 4
    gate, up, down = (make_weight(rng, n, k, 4, gs, lead=(E,)) for n, k in ((I, D), (I, D), (D, I)))
    x = rng.standard_normal((T, D)).astype(np.float16)
    # top-1 with unit weight == the plain expert FFN of that expert, token by token
    idx = np.array([2, 0, 1, 2], np.uint32)
    one = model.moe_forward(x, idx, np.ones(T, np.float32), gate, up, down, gs, 1)
    for t in range(T):
        wg, wu, wd = (model.dequantize(tr[0][idx[t]], tr[1][idx[t]], tr[2][idx[t]], gs, 4) for tr in (gate, up, down))
        assert np.array_equal(one[t], model.expert_ffn(x[t:t + 1], wg, wu, wd)[0])
    # linear in the routing weights; a zero weight removes the expert; the order of a token's experts is free
    idx2 = np.array([[0, 1], [1, 2], [2, 0], [0, 2]], np.uint32)
    w2 = rng.uniform(0.1, 1, (T, 2)).astype(np.float32)
    full = model.moe_forward(x, idx2.reshape(-1), w2.reshape(-1), gate, up, down, gs, 2)
    first = model.moe_forward(x, idx2[:, 0], w2[:, 0], gate, up, down, gs, 1)
    second = model.moe_forward(x, idx2[:, 1], w2[:, 1], gate, up, down, gs, 1)
    assert np.allclose(full, first + second, rtol=1e-13, atol=1e-12)
    w0 = w2.copy()
    w0[:, 1] = 0
    assert np.allclose(model.moe_forward(x, idx2.reshape(-1), w0.reshape(-1), gate, up, down, gs, 2), first, atol=1e-12)
    swapped = model.moe_forward(x, idx2[:, ::-1].reshape(-1), w2[:, ::-1].reshape(-1), gate, up, down, gs, 2)
    assert np.allclose(full, swapped, rtol=1e-13, atol=1e-12)
    # an all-zero down bias/scale trick: zero activations give a zero output (silu(0) * 0)
    assert np.all(model.moe_forward(np.zeros((2, D), np.float16), [0, 1], [1.0, 1.0], gate, up, down, gs, 1) == 0)
