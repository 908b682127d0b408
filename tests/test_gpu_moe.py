"""GPU parity of routing, expert grouping, gather_qmm and the fused MoE block, through the C ABI.

Integer outputs (expert indices, counts, offsets, sort permutation) must be bit-exact; f16
outputs follow the 1e-2 * RMS bar; routing weights are f32 and compared to 1e-6.
"""
import numpy as np
import pytest

from oracle import model
from tests.helpers import assert_close, make_weight, make_x

pytestmark = pytest.mark.gpu


def _route(hip, logits, k, bias=None, dtype=np.float32):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    lb = DeviceBuffer.from_numpy(logits.astype(dtype))
    bb = DeviceBuffer.from_numpy(bias.astype(np.float32)) if bias is not None else None
    r = ops.gpu_topk_route(lb, k, bb)
    return r.expert_indices.numpy(), r.expert_weights.numpy(), r.expert_counts.numpy(), r.dispatch_offsets.numpy()


# ---- the reference's behavioural tests (topk_route.rs:665-878) -----------------------------------------

def test_topk_route_basic(hip):
    logits = np.array([[0.1, 0.1, 5.0, 0.1, 0.1, 3.0, 0.1, 0.1],
                       [4.0, 0.1, 0.1, 0.1, 0.1, 0.1, 0.1, 3.0],
                       [0.1, 0.1, 0.1, 5.0, 4.0, 0.1, 0.1, 0.1],
                       [0.1, 4.0, 0.1, 0.1, 0.1, 0.1, 3.5, 0.1]], np.float32)
    idx, w, counts, off = _route(hip, logits, 2)
    assert idx.shape == (8,) and w.shape == (8,) and counts.shape == (8,) and off.shape == (9,)
    assert list(idx) == [2, 5, 0, 7, 3, 4, 1, 6]  # descending per token
    assert np.allclose(w.reshape(4, 2).sum(1), 1.0, atol=1e-4)
    assert counts.sum() == 8 and off[0] == 0 and off[8] == 8
    assert np.array_equal(off[1:], np.cumsum(counts))


def test_topk_route_with_bias_and_single_token_and_f16(hip):
    logits = np.array([[3.0, 1.0, 2.9, 1.0], [1.0, 3.0, 1.0, 1.0]], np.float32)
    idx, _, _, _ = _route(hip, logits, 1, bias=np.array([0, 0, 5.0, 0]))
    assert idx[0] == 2
    idx, w, _, _ = _route(hip, np.array([[1.0, 5.0, 0.5, 4.0]], np.float32), 2)
    assert list(idx) == [1, 3] and abs(w.sum() - 1.0) < 1e-4
    idx, w, _, _ = _route(hip, np.array([[1.0, 5.0, 0.5, 4.0], [3.0, 0.1, 0.2, 0.1]]), 1, dtype=np.float16)
    assert list(idx) == [1, 0] and abs(w[0] - 1.0) < 1e-3


def test_topk_route_validation(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    bad = DeviceBuffer.from_numpy(np.array([1.0, 2.0, 3.0], np.float32))
    with pytest.raises(ops.KernelError, match="must be 2D"):
        ops.gpu_topk_route(bad, 2)
    lg = DeviceBuffer.from_numpy(np.ones((2, 4), np.float32))
    for k in (0, 9):
        with pytest.raises(ops.KernelError, match=r"top_k must be in \[1, 8\]"):
            ops.gpu_topk_route(lg, k)
    with pytest.raises(ops.KernelError, match="> num_experts"):
        ops.gpu_topk_route(lg, 5)
    with pytest.raises(ops.KernelError, match="exceeds maximum 256"):
        ops.gpu_topk_route(DeviceBuffer.from_numpy(np.ones((1, 300), np.float32)), 2)
    with pytest.raises(ops.KernelError, match="expert_bias length"):
        ops.gpu_topk_route(lg, 2, DeviceBuffer.from_numpy(np.ones(3, np.float32)))


# ---- brute force ----------------------------------------------------------------------------------------

@pytest.mark.parametrize("T,E,K", [(4, 128, 8), (32, 128, 8), (128, 128, 8), (7, 8, 2), (33, 256, 8), (5, 200, 3), (1, 1, 1)])
def test_topk_route_matches_oracle(hip, T, E, K):
    rng = np.random.default_rng(T * 1000 + E + K)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, counts, off = _route(hip, logits, K)
    ridx, rw, rcounts, roff = model.topk_route(logits, K)
    assert np.array_equal(idx, ridx)
    assert np.array_equal(counts, rcounts) and np.array_equal(off, roff)
    assert np.array_equal(w, rw)  # kernel and oracle evaluate the softmax with the same sequence of f32 operations
    # brute force: stable argsort of the float64 softmax; weights: float64 softmax over the picked logits
    e64 = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    brute = np.argsort(-e64, axis=1, kind="stable")[:, :K]
    assert np.array_equal(idx, brute.reshape(-1).astype(np.uint32))
    sel = np.take_along_axis(e64, brute, axis=1)
    assert np.allclose(w.reshape(T, K), sel / sel.sum(axis=1, keepdims=True), rtol=0, atol=1e-6)


def test_topk_route_ties_go_to_lower_index(hip):
    logits = np.zeros((3, 130), np.float32)
    logits[1, [5, 70, 129]] = 1.0
    logits[2, :] = -3.0
    idx, w, _, _ = _route(hip, logits, 4)
    assert list(idx[:4]) == [0, 1, 2, 3]
    assert list(idx[4:8]) == [5, 70, 129, 0]
    assert list(idx[8:]) == [0, 1, 2, 3]
    assert np.allclose(w[:4], 0.25)


def test_topk_route_ranks_softmax_values(hip):
    """The reference ranks the f32 softmax value with strict > (topk_route.rs:283-300): logits whose softmax value
    underflows tie at 0.0 and go to the lowest free index, whatever their own order.  Expected picks written by hand."""
    logits = np.array([
        [0, -200, -150, -160, -170, -300, -120, -110],   # after expert 0 everything is 0.0 -> 1, 2
        [-500, -400, -300, -200, -100, 0, -450, -350],   # 5, then 0, 1
        [1, 1, 1, 1, 1, 1, 1, 1],                        # all equal -> 0, 1, 2
        [-100, -100, -100, 7, -100, -100, 7, -100],      # exact tie at the top, then an underflowing tail -> 3, 6, 0
    ], np.float32)
    want = np.array([[0, 1, 2], [5, 0, 1], [0, 1, 2], [3, 6, 0]], np.uint32)
    idx, w, counts, _ = _route(hip, logits, 3)
    assert np.array_equal(idx.reshape(4, 3), want)
    assert np.allclose(w.reshape(4, 3), [[1, 0, 0], [1, 0, 0], [1 / 3] * 3, [0.5, 0.5, 0]], atol=1e-6)
    assert np.array_equal(counts, np.bincount(want.reshape(-1), minlength=8))
    ridx, rw, _, _ = model.topk_route(logits, 3)
    assert np.array_equal(idx, ridx) and np.array_equal(w, rw)
    for r in range(4):  # the same rows reached through a wide expert_bias on all-zero logits
        idx_b, w_b, _, _ = _route(hip, np.zeros((1, 8), np.float32), 3, bias=logits[r])
        assert np.array_equal(idx_b, want[r]) and np.array_equal(w_b, w.reshape(4, 3)[r])
    # a wide row over all four expert slots of a lane (E = 256), ties far apart in index
    wide = np.full((2, 256), -300.0, np.float32)
    wide[0, [200, 13]] = [5.0, 4.0]
    wide[0, 100] = -250.0  # larger logit than the rest of the tail, same softmax value: must not be preferred
    wide[1, 255] = 0.0
    idx, _, _, _ = _route(hip, wide, 5)
    assert list(idx[:5]) == [200, 13, 0, 1, 2] and list(idx[5:]) == [255, 0, 1, 2, 3]
    assert np.array_equal(idx, model.topk_route(wide, 5)[0])


@pytest.mark.parametrize("A,E", [(32, 128), (256, 128), (1024, 128), (2500, 7), (1, 4), (4096, 256), (16384, 128), (20011, 1000), (3000, 1)])
def test_moe_sort_is_stable_argsort(hip, A, E):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(A + E)
    idx = rng.integers(0, E, size=A).astype(np.uint32)
    s, off = ops.moe_sort(DeviceBuffer.from_numpy(idx), E)
    rs, roff = model.moe_sort(idx, E)
    assert np.array_equal(s.numpy(), rs) and np.array_equal(off.numpy(), roff)


def test_moe_sort_equals_expert_dispatch_order(hip):
    """The on-device sort reproduces the host-side `expert_dispatch` build (moe.rs:1439-1447)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(3)
    T, K, E = 40, 8, 16
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    disp = model.expert_dispatch(idx, w, T, K, E)
    s, off = ops.moe_sort(DeviceBuffer.from_numpy(idx), E)
    s, off = s.numpy(), off.numpy()
    for e in range(E):
        assert [int(a) // K for a in s[off[e]:off[e + 1]]] == [tok for tok, _ in disp[e]]


# ---- data movement known answers (moe_kernels.rs:396-451) ---------------------------------------------------

def test_index_gather_and_scatter_weighted_add(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    src = np.arange(1, 13, dtype=np.float16).reshape(4, 3)
    out = ops.index_gather(DeviceBuffer.from_numpy(src), DeviceBuffer.from_numpy(np.array([2, 0, 3], np.uint32)))
    assert np.array_equal(out.numpy().reshape(-1), np.array([7, 8, 9, 1, 2, 3, 10, 11, 12], np.float16))
    src = np.array([[10, 20], [30, 40], [50, 60]], np.float16)
    dst = DeviceBuffer.from_numpy(np.zeros((2, 2), np.float16))
    ops.scatter_weighted_add(DeviceBuffer.from_numpy(src), dst, DeviceBuffer.from_numpy(np.array([0, 1, 0], np.uint32)),
                             DeviceBuffer.from_numpy(np.array([0.5, 1.0, 0.25], np.float32)))
    assert np.array_equal(dst.numpy(), np.array([[17.5, 25.0], [30.0, 40.0]], np.float16))


def test_silu_gate(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(4)
    g = (3 * rng.standard_normal(1001)).astype(np.float16)
    u = rng.standard_normal(1001).astype(np.float16)
    out = ops.silu_gate(DeviceBuffer.from_numpy(g), DeviceBuffer.from_numpy(u)).numpy().astype(np.float64)
    ref = model.silu(g.astype(np.float64)) * u.astype(np.float64)
    assert np.max(np.abs(out - ref)) <= 2e-3 * np.maximum(1.0, np.abs(ref)).max()


# ---- gather_qmm --------------------------------------------------------------------------------------------

def _gather_setup(rng, E, n, k, batch, mpb, dtype=np.float16):
    from rmlx_amd.runtime import DeviceBuffer
    words, s, b = make_weight(rng, n, k, 4, lead=(E,))
    x = rng.standard_normal((batch, mpb, k)).astype(dtype)
    idx = rng.integers(0, E, size=batch).astype(np.uint32)
    bufs = [DeviceBuffer.from_numpy(a) for a in (x, words, s, b, idx)]
    return words, s, b, x, idx, bufs


@pytest.mark.parametrize("E,n,k,batch,mpb", [(2, 4, 32, 2, 1), (4, 64, 512, 9, 1), (8, 128, 1024, 5, 3),
                                              (3, 48, 1536, 4, 11), (128, 1536, 4096, 32, 1), (6, 256, 2048, 7, 2),
                                              (5, 64, 640, 6, 3), (4, 48, 1408, 3, 8), (7, 32, 768, 9, 1),
                                              (5, 64, 960, 6, 3), (3, 48, 2880, 4, 11)])
def test_gather_qmm_matches_oracle(hip, E, n, k, batch, mpb):
    from rmlx_amd import ops
    rng = np.random.default_rng(E * 7 + n)
    gs = 32 if k == 32 else (128 if k == 2048 else 64)
    from rmlx_amd.runtime import DeviceBuffer
    words, s, b = make_weight(rng, n, k, 4, gs, lead=(E,))
    x = rng.standard_normal((batch, mpb, k)).astype(np.float16)
    idx = rng.integers(0, E, size=batch).astype(np.uint32)
    xd, wd, sd, bd, idd = [DeviceBuffer.from_numpy(a) for a in (x, words, s, b, idx)]
    out = ops.gather_qmm(xd, wd, sd, bd, idd, batch, mpb, n, k, E, gs).numpy()
    ref = model.gather_qmm(x, words, s, b, idx, gs)
    assert_close(out, ref, "gather_qmm")
    # f32 activations take the same path after a cast
    out32 = ops.gather_qmm(DeviceBuffer.from_numpy(x.astype(np.float32)), wd, sd, bd, idd, batch, mpb, n, k, E, gs).numpy()
    assert np.array_equal(out32, out)


@pytest.mark.parametrize("n,k,mpb", [(128, 1024, 1), (48, 512, 3), (256, 4096, 8), (64, 2048, 5)])
def test_gather_qmm_group_size_32_streams_on_the_wave_per_tile_kernel(hip, n, k, mpb):
    """Group size 32 with a few rows per entry: the wave-per-tile streaming kernel (automatic and forced) against the
    oracle and the portable kernel."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(n + k + mpb + 32)
    E, batch = 5, 7
    words, s, b = make_weight(rng, n, k, 4, 32, lead=(E,))
    x = rng.standard_normal((batch, mpb, k)).astype(np.float16)
    idx = rng.integers(0, E, size=batch).astype(np.uint32)
    xd, wd, sd, bd, idd = [DeviceBuffer.from_numpy(a) for a in (x, words, s, b, idx)]
    ref = model.gather_qmm(x, words, s, b, idx, 32)
    assert_close(ops.gather_qmm(xd, wd, sd, bd, idd, batch, mpb, n, k, E, 32).numpy(), ref, "gather_qmm gs32 (auto)")
    assert_close(ops.gather_qmm(xd, wd, sd, bd, idd, batch, mpb, n, k, E, 32, kernel=rt.GATHER_STREAM).numpy(), ref, "gather_qmm gs32 (streaming)")
    assert_close(ops.gather_qmm(xd, wd, sd, bd, idd, batch, mpb, n, k, E, 32, kernel=rt.GATHER_PORTABLE).numpy(), ref, "gather_qmm gs32 (portable)")


@pytest.mark.parametrize("n,k,gs,batch", [(64, 512, 64, 9), (8, 32, 32, 5), (256, 4096, 64, 33), (128, 1056, 32, 4), (48, 2048, 128, 7),
                                          (16384, 512, 64, 3), (64, 12288, 64, 2), (8, 64, 64, 70000)])
def test_gather_qmm_of_single_rows(hip, n, k, gs, batch):
    """One activation row per index (the reference's gather_qmv_fast_f16_q4 case): the single-row kernel with a weight
    matrix per activation row -- one launch, whole-row contiguous loads.  Against the oracle and the other kernels;
    repeated experts, the looping and the two-rows-per-wave forms, more entries than one grid dimension holds; on a
    stream, rows of an out-of-range index are zero."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer, Stream
    rng = np.random.default_rng(n + k + gs + batch)
    E = 6
    words, s, b = make_weight(rng, n, k, 4, gs, lead=(E,))
    x = rng.standard_normal((batch, 1, k)).astype(np.float16)
    idx = rng.integers(0, E, size=batch).astype(np.uint32)
    idx[: min(batch, 2)] = 3  # one expert twice
    print(f"gather_qmm single rows n={n} k={k} gs={gs} batch={batch}", flush=True)
    xd, wd, sd, bd = [DeviceBuffer.from_numpy(a) for a in (x, words, s, b)]
    ref = model.gather_qmm(x, words, s, b, idx, gs)
    out = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(idx), batch, 1, n, k, E, gs).numpy()
    assert_close(out, ref, "gather_qmm (single-row kernel)")
    if batch <= 64:
        port = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(idx), batch, 1, n, k, E, gs, kernel=rt.GATHER_PORTABLE).numpy()
        assert np.abs(out.astype(np.float64) - port.astype(np.float64)).max() <= model.tolerance(ref)
    bad = idx.copy()
    bad[batch // 2] = E + 3
    st = Stream()
    o = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(bad), batch, 1, n, k, E, gs, stream=st)
    st.sync()
    o = o.numpy()
    assert np.all(o[batch // 2] == 0)
    keep = np.arange(batch) != batch // 2
    assert np.array_equal(o[keep], out[keep])


def test_gather_qmm_validation(hip):
    """The reference's argument-validation tests (quantized.rs:11088-11540)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer, F32
    rng = np.random.default_rng(9)
    E, n, k, batch = 2, 4, 32, 2
    words = np.full((E, n, k // 8), 0x77777777, np.uint32)
    s = np.ones((E, n, 1), np.float16)
    b = np.zeros((E, n, 1), np.float16)
    x = np.ones((batch, 1, k), np.float32)
    xd, wd, sd, bd = [DeviceBuffer.from_numpy(a) for a in (x, words, s, b)]
    idx = DeviceBuffer.from_numpy(np.array([0, 1], np.uint32))
    out = ops.gather_qmm(xd, wd, sd, bd, idx, 2, 1, 4, 32, 2, 32).numpy()
    assert np.array_equal(out, np.full((2, 1, 4), 224.0, np.float16))  # valid inputs; all nibbles 7

    def bad(match, **kw):
        args = dict(x=xd, w=wd, s=sd, b=bd, idx=idx, batch=2, m=1, n=4, k=32, e=2, gs=32)
        args.update(kw)
        with pytest.raises(ops.KernelError, match=match):
            ops.gather_qmm(args["x"], args["w"], args["s"], args["b"], args["idx"], args["batch"], args["m"],
                           args["n"], args["k"], args["e"], args["gs"])

    bad("non-zero", x=DeviceBuffer((2, 1, 0), F32), k=0)
    bad("non-zero", n=0)
    bad("n_experts must be non-zero", e=0)
    bad("elements but expected", x=DeviceBuffer.from_numpy(np.ones((2, 1, 16), np.float32)))
    bad("must be even", x=DeviceBuffer.from_numpy(np.ones((2, 1, 31), np.float32)), k=31)
    bad("multiple of group_size", x=DeviceBuffer.from_numpy(np.ones((2, 1, 48), np.float32)), k=48)
    bad("w_packed_buf too small", w=DeviceBuffer.from_numpy(words[:1]))
    bad("scales_buf too small", s=DeviceBuffer.from_numpy(s[:1]))
    bad("biases_buf too small", b=DeviceBuffer.from_numpy(b[:1]))
    bad("out of range", idx=DeviceBuffer.from_numpy(np.array([0, 5], np.uint32)))
    bad("Float32 or Float16", x=DeviceBuffer.from_numpy(np.ones((2, 1, 32), np.uint32)))
    bad("indices must be UInt32", idx=DeviceBuffer.from_numpy(np.array([0, 1], np.float32)))
    bad("indices length", idx=DeviceBuffer.from_numpy(np.array([0, 1, 1], np.uint32)))
    # batch == 0 -> empty result (quantized.rs:10100-10103)
    out = ops.gather_qmm(DeviceBuffer((0, 1, 32), F32), wd, sd, bd, DeviceBuffer((0,), 3), 0, 1, 4, 32, 2, 32)
    assert out.shape == (0, 1, 4)


def test_gather_qmm_async_out_of_range_rows_are_zero(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer, Stream
    rng = np.random.default_rng(10)
    E, n, k, batch = 4, 64, 512, 6
    words, s, b = make_weight(rng, n, k, 4, lead=(E,))
    x = rng.standard_normal((batch, 1, k)).astype(np.float16)
    idx = np.array([0, 9, 3, 1, 7, 2], np.uint32)
    st = Stream()
    out = ops.gather_qmm(*[DeviceBuffer.from_numpy(a) for a in (x, words, s, b, idx)], batch, 1, n, k, E, 64, stream=st)
    st.sync()
    out = out.numpy()
    good = idx < E
    ref = model.gather_qmm(x[good], words, s, b, idx[good], 64)
    assert_close(out[good], ref, "valid rows")
    assert np.all(out[~good] == 0)


@pytest.mark.parametrize("n,k,mpb,gs", [(128, 512, 9, 64), (128, 512, 12, 64), (256, 1024, 17, 64), (384, 1024, 70, 64), (256, 512, 64, 64), (128, 1536, 129, 64),
                                        (128, 512, 40, 32), (256, 1024, 70, 128), (128, 768, 12, 64), (256, 640, 70, 64), (128, 1408, 40, 32),
                                        (192, 320, 40, 64), (64, 2880, 17, 64), (320, 448, 130, 32)])
def test_gather_qmm_many_rows_per_entry_on_the_grouped_gemm(hip, n, k, mpb, gs):
    """From 9 rows per batch entry on, gather_qmm multiplies with the grouped MFMA GEMMs (row tiles of 16, 32, 64 or 128 rows
    of one expert; the last tile of an entry ragged).  Against the oracle; on a stream, rows of an out-of-range index are zero."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer, Stream
    rng = np.random.default_rng(n + k + mpb)
    E, batch = 5, 6
    words, s, b = make_weight(rng, n, k, 4, gs, lead=(E,))
    x = rng.standard_normal((batch, mpb, k)).astype(np.float16)
    idx = np.array([4, 0, 3, 3, 1, 0], np.uint32)
    print(f"gather_qmm gemm n={n} k={k} mpb={mpb} gs={gs}", flush=True)
    xd, wd, sd, bd = [DeviceBuffer.from_numpy(a) for a in (x, words, s, b)]
    out = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(idx), batch, mpb, n, k, E, gs).numpy()
    ref = model.gather_qmm(x, words, s, b, idx, gs)
    assert_close(out, ref, "gather_qmm (GEMM)")
    if k % 128 == 0 and (gs != 32 or k % 512 == 0):  # (group sizes 64 and 128 on the K-split streaming GEMV, 32 on the wave-per-tile one: whole 512s)
        out_stream = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(idx), batch, mpb, n, k, E, gs, kernel=rt.GATHER_STREAM).numpy()
        assert_close(out_stream, ref, "gather_qmm (streaming GEMV)")
    out_port = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(idx), batch, mpb, n, k, E, gs, kernel=rt.GATHER_PORTABLE).numpy()
    assert_close(out_port, ref, "gather_qmm (portable)")
    bad = np.array([4, 9, 3, 7, 1, 0], np.uint32)
    st = Stream()
    out = ops.gather_qmm(xd, wd, sd, bd, DeviceBuffer.from_numpy(bad), batch, mpb, n, k, E, gs, stream=st)
    st.sync()
    out = out.numpy()
    good = bad < E
    assert_close(out[good], model.gather_qmm(x[good], words, s, b, bad[good], gs), "valid entries")
    assert np.all(out[~good] == 0)


# ---- expert FFN and the fused block ----------------------------------------------------------------------------

def _experts(rng, E, D, I, fused):
    from rmlx_amd import ops
    if fused:
        gu = make_weight(rng, 2 * I, D, 4, lead=(E,))
        gate = tuple(a[:, :I] for a in gu)
        up = tuple(a[:, I:] for a in gu)
        gate_h, up_h = ops.QuantizedWeight.from_numpy(*gu, 64, 4), None
    else:
        gate = make_weight(rng, I, D, 4, lead=(E,))
        up = make_weight(rng, I, D, 4, lead=(E,))
        gate_h, up_h = ops.QuantizedWeight.from_numpy(*gate, 64, 4), ops.QuantizedWeight.from_numpy(*up, 64, 4)
    down = make_weight(rng, D, I, 4, lead=(E,))
    down_h = ops.QuantizedWeight.from_numpy(*down, 64, 4)
    return gate, up, down, gate_h, up_h, down_h


@pytest.mark.parametrize("T,E,K,D,I", [(6, 8, 4, 512, 512), (20, 32, 4, 512, 512), (100, 4, 2, 512, 512), (12, 6, 2, 256, 384),
                                       (2, 64, 8, 1024, 512), (5, 128, 8, 512, 1024)])
def test_moe_forward_grouped_skips_out_of_range_experts(hip, T, E, K, D, I):
    """Caller-supplied expert ids outside [0, E) contribute nothing (the reference's combine skips them,
    crates/rmlx-distributed/src/moe_exchange.rs:2305): one-wave grouping (<= 64 assignments), the workgroup-wide
    grouping below and above the grouped-GEMM threshold, the portable kernels (D, I no multiples of 512), and the form
    without grouping that a few tokens take (the last two cases)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(T + E + K + D)
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, False)
    x = make_x(rng, T, D)
    idx = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint32).reshape(-1)
    w = rng.uniform(0.1, 1.0, T * K).astype(np.float32)
    bad = rng.choice(T * K, size=max(2, T * K // 7), replace=False)
    idx_bad = idx.copy()
    idx_bad[bad] = np.where(np.arange(bad.size) % 2 == 0, E, 0xFFFFFFFF).astype(np.uint32)
    w_ref = w.copy()
    w_ref[bad] = 0.0
    ref = model.moe_forward(x, idx, w_ref, gate, up, down, 64, K)
    print(f"out-of-range experts T={T} E={E} K={K} D={D} I={I} bad={sorted(bad.tolist())}", flush=True)
    out = ops.moe_forward_grouped(gh, uh, dh, DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(idx_bad),
                                  DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out, ref, "out-of-range experts skipped")


@pytest.mark.parametrize("T,E,K", [(1, 128, 8), (8, 128, 8), (7, 200, 3), (8, 256, 8), (3, 5, 5), (9, 128, 7)])
def test_moe_forward_routes_like_the_two_step_path(hip, T, E, K):
    """Up to 8 tokens / 64 assignments with f32 logits, routing and grouping share one launch: the picks must
    be those of routing alone, and the result that of calling the grouped block with them -- with and without
    an expert bias, and also for an f16 bias (which takes the two-step path inside)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(T * 31 + E + K)
    D, I = 512, 512
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, False)
    xd = DeviceBuffer.from_numpy(make_x(rng, T, D))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[0, : min(E, 3)] = 1.5  # ties go to the lower index on both paths
    ld = DeviceBuffer.from_numpy(logits)
    for bias in (None, rng.standard_normal(E).astype(np.float32), rng.standard_normal(E).astype(np.float16)):
        bd = DeviceBuffer.from_numpy(bias) if bias is not None else None
        print(f"moe route T={T} E={E} K={K} bias={None if bias is None else bias.dtype}", flush=True)
        one = ops.moe_forward(gh, uh, dh, xd, ld, K, expert_bias=bd).numpy()
        r = ops.gpu_topk_route(ld, K, expert_bias=bd)
        two = ops.moe_forward_grouped(gh, uh, dh, xd, r.expert_indices, r.expert_weights, K).numpy()
        idx, w, _, _ = model.topk_route(logits, K, bias=None if bias is None else bias.astype(np.float32))
        assert np.array_equal(r.expert_indices.numpy(), idx)
        ref = model.moe_forward(xd.numpy(), idx, w, gate, up, down, 64, K)
        assert_close(one, ref, "moe_forward")
        assert_close(two, ref, "moe_forward_grouped")
        # (the one-call path knows its picks are distinct per token and may run kernels built for fewer rows
        # per expert than the grouped entry point, which must allow for repeated experts: same picks, same
        # weights, results within the tolerance of each other rather than bit-equal)
        assert np.abs(one.astype(np.float64) - two.astype(np.float64)).max() <= model.tolerance(ref)


@pytest.mark.parametrize("T,K,E,D,I,fused", [(1, 8, 16, 1024, 1536, True), (1, 1, 4, 512, 512, False), (2, 7, 16, 512, 1024, True),
                                              (3, 5, 8, 2048, 512, False), (2, 8, 32, 1024, 512, True), (4, 8, 128, 512, 1024, True),
                                              (9, 8, 128, 512, 1024, True), (16, 2, 64, 512, 512, False), (12, 8, 128, 512, 512, True),
                                              (10, 1, 16, 512, 512, True)])
def test_moe_forward_of_a_few_tokens(hip, T, K, E, D, I, fused):
    """While the assignments are at most 1.3 x the distinct experts a uniform router would pick, they are not grouped.
    Fewer than 16: a routing launch, then the gate / up projection on the single-row kernel (a wave per pair of gate and
    up rows of the assignment's expert); from 16 on the gate / up workgroups rank their token's experts themselves (any
    number of tokens).  The last cases lie past those bounds: more than 8 tokens that route with the routing kernel and
    are grouped.  All against the oracle and against the two-step path."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(T * 100 + K * 10 + E)
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, fused)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[0, : min(E, 2)] = logits[0].max() + 1.0  # a tie at the top: the lower index first on every path
    xd, ld = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits)
    for bias in (None, rng.standard_normal(E).astype(np.float32)):
        print(f"few tokens T={T} K={K} E={E} D={D} I={I} fused={fused} bias={bias is not None}", flush=True)
        bd = DeviceBuffer.from_numpy(bias) if bias is not None else None
        one = ops.moe_forward(gh, uh, dh, xd, ld, K, expert_bias=bd).numpy()
        idx, w, _, _ = model.topk_route(logits, K, bias=bias)
        ref = model.moe_forward(x, idx, w, gate, up, down, 64, K)
        assert_close(one, ref, "moe_forward")
        r = ops.gpu_topk_route(ld, K, expert_bias=bd)
        assert np.array_equal(r.expert_indices.numpy(), idx)
        two = ops.moe_forward_grouped(gh, uh, dh, xd, r.expert_indices, r.expert_weights, K).numpy()
        assert np.abs(one.astype(np.float64) - two.astype(np.float64)).max() <= model.tolerance(ref)


@pytest.mark.parametrize("bits,gs", [(8, 64), (8, 32), (8, 128), (4, 32), (4, 128)])
@pytest.mark.parametrize("T,K,E,D,I", [(1, 8, 16, 1024, 512), (3, 4, 32, 512, 1024), (2, 8, 16, 512, 1536), (2, 3, 8, 512, 2560)])
def test_moe_forward_of_a_few_tokens_other_formats(hip, bits, gs, T, K, E, D, I):
    """The form without grouping for 8-bit experts and for group sizes 32 / 128: gate / up on the single-row kernel; the down
    projection of 8-bit experts with the combine behind it on the single-row layout (intermediate dimension up to one / two
    wave-wide chunks: 512, 1024 / 1536), else as a single-row gather and the weighted sum of a token's rows in a launch of
    its own.  Against the oracle, with logits and with the caller's picks, and through ExpertGroup with one row per item."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits * 1000 + gs + T)
    gu = make_weight(rng, 2 * I, D, bits, gs, lead=(E,))
    down = make_weight(rng, D, I, bits, gs, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), ops.QuantizedWeight.from_numpy(*down, gs, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=bits)
    print(f"few tokens Q{bits} gs{gs} T={T} K={K} E={E} D={D} I={I}", flush=True)
    xd = DeviceBuffer.from_numpy(x)
    assert_close(ops.moe_forward(gh, None, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward")
    bad = idx.copy().reshape(-1)
    w_ref = w.copy().reshape(-1)
    bad[1 % bad.size] = E + 7
    w_ref[1 % bad.size] = 0.0
    out = ops.moe_forward_grouped(gh, None, dh, xd, DeviceBuffer.from_numpy(bad.astype(np.uint32)), DeviceBuffer.from_numpy(w.reshape(-1)), K).numpy()
    assert_close(out, model.moe_forward(x, idx, w_ref.reshape(w.shape), gate, up, down, gs, K, bits=bits), "moe_forward_grouped, one pick out of range")
    group = ops.ExpertGroup(gh, None, dh)
    items = [(int(e), x[:1]) for e in idx.reshape(-1)[:3]]
    for (e, xi), (_, y) in zip(items, group.grouped_forward([(e, DeviceBuffer.from_numpy(xi)) for e, xi in items])):
        one = model.moe_forward(xi, np.array([[e]]), np.ones((1, 1), np.float32), gate, up, down, gs, 1, bits=bits)
        assert_close(y, one, f"ExpertGroup expert {e}")


@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("T,K,E,D,I,fused", [(1, 8, 16, 1024, 512, True), (3, 4, 32, 512, 1024, False), (2, 2, 8, 4096, 1536, True)])
def test_moe_forward_of_a_few_tokens_two_bit_experts(hip, gs, T, K, E, D, I, fused):
    """2-bit experts, a few tokens: the form without grouping on the 2-bit single-row kernel with a weight matrix per row
    (gate / up, SwiGLU, down, weighted sum).  Against the oracle, with logits and with the caller's picks (one of them out
    of range), stacked and separate gate / up weights."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(gs * 10 + T + E)
    if fused:
        gu = _two_bit(rng, E, 2 * I, D, gs)
        gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
        gh, uh = ops.QuantizedWeight.from_numpy(*gu, gs, 2), None
    else:
        gate, up = _two_bit(rng, E, I, D, gs), _two_bit(rng, E, I, D, gs)
        gh, uh = ops.QuantizedWeight.from_numpy(*gate, gs, 2), ops.QuantizedWeight.from_numpy(*up, gs, 2)
    down = _two_bit(rng, E, D, I, gs)
    dh = ops.QuantizedWeight.from_numpy(*down, gs, 2)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=2)
    print(f"few tokens Q2 gs{gs} T={T} K={K} E={E} D={D} I={I} fused={fused}", flush=True)
    xd = DeviceBuffer.from_numpy(x)
    assert_close(ops.moe_forward(gh, uh, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward")
    bad = idx.copy().reshape(-1)
    w_ref = w.copy().reshape(-1)
    bad[-1] = E + 1
    w_ref[-1] = 0.0
    out = ops.moe_forward_grouped(gh, uh, dh, xd, DeviceBuffer.from_numpy(bad.astype(np.uint32)), DeviceBuffer.from_numpy(w.reshape(-1)), K).numpy()
    assert_close(out, model.moe_forward(x, idx, w_ref.reshape(w.shape), gate, up, down, gs, K, bits=2), "moe_forward_grouped, one pick out of range")


@pytest.mark.parametrize("bits,gs,D,I", [(4, 32, 1056, 800), (4, 64, 2880, 2880), (8, 32, 512, 1024), (8, 64, 1088, 576)])
@pytest.mark.parametrize("T", [3, 40])
def test_moe_forward_of_shapes_without_a_grouped_kernel(hip, bits, gs, D, I, T):
    """Expert dimensions off the multiples of 512 / 256 (e.g. a hidden size of 2880) and 8-bit weights at group size 32:
    no chunked or grouped fast kernel takes them, the single-row kernels do (K % 32 == 0, N % 8 == 0), so the form without
    grouping runs them at every batch size.  Against the oracle, with logits and with the caller's picks."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits + gs + D + T)
    E, K = 6, 2
    gu = make_weight(rng, 2 * I, D, bits, gs, lead=(E,))
    down = make_weight(rng, D, I, bits, gs, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), ops.QuantizedWeight.from_numpy(*down, gs, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=bits)
    print(f"no grouped kernel Q{bits} gs{gs} D={D} I={I} T={T}", flush=True)
    xd = DeviceBuffer.from_numpy(x)
    assert_close(ops.moe_forward(gh, None, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward")
    out = ops.moe_forward_grouped(gh, None, dh, xd, DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out, ref, "moe_forward_grouped")


@pytest.mark.parametrize("bits,gs,D,I", [(4, 64, 512, 384), (4, 64, 1024, 640), (4, 64, 2048, 768), (4, 64, 768, 1408),
                                         (8, 64, 1024, 640), (4, 32, 1024, 640), (8, 32, 640, 384), (4, 128, 1024, 640)])
@pytest.mark.parametrize("T", [3, 24, 70, 300])
def test_moe_forward_of_dimensions_in_whole_blocks_of_128(hip, bits, gs, D, I, T):
    """Expert dimensions that are multiples of 128 but not of 512 (an intermediate size of 768 or 1408): the K-split
    streaming GEMV walks whole slabs of 128 with a shorter last part, the grouped GEMM pads its last unrolled round with
    zero activations (group sizes 32 and 64).  3 tokens run the form without grouping, 24 the streaming chunks (group size
    32, which has none for these rows: the GEMM), 70 and 300 the grouped GEMM on 32- and 64-row tiles; group size 128 has no
    tail form and stays on the streaming chunks.  Against the oracle, with logits and with the caller's picks."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits + gs + D + I + T)
    E, K = 8, 2
    gu = make_weight(rng, 2 * I, D, bits, gs, lead=(E,))
    down = make_weight(rng, D, I, bits, gs, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), ops.QuantizedWeight.from_numpy(*down, gs, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=bits)
    print(f"blocks of 128 Q{bits} gs={gs} D={D} I={I} T={T}", flush=True)
    xd = DeviceBuffer.from_numpy(x)
    assert_close(ops.moe_forward(gh, None, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward")
    out = ops.moe_forward_grouped(gh, None, dh, xd, DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out, ref, "moe_forward_grouped")
    if bits == 4:  # every streaming / tile choice the handle offers
        for min_rows, kind in ((0, 1), (1, 0)):
            gh.set_expert_gemm_min_rows(min_rows)
            gh.set_expert_stream_kernel(kind)
            out = ops.moe_forward_grouped(gh, None, dh, xd, DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w), K).numpy()
            assert_close(out, ref, f"moe_forward_grouped min_rows={min_rows} stream kernel {kind}")


@pytest.mark.parametrize("bits,gs,D,I", [(4, 64, 1024, 512), (8, 64, 512, 768), (4, 32, 512, 640)])
@pytest.mark.parametrize("T", [1, 3, 40])
def test_moe_forward_of_bf16_activations(hip, bits, gs, D, I, T):
    """bf16 activations: a few tokens are converted inside the gate / up kernel of the form without grouping while it stages
    them (no cast launch), larger batches by a cast in front.  Bit-identical to the same call over the rows converted on the
    host (through f32, round to nearest even), and on the oracle."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import BF16, DeviceBuffer
    rng = np.random.default_rng(bits + gs + D + I + T)
    E, K = 8, 2
    gu = make_weight(rng, 2 * I, D, bits, gs, lead=(E,))
    down = make_weight(rng, D, I, bits, gs, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), ops.QuantizedWeight.from_numpy(*down, gs, bits)
    xb = make_x(rng, T, D, "bf16")
    x16 = model.bf16_bits_to_f32(xb).astype(np.float16)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ld = DeviceBuffer.from_numpy(logits)
    print(f"moe bf16 Q{bits} gs{gs} D={D} I={I} T={T}", flush=True)
    got = ops.moe_forward(gh, None, dh, DeviceBuffer.from_numpy(xb, BF16), ld, K).numpy()
    want = ops.moe_forward(gh, None, dh, DeviceBuffer.from_numpy(x16), ld, K).numpy()
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert_close(got, model.moe_forward(x16, idx, w, gate, up, down, gs, K, bits=bits), "bf16 activations")
    got2 = ops.moe_forward_grouped(gh, None, dh, DeviceBuffer.from_numpy(xb, BF16), DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w), K).numpy()
    assert np.array_equal(got2.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("bits,gs,D,I,fused", [(4, 64, 320, 448, True), (4, 64, 2880, 960, True), (8, 64, 576, 320, False),
                                               (4, 32, 448, 320, True), (4, 128, 384, 640, False), (4, 64, 768, 320, True), (8, 64, 512, 1088, True)])
@pytest.mark.parametrize("T", [24, 70, 200, 400])
def test_moe_forward_on_the_grouped_lds_staged_gemm(hip, bits, gs, D, I, fused, T):
    """Expert dimensions in multiples of 64 that are no multiples of 128 (a hidden size of 2880): from one row per expert on
    the block groups the rows into tiles of 64 rows of one expert and multiplies them with the grouped form of the
    LDS-staged GEMM (activations re-laid through the token map, K padded to whole iterations, SwiGLU and combine as passes
    of their own).  Stacked and separate gate / up weights, every group size, experts with no rows, with one row and with
    more than a tile (tiles of 128 rows from 64 rows per expert on: T = 400); an expert index out of range gives zeros.  Against the oracle."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits + gs + D + I + T)
    E, K = 7, 2
    gu = make_weight(rng, 2 * I, D, bits, gs, lead=(E,))
    down = make_weight(rng, D, I, bits, gs, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(np.ascontiguousarray(a[:, I:]) for a in gu)
    if fused:
        gh, uh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), None
    else:
        gh = ops.QuantizedWeight.from_numpy(*(np.ascontiguousarray(a) for a in gate), gs, bits)
        uh = ops.QuantizedWeight.from_numpy(*up, gs, bits)
    dh = ops.QuantizedWeight.from_numpy(*down, gs, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 5] -= 20.0          # expert 5 gets no rows
    logits[: T // 2, 2] += 4.0    # expert 2 gets half the batch: more than one tile at T = 200 and T = 400
    idx, w, counts, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=bits)
    print(f"grouped LDS GEMM Q{bits} gs{gs} D={D} I={I} fused={fused} T={T} counts={counts.tolist()}", flush=True)
    xd = DeviceBuffer.from_numpy(x)
    assert_close(ops.moe_forward(gh, uh, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward")
    out = ops.moe_forward_grouped(gh, uh, dh, xd, DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out, ref, "moe_forward_grouped")
    bad = idx.copy()
    bad[3] = E + 2
    w_ref = w.copy()
    w_ref[3] = 0.0
    from rmlx_amd.runtime import Stream
    st = Stream()
    out = ops.moe_forward_grouped(gh, uh, dh, xd, DeviceBuffer.from_numpy(bad), DeviceBuffer.from_numpy(w), K, stream=st)
    st.sync()
    idx_ok = np.where(bad < E, bad, 0).astype(np.uint32)
    assert_close(out.numpy(), model.moe_forward(x, idx_ok, w_ref, gate, up, down, gs, K, bits=bits), "one pick out of range")


@pytest.mark.parametrize("T,K", [(1, 2), (1, 8), (2, 3), (3, 4)])
def test_moe_forward_grouped_with_repeated_experts(hip, T, K):
    """Caller-supplied picks may name one expert several times for a token; decode-sized batches run kernels
    built for few rows per expert, whose bound must then count assignments, not tokens."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(T * 10 + K)
    E, D, I = 6, 512, 1024
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, False)
    x = make_x(rng, T, D)
    idx = np.full(T * K, 4, np.uint32)   # every assignment goes to expert 4
    idx[-1] = 1
    w = rng.uniform(0.1, 1.0, size=T * K).astype(np.float32)
    out = ops.moe_forward_grouped(gh, uh, dh, DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(idx),
                                  DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out, model.moe_forward(x, idx, w, gate, up, down, 64, K), "repeated experts")


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("T,E,K,D,I", [(1, 4, 2, 512, 512), (9, 8, 2, 1024, 512), (40, 6, 3, 512, 1536), (64, 4, 4, 512, 512)])
def test_moe_forward_small(hip, fused, T, E, K, D, I):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(T + E + D)
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, fused)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, K)
    out = ops.moe_forward(gh, uh, dh, DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits), K).numpy()
    assert_close(out, ref, "moe_forward")
    # routing on the device followed by the grouped block == the one-call entry point
    r = ops.gpu_topk_route(DeviceBuffer.from_numpy(logits), K)
    assert np.array_equal(r.expert_indices.numpy(), idx)
    out2 = ops.moe_forward_grouped(gh, uh, dh, DeviceBuffer.from_numpy(x), r.expert_indices, r.expert_weights, K).numpy()
    if T > 8:  # (smaller batches: the one-call path may run kernels built for fewer rows per expert)
        assert np.array_equal(out, out2)
    assert_close(out2, ref, "moe_forward_grouped with device routing")
    out3 = ops.moe_forward_grouped(gh, uh, dh, DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(idx),
                                   DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out3, ref, "moe_forward_grouped with host routing")


def test_random_moe_shapes(hip):
    """Twenty seeded random (T, E, K, D, I, fused, bias) blocks through the one-call entry point."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(20250101)
    for case in range(20):
        E = int(rng.integers(1, 40))
        K = int(rng.integers(1, min(8, E) + 1))
        T = int(rng.choice([1, 2, 3, 5, 8, 9, 17, 40]))
        D, I = int(rng.integers(1, 4)) * 512, int(rng.integers(1, 4)) * 512
        fused = bool(rng.integers(0, 2))
        gate, up, down, gh, uh, dh = _experts(rng, E, D, I, fused)
        x = make_x(rng, T, D)
        logits = (2.0 * rng.standard_normal((T, E))).astype(np.float32)
        bias = rng.standard_normal(E).astype(np.float32) if rng.integers(0, 2) else None
        print(f"moe case {case}: T={T} E={E} K={K} D={D} I={I} fused={fused} bias={bias is not None}", flush=True)
        out = ops.moe_forward(gh, uh, dh, DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits), K,
                              expert_bias=DeviceBuffer.from_numpy(bias) if bias is not None else None).numpy()
        idx, w, _, _ = model.topk_route(logits, K, bias=bias)
        assert_close(out, model.moe_forward(x, idx, w, gate, up, down, 64, K), f"case {case}")


@pytest.mark.parametrize("bits,gs,D,I,fused", [(8, 64, 512, 512, False), (4, 32, 512, 1024, True), (4, 128, 384, 640, False),
                                               (8, 32, 96, 160, True), (2, 64, 256, 128, False),
                                               (4, 128, 512, 1024, True), (4, 128, 1024, 1536, False),   # streaming kernels, group 128
                                               (8, 64, 1024, 1536, True), (8, 64, 4096, 768, False),    # streaming 8-bit kernel
                                               (8, 128, 512, 1024, True), (8, 128, 1024, 768, False),   # ... at group size 128
                                               (4, 32, 1024, 1536, False), (4, 32, 2048, 512, True)])   # wave-per-tile kernel, group 32
def test_moe_other_bit_widths_and_group_sizes(hip, bits, gs, D, I, fused):
    """Expert weights beyond 4 bits / group 64: 8-bit (group 64 / 128) and 4-bit group 128 weights stream through the
    K-split kernels and 4-bit group 32 weights through the wave-per-tile kernel when the dimensions allow; 2-bit
    weights, 8-bit weights at group size 32 and other dimensions run the same block on the portable kernels.  Routed block (one call and grouped) and `ExpertGroup::grouped_forward`,
    against the oracle."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits * 100 + gs + D)
    E, T, K = 5, 21 if D >= 1024 or (gs == 128 and D % 512 == 0) else 6, 2

    def weight(n, k):
        return make_weight(rng, n, k, bits if bits != 2 else 4, gs, lead=(E,)) if bits != 2 else _two_bit(rng, E, n, k, gs)

    if fused:
        gu = weight(2 * I, D)
        gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
        gh, uh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), None
    else:
        gate, up = weight(I, D), weight(I, D)
        gh, uh = ops.QuantizedWeight.from_numpy(*gate, gs, bits), ops.QuantizedWeight.from_numpy(*up, gs, bits)
    down = weight(D, I)
    dh = ops.QuantizedWeight.from_numpy(*down, gs, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=bits)
    xd = DeviceBuffer.from_numpy(x)
    print(f"portable moe bits={bits} gs={gs} D={D} I={I} fused={fused}", flush=True)
    assert_close(ops.moe_forward(gh, uh, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward")
    assert_close(ops.moe_forward_grouped(gh, uh, dh, xd, DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w), K).numpy(),
                 ref, "moe_forward_grouped")
    group = ops.ExpertGroup(gh, uh, dh)
    items = [(3, make_x(rng, 2, D)), (0, make_x(rng, 5, D))]
    outs = group.grouped_forward([(e, DeviceBuffer.from_numpy(v)) for e, v in items])
    for (e, v), (_, yv) in zip(items, outs):
        ones = np.ones((len(v), 1))
        assert_close(yv, model.moe_forward(v, np.full((len(v), 1), e), ones, gate, up, down, gs, 1, bits=bits), f"expert {e}")


@pytest.mark.parametrize("T", [150, 50])
@pytest.mark.parametrize("bits,gs,D,I,fused", [(4, 64, 512, 512, True), (4, 64, 1024, 1536, False), (8, 64, 512, 1024, True),
                                               (8, 64, 1024, 512, False), (4, 32, 512, 1024, True), (4, 128, 1024, 512, False),
                                               (8, 32, 512, 512, False), (8, 128, 512, 512, True)])
def test_moe_many_rows_per_expert_on_the_grouped_gemm(hip, bits, gs, D, I, fused, T):
    """Batches with many rows per expert (here 75 or 25 on average; from 6 on) multiply with the grouped MFMA GEMM: row
    tiles of 64 rows of one expert (32 rows while the average is at most 32).  Skewed routing gives one expert
    three tiles, another a ragged one and one almost nothing.  Group sizes 32, 64 and 128.  Checked against the
    oracle, and the path below the threshold (streaming GEMV, or the portable kernels where it does not take the
    group size) on the same inputs beside it."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits * 1000 + D + I + T + gs)
    E, K = 4, 2

    def weight(n, k):
        return make_weight(rng, n, k, bits, gs, lead=(E,))

    if fused:
        gu = weight(2 * I, D)
        gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
        gh, uh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), None
    else:
        gate, up = weight(I, D), weight(I, D)
        gh, uh = ops.QuantizedWeight.from_numpy(*gate, gs, bits), ops.QuantizedWeight.from_numpy(*up, gs, bits)
    down = weight(D, I)
    dh = ops.QuantizedWeight.from_numpy(*down, gs, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] += 3.0
    logits[:, 3] -= 4.0
    idx, w, counts, _ = model.topk_route(logits, K)
    assert counts.max() > (128 if T == 150 else 32) and counts.min() < 8, counts
    ref = model.moe_forward(x, idx, w, gate, up, down, gs, K, bits=bits)
    xd, idxd, wd = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w)
    print(f"grouped gemm moe T={T} bits={bits} gs={gs} D={D} I={I} fused={fused} counts={counts.tolist()}", flush=True)
    prev = gh.set_expert_gemm_min_rows(6)
    try:
        out_gemm = ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, K).numpy()
        assert_close(out_gemm, ref, "moe_forward_grouped (GEMM)")
        assert_close(ops.moe_forward(gh, uh, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward (GEMM)")
        group = ops.ExpertGroup(gh, uh, dh)
        sizes = (70, 1, 64, 33, 129) if T == 150 else (20, 1, 32, 33, 40)
        items = [(e, make_x(rng, m, D)) for e, m in zip((3, 0, 2, 3, 1), sizes)]
        outs = group.grouped_forward([(e, DeviceBuffer.from_numpy(v)) for e, v in items])
        for (e, v), (_, yv) in zip(items, outs):
            ones = np.ones((len(v), 1))
            assert_close(yv, model.moe_forward(v, np.full((len(v), 1), e), ones, gate, up, down, gs, 1, bits=bits),
                         f"ExpertGroup (GEMM) expert {e} rows {len(v)}")
        gh.set_expert_gemm_min_rows(0)
        out_stream = ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, K).numpy()
        assert_close(out_stream, ref, "moe_forward_grouped (below the threshold)")
    finally:
        gh.set_expert_gemm_min_rows(prev)


@pytest.mark.parametrize("E,K,T,x_dtype", [(1, 1, 100, "f16"), (3, 3, 40, "f32"), (2, 1, 129, "f16"), (6, 2, 33, "f32")])
def test_grouped_gemm_edge_routings(hip, E, K, T, x_dtype):
    """Corner cases of the routed block above the GEMM threshold: a single expert, every expert for every token,
    one row more than two full tiles, f32 activations (cast on the way in)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(E * 100 + K * 10 + T)
    D, I = 512, 512
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, E % 2 == 0)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    idx, w, counts, _ = model.topk_route(logits, K)
    assert T * K >= 8 * E
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, K)
    xin = x if x_dtype == "f16" else x.astype(np.float32)
    print(f"grouped gemm edge E={E} K={K} T={T} x={x_dtype} counts={counts.tolist()}", flush=True)
    out = ops.moe_forward_grouped(gh, uh, dh, DeviceBuffer.from_numpy(xin), DeviceBuffer.from_numpy(idx),
                                  DeviceBuffer.from_numpy(w), K).numpy()
    assert_close(out, ref, "moe_forward_grouped")
    out2 = ops.moe_forward(gh, uh, dh, DeviceBuffer.from_numpy(xin), DeviceBuffer.from_numpy(logits), K).numpy()
    assert_close(out2, ref, "moe_forward")  # (routing weights from the device: equal to the oracle's up to f32 rounding)


def _two_bit(rng, E, n, k, gs):
    words = rng.integers(0, 2**32, size=(E, n, k // 16), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.02, 0.08, size=(E, n, k // gs)).astype(np.float16)
    return words, scales, (-1.5 * scales.astype(np.float32)).astype(np.float16)


def test_grouped_forward_equals_per_expert_loop(hip):
    """grouped == individual (expert_group.rs:972-1019), against the float64 expert FFN."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(21)
    E, D, I = 5, 512, 1024
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, False)
    group = ops.ExpertGroup(gh, uh, dh)
    assert group.grouped_forward([]) == []
    items = [(3, make_x(rng, 2, D)), (0, make_x(rng, 11, D)), (3, make_x(rng, 1, D)), (4, make_x(rng, 8, D))]
    outs = group.grouped_forward([(e, DeviceBuffer.from_numpy(x)) for e, x in items])
    assert [e for e, _ in outs] == [3, 0, 3, 4]
    for (e, x), (_, y) in zip(items, outs):
        xe = x.astype(np.float64)
        g = xe @ model.dequantize(gate[0][e], gate[1][e], gate[2][e], 64, 4).T
        u = xe @ model.dequantize(up[0][e], up[1][e], up[2][e], 64, 4).T
        h = (model.silu(g) * u).astype(np.float16).astype(np.float64)
        ref = h @ model.dequantize(down[0][e], down[1][e], down[2][e], 64, 4).T
        assert_close(y, ref, f"expert {e}")
    with pytest.raises(ops.KernelError, match="expert_idx 9 >= num_experts 5"):
        group.grouped_forward([(9, DeviceBuffer.from_numpy(make_x(rng, 1, D)))])
    with pytest.raises(ops.KernelError, match="input dim"):
        group.grouped_forward([(0, DeviceBuffer.from_numpy(make_x(rng, 1, D + 512)))])


@pytest.mark.parametrize("E,D,I,fused,n_items", [(16, 1024, 1536, True, 8), (6, 512, 512, False, 1), (128, 512, 1024, True, 40)])
def test_grouped_forward_of_single_rows(hip, E, D, I, fused, n_items):
    """Every item one row (a decoding token's experts, the same expert allowed twice): both projections on the single-row
    kernel.  Against the float64 expert FFN and against the same items with one row more on the first (which takes the
    streaming kernels over chunks)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(E + D + n_items)
    gate, up, down, gh, uh, dh = _experts(rng, E, D, I, fused)
    group = ops.ExpertGroup(gh, uh, dh)
    experts = rng.integers(0, E, size=n_items)
    if n_items > 1:
        experts[1] = experts[0]
    items = [(int(e), make_x(rng, 1, D)) for e in experts]
    print(f"ExpertGroup single rows E={E} D={D} I={I} fused={fused} items={n_items}", flush=True)
    outs = group.grouped_forward([(e, DeviceBuffer.from_numpy(x)) for e, x in items])
    assert [e for e, _ in outs] == [e for e, _ in items]
    refs = []
    for (e, x), (_, y) in zip(items, outs):
        xe = x.astype(np.float64)
        g = xe @ model.dequantize(gate[0][e], gate[1][e], gate[2][e], 64, 4).T
        u = xe @ model.dequantize(up[0][e], up[1][e], up[2][e], 64, 4).T
        h = (model.silu(g) * u).astype(np.float16).astype(np.float64)
        refs.append(h @ model.dequantize(down[0][e], down[1][e], down[2][e], 64, 4).T)
        assert_close(y, refs[-1], f"expert {e}")
    first = np.concatenate([items[0][1], make_x(rng, 1, D)])
    outs2 = group.grouped_forward([(items[0][0], DeviceBuffer.from_numpy(first))] + [(e, DeviceBuffer.from_numpy(x)) for e, x in items[1:]])
    for (_, y), (_, y2), ref in zip(outs, outs2, refs):
        assert np.abs(y.astype(np.float64) - y2[:1].astype(np.float64)).max() <= 0.5 * model.tolerance(ref)


@pytest.mark.parametrize("bits,gs,D,I", [(4, 64, 960, 2880), (8, 32, 544, 96), (4, 32, 1056, 800)])
def test_grouped_forward_of_shapes_without_a_grouped_kernel(hip, bits, gs, D, I):
    """ExpertGroup over expert dimensions that no chunked or grouped kernel takes (off the multiples of 128, 8-bit at group
    size 32 with short rows): every row multiplies with its own expert on the single-row kernels instead of the portable ones.
    Items of 1, 5, 17 and 40 rows, an expert named twice; then items of 1, 150 and 200 rows.  Against the float64 expert FFN."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits + gs + D + I)
    E = 5
    gu = make_weight(rng, 2 * I, D, bits, gs, lead=(E,))
    down = make_weight(rng, D, I, bits, gs, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, gs, bits), ops.QuantizedWeight.from_numpy(*down, gs, bits)
    group = ops.ExpertGroup(gh, None, dh)
    # (the second set: 64 rows per item and more on average, where dimensions in multiples of 64 take row tiles of 128 rows)
    for counts in (((3, 1), (0, 5), (3, 17), (4, 40)), ((3, 1), (0, 150), (4, 200))):
        items = [(e, make_x(rng, m, D)) for e, m in counts]
        print(f"ExpertGroup without a grouped kernel Q{bits} gs{gs} D={D} I={I} items {counts}", flush=True)
        outs = group.grouped_forward([(e, DeviceBuffer.from_numpy(x)) for e, x in items])
        for (e, x), (e2, y) in zip(items, outs):
            assert e == e2
            ones = np.ones((len(x), 1))
            assert_close(y, model.moe_forward(x, np.full((len(x), 1), e), ones, gate, up, down, gs, 1, bits=bits), f"expert {e} rows {len(x)}")


@pytest.fixture(scope="module")
def config5(hip):
    """Config 5 weights: 128 experts, hidden 4096, intermediate 1536, fused gate/up, Q4 group 64."""
    rng = np.random.default_rng(1005)
    return _experts(rng, 128, 4096, 1536, True)


@pytest.mark.parametrize("T", [4, 32, 128])
def test_config5_moe(hip, config5, T):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    gate, up, down, gh, uh, dh = config5
    rng = np.random.default_rng(5000 + T)
    x = make_x(rng, T, 4096)
    logits = rng.standard_normal((T, 128)).astype(np.float32)
    out = ops.moe_forward(gh, uh, dh, DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits), 8).numpy()
    idx, w, _, _ = model.topk_route(logits, 8)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, 8)  # every token (the model dequantises one expert at a time)
    assert_close(out, ref, f"config5 T={T}")
    # the two-step path on the same inputs: routing on the device, then the block on its outputs
    r = ops.gpu_topk_route(DeviceBuffer.from_numpy(logits), 8)
    assert np.array_equal(r.expert_indices.numpy(), idx) and np.array_equal(r.expert_weights.numpy(), w)
    out2 = ops.moe_forward_grouped(gh, uh, dh, DeviceBuffer.from_numpy(x), r.expert_indices, r.expert_weights, 8).numpy()
    assert_close(out2, ref, f"config5 T={T} (two-step)")


@pytest.mark.parametrize("T", [5, 37, 128])
def test_config5_expert_stream_kernels_agree(hip, config5, T):
    """The streaming kernels of decode-sized batches on config 5, every token against the oracle: K split over the waves
    of a workgroup (1), a wave per weight tile over chunks of 8 rows (2) and of 16 rows (3: at T = 128 most experts have
    9 to 16 rows, a few more than 16), the hybrid (4), the gate / up projection in two launches with the experts split by
    their row count (5: up to 8 rows on kernel 1, more on kernel 3) and the library's choice among them (0).  The grouped
    GEMM is switched off."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    gate, up, down, gh, uh, dh = config5
    rng = np.random.default_rng(5100 + T)
    x = make_x(rng, T, 4096)
    logits = rng.standard_normal((T, 128)).astype(np.float32)
    idx, w, counts, _ = model.topk_route(logits, 8)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, 8)
    xd, ld = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits)
    idxd, wd = DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w)
    prev_rows, prev_kind = gh.set_expert_gemm_min_rows(0), gh.set_expert_stream_kernel(0)
    try:
        for kind in (0, 1, 2, 3, 4, 5):
            gh.set_expert_stream_kernel(kind)
            print(f"config5 stream kernel {kind} T={T} max rows per expert {int(counts.max())}", flush=True)
            assert_close(ops.moe_forward(gh, uh, dh, xd, ld, 8).numpy(), ref, f"config5 T={T} stream kernel {kind}")
            assert_close(ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, 8).numpy(), ref, f"config5 T={T} stream kernel {kind} (two-step)")
    finally:
        gh.set_expert_gemm_min_rows(prev_rows)
        gh.set_expert_stream_kernel(prev_kind)


@pytest.mark.parametrize("E,T,K,D,I,fused", [(4, 9, 2, 1024, 1536, False), (3, 20, 3, 512, 2560, True), (8, 3, 2, 2048, 512, True)])
def test_wave_per_tile_kernel_shapes(hip, E, T, K, D, I, fused):
    """The wave-per-tile kernel on other shapes: separate gate and up weights, tile counts that are no multiple of a
    workgroup's share (I = 2560: 160 tiles over 8-wave workgroups), one pass per tile (K = 512), experts with more than 8
    and more than 16 rows, ExpertGroup on the same kernels."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(E * 100 + T + D)

    def weight(n, k):
        return make_weight(rng, n, k, 4, 64, lead=(E,))

    if fused:
        gu = weight(2 * I, D)
        gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
        gh, uh = ops.QuantizedWeight.from_numpy(*gu, 64, 4), None
    else:
        gate, up = weight(I, D), weight(I, D)
        gh, uh = ops.QuantizedWeight.from_numpy(*gate, 64, 4), ops.QuantizedWeight.from_numpy(*up, 64, 4)
    down = weight(D, I)
    dh = ops.QuantizedWeight.from_numpy(*down, 64, 4)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] += 3.0  # expert 0 takes (nearly) every token
    idx, w, counts, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, K)
    xd, ld = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits)
    gh.set_expert_gemm_min_rows(0)
    for kind in (1, 2, 3, 4, 5):
        gh.set_expert_stream_kernel(kind)
        print(f"wave-per-tile shapes E={E} T={T} D={D} I={I} fused={fused} kind={kind} counts={counts.tolist()}", flush=True)
        assert_close(ops.moe_forward(gh, uh, dh, xd, ld, K).numpy(), ref, f"stream kernel {kind}")
        group = ops.ExpertGroup(gh, uh, dh)
        sizes = (11, 1, 8, 17)
        items = [(e % E, make_x(rng, m, D)) for e, m in zip((1, 0, 2, 1), sizes)]
        outs = group.grouped_forward([(e, DeviceBuffer.from_numpy(v)) for e, v in items])
        for (e, v), (_, yv) in zip(items, outs):
            ones = np.ones((len(v), 1))
            assert_close(yv, model.moe_forward(v, np.full((len(v), 1), e), ones, gate, up, down, 64, 1),
                         f"ExpertGroup stream kernel {kind} expert {e} rows {len(v)}")


@pytest.mark.parametrize("T,E,K,D,I,bias", [(1, 128, 8, 1024, 512, False), (4, 16, 8, 512, 1536, True), (3, 8, 5, 2048, 1024, False),
                                            (16, 64, 2, 512, 512, False), (17, 64, 2, 512, 512, True), (2, 4, 1, 512, 4096, False)])
def test_few_tokens_run_without_grouping(hip, T, E, K, D, I, bias):
    """`moe_forward` of a few tokens routes without grouping (every assignment a row of its own) and adds the weighted
    expert outputs inside the down projection.  Against the oracle and against the grouped kernels (stream kernel 1) on
    the same inputs: experts shared by several tokens, fewer picks than waves, an expert bias, more than 8 tokens.  The
    two sides sum in different orders and round the intermediate to f16 on their own: half the tolerance apart at most."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(T * 1000 + E + K)
    gu = make_weight(rng, 2 * I, D, 4, 64, lead=(E,))
    down = make_weight(rng, D, I, 4, 64, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, 64, 4), ops.QuantizedWeight.from_numpy(*down, 64, 4)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    eb = rng.standard_normal(E).astype(np.float32) if bias else None
    idx, w, _, _ = model.topk_route(logits, K, eb)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, K)
    xd, ld = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits)
    bd = DeviceBuffer.from_numpy(eb) if bias else None
    print(f"few tokens T={T} E={E} K={K} D={D} I={I} bias={bias}", flush=True)
    direct = ops.moe_forward(gh, None, dh, xd, ld, K, expert_bias=bd).numpy()
    assert_close(direct, ref, "moe_forward (default)")
    prev = gh.set_expert_stream_kernel(1)
    try:
        grouped = ops.moe_forward(gh, None, dh, xd, ld, K, expert_bias=bd).numpy()
    finally:
        gh.set_expert_stream_kernel(prev)
    assert_close(grouped, ref, "moe_forward (grouped kernels)")
    assert np.abs(direct.astype(np.float64) - grouped.astype(np.float64)).max() <= 0.5 * model.tolerance(ref)


@pytest.mark.parametrize("T", [300, 700])
def test_config5_moe_prefill_sizes(hip, config5, T):
    """Config 5 at prefill-sized batches (19 / 44 rows per expert on average: the grouped GEMM with 32- / 64-row tiles).
    The oracle checks every token, of the GEMM path and of the streaming GEMV path (threshold 0) on the same inputs,
    which shares no matrix kernel with the GEMM path."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    gate, up, down, gh, uh, dh = config5
    rng = np.random.default_rng(7000 + T)
    x = make_x(rng, T, 4096)
    logits = rng.standard_normal((T, 128)).astype(np.float32)
    idx, w, _, _ = model.topk_route(logits, 8)
    xd, idxd, wd = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w)
    print(f"config5 prefill T={T}", flush=True)
    out = ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, 8).numpy()
    prev = gh.set_expert_gemm_min_rows(0)
    try:
        out_stream = ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, 8).numpy()
    finally:
        gh.set_expert_gemm_min_rows(prev)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, 8)
    assert_close(out, ref, f"config5 T={T} (GEMM)")
    assert_close(out_stream, ref, f"config5 T={T} (streaming)")


@pytest.mark.parametrize("bits,E,T,D,I,fused", [(4, 4, 13, 512, 512, True), (4, 4, 13, 1024, 1536, False), (8, 8, 12, 512, 512, True),
                                                (8, 16, 9, 1024, 512, False), (8, 128, 64, 512, 1024, True)])
def test_moe_few_rows_per_expert_on_16_row_tiles(hip, bits, E, T, D, I, fused):
    """With the GEMM threshold lowered to 6 rows per expert on average (the default is 10; 8-bit experts: an eighth of
    it, at least 1), batches of up to 7 rows per expert run the grouped GEMM on 16-row tiles in four-wave workgroups - for
    4-bit weights the fused gate / up instantiation that no default setting reaches.  Against the oracle, with the
    streaming GEMV path beside it."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits * 7 + E + T + D)
    K = 2
    assert (6 if bits == 4 else 1) * E <= T * K <= 7 * E

    def weight(n, k):
        return make_weight(rng, n, k, bits, 64, lead=(E,))

    if fused:
        gu = weight(2 * I, D)
        gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
        gh, uh = ops.QuantizedWeight.from_numpy(*gu, 64, bits), None
    else:
        gate, up = weight(I, D), weight(I, D)
        gh, uh = ops.QuantizedWeight.from_numpy(*gate, 64, bits), ops.QuantizedWeight.from_numpy(*up, 64, bits)
    down = weight(D, I)
    dh = ops.QuantizedWeight.from_numpy(*down, 64, bits)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if E <= 16:
        logits[:, 1] += 2.0  # one expert with more than 16 rows: two tiles
    idx, w, counts, _ = model.topk_route(logits, K)
    ref = model.moe_forward(x, idx, w, gate, up, down, 64, K, bits=bits)
    xd, idxd, wd = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(idx), DeviceBuffer.from_numpy(w)
    print(f"16-row tiles bits={bits} E={E} T={T} D={D} I={I} fused={fused} counts={counts.tolist()}", flush=True)
    prev = gh.set_expert_gemm_min_rows(6)
    try:
        assert_close(ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, K).numpy(), ref, "moe_forward_grouped (16-row tiles)")
        assert_close(ops.moe_forward(gh, uh, dh, xd, DeviceBuffer.from_numpy(logits), K).numpy(), ref, "moe_forward (16-row tiles)")
        gh.set_expert_gemm_min_rows(0)
        assert_close(ops.moe_forward_grouped(gh, uh, dh, xd, idxd, wd, K).numpy(), ref, "moe_forward_grouped (streaming)")
    finally:
        gh.set_expert_gemm_min_rows(prev)
