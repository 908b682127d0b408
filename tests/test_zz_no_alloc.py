"""The entry point that allocates nothing (rmlx_hip_moe_forward_noalloc) against rmlx_hip_moe_forward, through the
C ABI: same kernels over a static workspace instead of pooled scratch, so the outputs must be bit-identical.
Two calls in a row on the same workspace, the second with a smaller input, then the limits."""

import numpy as np
import pytest

from oracle import model
from tests.helpers import assert_close, make_weight, make_x

pytestmark = pytest.mark.gpu


def _experts(rng, E, D, I, bits=4):
    from rmlx_amd import ops
    gu = make_weight(rng, 2 * I, D, bits, lead=(E,))
    down = make_weight(rng, D, I, bits, lead=(E,))
    gate, up = tuple(a[:, :I] for a in gu), tuple(a[:, I:] for a in gu)
    return gate, up, down, ops.QuantizedWeight.from_numpy(*gu, 64, bits), ops.QuantizedWeight.from_numpy(*down, 64, bits)


def _both(gh, dh, x, logits, K, bias=None):
    """(pooled entry point, no-allocation entry point) on the same device inputs."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    xd, ld = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits)
    bd = DeviceBuffer.from_numpy(bias) if bias is not None else None
    want = ops.moe_forward(gh, None, dh, xd, ld, K, expert_bias=bd).numpy()
    out = DeviceBuffer.from_numpy(np.full((x.shape[0], x.shape[1]), np.nan, np.float16))  # must be overwritten
    got = ops.moe_forward(gh, None, dh, xd, ld, K, expert_bias=bd, out=out, noalloc=True).numpy()
    return want, got


def test_noalloc_matches_the_pooled_entry_point_on_two_calls_in_a_row(hip):
    rng = np.random.default_rng(77)
    E, D, I, K = 16, 1024, 512, 4
    gate, up, down, gh, dh = _experts(rng, E, D, I)
    # first call: 40 tokens (two-step routing, workgroup-wide grouping); second: 5 tokens (one fused launch) on the
    # workspace the first call left behind; third: enough rows per expert for the grouped GEMM
    for T in (40, 5, 48):
        x = make_x(rng, T, D)
        logits = rng.standard_normal((T, E)).astype(np.float32)
        print(f"noalloc T={T} E={E} D={D} I={I} K={K}", flush=True)
        want, got = _both(gh, dh, x, logits, K)
        assert np.array_equal(want.view(np.uint16), got.view(np.uint16)), f"T={T}"
        idx, w, _, _ = model.topk_route(logits, K)
        assert_close(got, model.moe_forward(x, idx, w, gate, up, down, 64, K), f"oracle T={T}")


def test_noalloc_with_the_gate_up_projection_in_two_launches(hip):
    """Between 6 rows per expert on average and the grouped GEMM's threshold, experts of config-5 size run the gate / up
    projection in two launches over two more chunk tables: those come from the workspace too.  Bit-identical to the pooled
    entry point, against the oracle on the first tokens, and again with a smaller batch behind it."""
    from rmlx_amd import ops
    rng = np.random.default_rng(81)
    E, D, I, K = 48, 4096, 1536, 8
    one = _experts(rng, 1, D, I)

    def tiled(a):  # (one random expert repeated: the routing still spreads the rows over all of them)
        return np.ascontiguousarray(np.broadcast_to(a, (E,) + a.shape[1:]))

    gate, up, down = (tuple(tiled(a) for a in t) for t in one[:3])
    gu = tuple(np.concatenate([g, u], axis=1) for g, u in zip(gate, up))
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, 64, 4), ops.QuantizedWeight.from_numpy(*down, 64, 4)
    for T in (40, 37):  # 6.7 and 6.2 rows per expert
        x = make_x(rng, T, D)
        logits = rng.standard_normal((T, E)).astype(np.float32)
        print(f"noalloc split gate / up T={T}", flush=True)
        want, got = _both(gh, dh, x, logits, K)
        assert np.array_equal(want.view(np.uint16), got.view(np.uint16)), f"T={T}"
        idx, w, _, _ = model.topk_route(logits, K)
        assert_close(got[:2], model.moe_forward(x[:2], idx[:2 * K], w[:2 * K], gate, up, down, 64, K), f"oracle T={T}")
        prev = gh.set_expert_stream_kernel(4)  # the same batch with one gate / up launch: both sides pass the oracle
        try:
            assert_close(_both(gh, dh, x, logits, K)[1][:2], model.moe_forward(x[:2], idx[:2 * K], w[:2 * K], gate, up, down, 64, K), "one launch")
        finally:
            gh.set_expert_stream_kernel(prev)


def test_noalloc_allocates_nothing(hip):
    """What the entry point is for: with the default stream's pool emptied first, a pooled call has to allocate and
    the call over the static workspace does not - for every dtype combination that carves casts from the workspace."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import F16, DeviceBuffer
    rng = np.random.default_rng(80)
    E, D, I, K = 16, 1024, 512, 4
    _, _, _, gh, dh = _experts(rng, E, D, I)
    cases = [(rng.standard_normal((40, D)).astype(np.float16), rng.standard_normal((40, E)).astype(np.float32), None),
             (rng.standard_normal((5, D)).astype(np.float32), rng.standard_normal((5, E)).astype(np.float16),
              rng.standard_normal(E).astype(np.float16)),
             (rng.standard_normal((48, D)).astype(np.float16), rng.standard_normal((48, E)).astype(np.float32), None)]
    bufs = [(DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(l), None if b is None else DeviceBuffer.from_numpy(b),
             DeviceBuffer((len(x), D), F16)) for x, l, b in cases]
    rt.check(rt.lib().rmlx_hip_trim_pool(None))
    before = rt.scratch_allocations()
    for xd, ld, bd, out in bufs:
        print(f"noalloc counter T={xd.shape[0]}", flush=True)
        ops.moe_forward(gh, None, dh, xd, ld, K, expert_bias=bd, out=out, noalloc=True)
    assert rt.scratch_allocations() == before
    ops.moe_forward(gh, None, dh, bufs[0][0], bufs[0][1], K)  # the pooled entry point on an empty pool
    assert rt.scratch_allocations() > before


def test_noalloc_casts_and_bias_come_from_the_workspace_too(hip):
    rng = np.random.default_rng(78)
    E, D, I, K = 8, 512, 512, 2
    gate, up, down, gh, dh = _experts(rng, E, D, I, bits=8)
    x = rng.standard_normal((9, D)).astype(np.float32)          # f32 activations: cast inside
    logits = rng.standard_normal((9, E)).astype(np.float16)     # f16 logits and bias: widened inside
    bias = rng.standard_normal(E).astype(np.float16)
    print("noalloc f32 x, f16 logits, f16 bias, 8-bit experts", flush=True)
    want, got = _both(gh, dh, x, logits, K, bias)
    assert np.array_equal(want.view(np.uint16), got.view(np.uint16))
    x2 = x[:3]
    want, got = _both(gh, dh, x2, logits[:3], K, bias)
    assert np.array_equal(want.view(np.uint16), got.view(np.uint16))


def test_noalloc_limits(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import F16, DeviceBuffer
    rng = np.random.default_rng(79)
    E, D, I, K = 8, 4096, 1536, 8
    _, _, _, gh, dh = _experts(rng, E, D, I)
    for T, ok in ((53, True), (54, False), (400, False)):
        xd = DeviceBuffer.from_numpy(make_x(rng, T, D))
        ld = DeviceBuffer.from_numpy(rng.standard_normal((T, E)).astype(np.float32))
        out = DeviceBuffer((T, D), F16)
        print(f"noalloc limit T={T}", flush=True)
        if ok:
            got = ops.moe_forward(gh, None, dh, xd, ld, K, out=out, noalloc=True).numpy()
            assert np.array_equal(got.view(np.uint16), ops.moe_forward(gh, None, dh, xd, ld, K).numpy().view(np.uint16))
        else:
            with pytest.raises(ops.KernelError, match="static workspace holds 8388608"):
                ops.moe_forward(gh, None, dh, xd, ld, K, out=out, noalloc=True)
    # expert formats with no grouped kernel run an expert per assignment on the single-row kernels, workspace included:
    # 4-bit at group size 32 below the grouped GEMM's dimensions, and 2-bit experts
    for bits, gs, d, i in ((4, 32, 64, 64), (2, 64, 128, 64)):
        gu = make_weight(rng, 2 * i, d, bits, gs, lead=(4,))
        dn = make_weight(rng, d, i, bits, gs, lead=(4,))
        gq, dq = ops.QuantizedWeight.from_numpy(*gu, gs, bits), ops.QuantizedWeight.from_numpy(*dn, gs, bits)
        xd = DeviceBuffer.from_numpy(make_x(rng, 3, d))
        ld = DeviceBuffer.from_numpy(rng.standard_normal((3, 4)).astype(np.float32))
        print(f"noalloc ungrouped-only experts bits={bits} gs={gs}", flush=True)
        got = ops.moe_forward(gq, None, dq, xd, ld, 2, out=DeviceBuffer((3, d), F16), noalloc=True).numpy()
        assert np.array_equal(got.view(np.uint16), ops.moe_forward(gq, None, dq, xd, ld, 2).numpy().view(np.uint16))
    # weights that only the portable kernels take (2-bit rows that are no whole 16-byte pieces)
    gu = make_weight(rng, 2 * 96, 96, 2, 32, lead=(4,))
    dn = make_weight(rng, 96, 96, 2, 32, lead=(4,))
    gp, dp = ops.QuantizedWeight.from_numpy(*gu, 32, 2), ops.QuantizedWeight.from_numpy(*dn, 32, 2)
    xd = DeviceBuffer.from_numpy(make_x(rng, 2, 96))
    ld = DeviceBuffer.from_numpy(rng.standard_normal((2, 4)).astype(np.float32))
    with pytest.raises(ops.KernelError, match="portable kernels"):
        ops.moe_forward(gp, None, dp, xd, ld, 2, out=DeviceBuffer((2, 96), F16), noalloc=True)
