"""Stream capture through the C ABI (rmlx_hip_graph_begin / _end / _launch): a recorded train of launches replays to the
results of running the same calls eagerly, bit for bit, on every replay, with the program's own eager work and
synchronisations between the replays.  The `_into_cb` contract of the reference (encode into a caller's command buffer,
commit later: crates/rmlx-core/src/ops/quantized.rs:7797-7802) is what this stands for on a HIP stream."""

import numpy as np
import pytest

from oracle import model
from tests.helpers import assert_close, make_weight, make_x

pytestmark = pytest.mark.gpu


def _poison(buf):
    from rmlx_amd import runtime as rt
    rt.check(rt.lib().rmlx_hip_memcpy_h2d(buf.ptr, np.full(buf.shape, np.nan, np.float16).ctypes.data, buf.nbytes, None))


@pytest.mark.parametrize("m,n,k,bits", [(1, 512, 1024, 4), (4, 256, 512, 4), (2, 128, 512, 8), (40, 256, 1024, 4)])
def test_recorded_matmuls_replay_bit_for_bit(hip, m, n, k, bits):
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(m + n + k + bits)
    sets = [make_weight(rng, n, k, bits) for _ in range(3)]
    qws = [ops.QuantizedWeight.from_numpy(*w, 64, bits) for w in sets]
    x = make_x(rng, m, k)
    xd = DeviceBuffer.from_numpy(x)
    eager = [ops.affine_quantized_matmul_batched(xd, qw).numpy() for qw in qws]
    for w, e in zip(sets, eager):
        assert_close(e, model.qmm(x.astype(np.float64), *w, 64, bits), "eager")
    stream = rt.Stream()
    outs = [DeviceBuffer((m, n), rt.F16) for _ in qws]
    ops.qmm_encode_many(qws, xd, outs, len(qws), stream=stream)  # warm-up: attributes, scratch pool
    stream.sync()
    before = rt.scratch_allocations()
    with rt.Graph.record(stream) as g:
        ops.qmm_encode_many(qws, xd, outs, len(qws), stream=stream)
    assert rt.scratch_allocations() == before  # nothing was allocated while recording
    for replay in range(3):
        for o in outs:
            _poison(o)
        g.launch(stream)
        stream.sync()
        for o, e in zip(outs, eager):
            assert np.array_equal(o.numpy(), e), f"replay {replay}"
        # eager work of the program between replays
        assert np.array_equal(ops.affine_quantized_matmul_batched(xd, qws[0]).numpy(), eager[0])


@pytest.mark.parametrize("T", [1, 4, 16, 40])
def test_recorded_routed_block_replays_bit_for_bit(hip, T):
    """The entry point that allocates nothing, recorded: few tokens (routing without grouping, down projection with the
    combine), the fused routing + grouping launch, and the two-step path."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(500 + T)
    E, D, I, K = 16, 1024, 512, 4
    gu = make_weight(rng, 2 * I, D, 4, lead=(E,))
    down = make_weight(rng, D, I, 4, lead=(E,))
    gh, dh = ops.QuantizedWeight.from_numpy(*gu, 64, 4), ops.QuantizedWeight.from_numpy(*down, 64, 4)
    x = make_x(rng, T, D)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    xd, ld = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(logits)
    want = ops.moe_forward(gh, None, dh, xd, ld, K).numpy()
    stream = rt.Stream()
    out = DeviceBuffer((T, D), rt.F16)
    ops.moe_forward(gh, None, dh, xd, ld, K, out=out, noalloc=True, stream=stream)  # warm-up
    stream.sync()
    assert np.array_equal(out.numpy(), want)
    with rt.Graph.record(stream) as g:
        ops.moe_forward(gh, None, dh, xd, ld, K, out=out, noalloc=True, stream=stream)
    for replay in range(3):
        _poison(out)
        g.launch(stream)
        stream.sync()
        assert np.array_equal(out.numpy(), want), f"replay {replay}"
        assert np.array_equal(ops.moe_forward(gh, None, dh, xd, ld, K).numpy(), want)  # eager work between replays
