"""Several host threads drive the library at once, each on its own stream (the reference's registry is
shareable across threads, crates/rmlx-core/src/kernels/mod.rs:103-122; its array pool is per thread,
array.rs:33-47).  Every call that needs device scratch (f32 activations, the split-K GEMM, the MoE
block) draws it from the per-stream pool, so concurrent calls must never see each other's blocks:
each thread's results must equal, bit for bit, what the same calls return when run alone."""
import threading

import numpy as np
import pytest

from tests.helpers import make_weight, make_x

pytestmark = pytest.mark.gpu


def test_concurrent_streams_do_not_share_scratch(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer, Stream
    rng = np.random.default_rng(2024)
    n, k, E, I, T, top_k = 1024, 2048, 4, 512, 6, 2
    qw = ops.QuantizedWeight.from_numpy(*make_weight(rng, n, k, 4), 64, 4)
    q8 = ops.QuantizedWeight.from_numpy(*make_weight(rng, n, k, 8), 64, 8)
    gate = ops.QuantizedWeight.from_numpy(*make_weight(rng, I, k, 4, lead=(E,)), 64, 4)
    up = ops.QuantizedWeight.from_numpy(*make_weight(rng, I, k, 4, lead=(E,)), 64, 4)
    down = ops.QuantizedWeight.from_numpy(*make_weight(rng, k, I, 4, lead=(E,)), 64, 4)

    def make_job(seed):
        r = np.random.default_rng(seed)
        x32 = DeviceBuffer.from_numpy(r.standard_normal((3 + seed, k)).astype(np.float32))  # cast scratch
        x24 = DeviceBuffer.from_numpy(make_x(r, 24 + seed, k))                                # split-K partial sums
        x1 = DeviceBuffer.from_numpy(make_x(r, 1, k))
        xt = DeviceBuffer.from_numpy(make_x(r, T, k))
        logits = DeviceBuffer.from_numpy(r.standard_normal((T, E)).astype(np.float32))       # MoE intermediates

        def run(stream):
            outs = [ops.affine_quantized_matmul_batched(x32, qw, stream=stream),
                    ops.affine_quantized_matmul_batched(x24, qw, stream=stream),
                    ops.affine_quantized_matmul_batched(x24, q8, stream=stream),
                    ops.affine_quantized_matmul_batched(x1, qw, stream=stream),
                    ops.moe_forward(gate, up, down, xt, logits, top_k, stream=stream)]
            if stream is not None:
                stream.sync()
            return [o.numpy() for o in outs]
        return run

    jobs = [make_job(seed) for seed in range(4)]
    alone = [job(None) for job in jobs]
    failures = []

    def worker(i):
        try:
            stream = Stream()
            for rep in range(25):
                got = jobs[i](stream)
                for a, b in zip(got, alone[i]):
                    if not np.array_equal(a, b):
                        failures.append((i, rep))
                        return
        except Exception as e:  # noqa: BLE001 - reported below
            failures.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not failures, failures
