"""The automatic kernel choice against every forced kernel family, by the clock.  Collected late on purpose: it is the one
GPU test here whose verdict depends on timings, so a noisy box cannot hide the parity tests behind it."""
import numpy as np
import pytest

from oracle import model
from tests.helpers import assert_close, make_weight, make_x

pytestmark = pytest.mark.gpu


LADDER_SHAPES = [(4096, 14336, 4, (3, 9, 16)), (2048, 16384, 4, (5, 16)), (4096, 8192, 4, (9, 16)), (12288, 4096, 4, (9, 24)),
                 (28672, 4096, 4, (8, 16, 100)), (12288, 4096, 8, (9, 16, 32)), (4096, 4096, 4, (128, 160, 256)),
                 (9216, 4096, 4, (64, 128)), (4096, 4096, 8, (128, 192)), (4096, 8192, 4, (128,)),
                 # short rows of tall matrices, K in whole blocks of 128, one or two rows over many weight rows
                 (9728, 896, 4, (1, 2, 24)), (16384, 1024, 4, (1, 2, 17, 32)), (4096, 11008, 4, (8, 64, 512)), (8192, 3072, 4, (2,)),
                 (13824, 1152, 4, (32, 512)), (65536, 1024, 4, (1,)), (8192, 512, 8, (2,))]


@pytest.mark.parametrize("n,k,bits,ms", LADDER_SHAPES)
def test_ladder_picks_within_15_percent_of_the_fastest_family(hip, n, k, bits, ms):
    """The automatic dispatch on shapes its crossovers were not tuned on: against every forced kernel family that takes the
    shape, the ladder's pick is within 15 % of the fastest (trains of launches between two events, weight sets cycled), and
    every family lands on the oracle (checked on the first 256 weight rows)."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(n + k + bits)
    base = make_weight(rng, n, k, bits, 64)
    n_sets = max(2, min(6, (400 << 20) // (n * k * bits // 8)))
    qws = [ops.QuantizedWeight.from_numpy(np.roll(base[0], i, 0), np.roll(base[1], i, 0), np.roll(base[2], i, 0), 64, bits)
           for i in range(n_sets)]
    stream, e0, e1 = rt.Stream(), rt.Event(), rt.Event()
    families = {"auto": rt.KERNEL_AUTO, "qmv": rt.KERNEL_QMV_ROWS, "single": rt.KERNEL_QMV, "qmm": rt.KERNEL_QMM, "k2": rt.KERNEL_QMM_K2,
                "lds": rt.KERNEL_QMM_LDS,
                "rw": rt.KERNEL_QMM_RW, "k2_tall": rt.KERNEL_QMM_K2_TALL, "k2_flat": rt.KERNEL_QMM_K2_FLAT, "k4": rt.KERNEL_QMM_K4}

    def train_us(xd, outs, kernel, count=300):
        e0.record(stream)
        ops.qmm_encode_many(qws, xd, outs, count, stream=stream, kernel=kernel)
        e1.record(stream)
        e1.sync()
        return e0.elapsed_ms(e1) / count * 1e3

    for m in ms:
        x = make_x(rng, m, k)
        xd = DeviceBuffer.from_numpy(x)
        outs = [DeviceBuffer((m, n), rt.F16) for _ in range(2)]
        ref = model.qmm(x.astype(np.float64), base[0][:256], base[1][:256], base[2][:256], 64, bits)
        times = {}
        print(f"ladder N={n} K={k} Q{bits} M={m}", flush=True)
        for name, kernel in families.items():
            try:
                ops.qmm_encode_many(qws[:1], xd, outs[:1], 1, stream=stream, kernel=kernel)
            except ops.KernelError:
                continue  # the family does not take this shape
            stream.sync()
            assert_close(outs[0].numpy()[:, :256], ref, f"N={n} K={k} Q{bits} M={m} family {name}")
            train_us(xd, outs, kernel, 100)  # clocks and caches as in the timed train
            times[name] = min(train_us(xd, outs, kernel) for _ in range(3))
        fastest = min((f for f in times if f != "auto"), key=times.get)
        if times["auto"] > 1.15 * times[fastest]:
            # (clock noise between two measurements taken seconds apart: time the two in turns before deciding)
            for _ in range(3):
                times["auto"] = min(times["auto"], train_us(xd, outs, families["auto"]))
                times[fastest] = min(times[fastest], train_us(xd, outs, families[fastest]))
        print("  " + " ".join(f"{f}={v:.1f}us" for f, v in times.items()), flush=True)
        assert times["auto"] <= 1.15 * times[fastest], (m, times)
