"""Seeded synthetic inputs of the benchmark configurations and comparison helpers (tests only)."""
import numpy as np

from oracle import model


def make_weight(rng, n, k, bits=4, group_size=64, lead=()):
    """Uniform q, f16 scale ~ U[lo,hi], bias = -(2^(bits-1)) * scale (exact in f16)."""
    lo, hi = (0.005, 0.02) if bits <= 4 else (0.0005, 0.002)
    shape = tuple(lead) + (n, k // group_size * model.words_per_group(group_size, bits))  # k * bits / 32 at 2, 4, 8 bits
    words = rng.integers(0, 2**32, size=shape, dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(lo, hi, size=tuple(lead) + (n, k // group_size)).astype(np.float16)
    biases = (-(2.0 ** (bits - 1)) * scales.astype(np.float32)).astype(np.float16)
    return words, scales, biases


def make_x(rng, m, k, dtype="f16"):
    x = rng.standard_normal((m, k)).astype(np.float32)
    if dtype == "f16":
        return x.astype(np.float16)
    if dtype == "bf16":
        return model.f32_to_bf16_bits(x)  # uint16 bit patterns
    return x


def x_as_f64(x, dtype):
    if dtype == "bf16":
        return model.bf16_bits_to_f32(x).astype(np.float64)
    return x.astype(np.float64)


def assert_close(got_f16, ref_f64, what=""):
    """The acceptance bar: max|err| <= 1e-2 * RMS(reference output)."""
    got = np.asarray(got_f16, dtype=np.float64)
    tol = model.tolerance(ref_f64)
    err = float(np.max(np.abs(got - ref_f64))) if got.size else 0.0
    assert got.shape == ref_f64.shape, (got.shape, ref_f64.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    assert err <= tol, f"{what}: max|err| {err:.5f} > tol {tol:.5f} (1e-2 * RMS)"
    return err, tol
