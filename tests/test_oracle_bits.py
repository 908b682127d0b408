"""CPU pins of the oracle's 3- and 6-bit weights (and of the word layout at every bit width).

The reference takes such weights only in its portable kernel `affine_qmv`
(crates/rmlx-core/src/ops/quantized.rs:210-291) and holds no test or fixture with them, so the oracle is pinned
against a loop-for-loop restatement of that kernel on small shapes and against the closed forms its coverage
rule fixes (a group's values past its last whole word count for nothing)."""
import numpy as np
import pytest

from oracle import model


def _affine_qmv_loops(words, scales, biases, vec, group_size, bits):
    """quantized.rs:232-270 with Python loops: per row, per group, per word, per value."""
    n, k = words.shape[0], len(vec)
    elems_per_u32 = 32 // bits
    groups_per_row = k // group_size
    u32s_per_group = group_size // elems_per_u32
    u32s_per_row = groups_per_row * u32s_per_group
    mask = (1 << bits) - 1
    assert words.shape[1] == u32s_per_row
    out = np.zeros(n)
    for row in range(n):
        accum = 0.0
        for g in range(groups_per_row):
            group_dot = group_xsum = 0.0
            for w in range(u32s_per_group):
                word = int(words[row, g * u32s_per_group + w])
                for kk in range(elems_per_u32):
                    q = (word >> (kk * bits)) & mask
                    x = float(vec[g * group_size + w * elems_per_u32 + kk])
                    group_dot += q * x
                    group_xsum += x
            accum += float(scales[row, g]) * group_dot + float(biases[row, g]) * group_xsum
        out[row] = accum
    return out


@pytest.mark.parametrize("bits", [2, 3, 4, 6, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_qmm_follows_the_portable_kernel_loop_for_loop(bits, gs):
    rng = np.random.default_rng(bits * 10 + gs)
    n, k = 5, 2 * gs
    wpg = model.words_per_group(gs, bits)
    words = rng.integers(0, 2**32, size=(n, k // gs * wpg), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.01, 0.1, size=(n, k // gs)).astype(np.float16)
    biases = rng.uniform(-1, 1, size=(n, k // gs)).astype(np.float16)
    vec = rng.standard_normal(k).astype(np.float16)
    ref = _affine_qmv_loops(words, scales, biases, vec, gs, bits)
    got = model.qmm(vec[None, :].astype(np.float64), words, scales, biases, gs, bits)[0]
    np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-12)


def test_words_per_group_values():
    assert [model.words_per_group(g, 3) for g in (32, 64, 128)] == [3, 6, 12]
    assert [model.words_per_group(g, 6) for g in (32, 64, 128)] == [6, 12, 25]
    for bits in (2, 4, 8):
        for g in (32, 64, 128):
            assert model.words_per_group(g, bits) == g * bits // 32


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_grouped_layout_is_the_flat_layout_at_powers_of_two(bits):
    rng = np.random.default_rng(bits)
    q = rng.integers(0, 1 << bits, size=(3, 256)).astype(np.uint32)
    for gs in (32, 64, 128):
        assert np.array_equal(model.pack_grouped(q, gs, bits), model.pack_u32(q, bits))
        back, covered = model.unpack_grouped(model.pack_u32(q, bits), gs, bits)
        assert covered.all() and np.array_equal(back, q)


@pytest.mark.parametrize("bits,gs,covered_per_group", [(3, 32, 30), (3, 64, 60), (3, 128, 120), (6, 32, 30), (6, 64, 60),
                                                       (6, 128, 125)])
def test_three_and_six_bit_coverage_and_closed_forms(bits, gs, covered_per_group):
    rng = np.random.default_rng(bits + gs)
    n, groups = 4, 3
    k = groups * gs
    q = rng.integers(0, 1 << bits, size=(n, k)).astype(np.uint32)
    words = model.pack_grouped(q, gs, bits)
    assert words.shape == (n, groups * model.words_per_group(gs, bits))
    back, covered = model.unpack_grouped(words, gs, bits)
    assert covered.sum() == groups * covered_per_group
    assert np.array_equal(back[:, covered], q[:, covered]) and not back[:, ~covered].any()
    # bit positions: value j of a word sits at bit offset bits * j, the top 2 bits of a word stay clear
    per = 32 // bits
    assert int(words[0, 0]) == sum(int(q[0, j]) << (bits * j) for j in range(per))
    assert not (words >> np.uint32(per * bits)).any()
    # all values c, scale 1, bias 0, x = 1: c times the covered count; values 0, bias 1: the covered count
    ones = np.ones((1, k))
    c = (1 << bits) - 2
    wc = model.pack_grouped(np.full((n, k), c, np.uint32), gs, bits)
    s1, b0 = np.ones((n, groups), np.float16), np.zeros((n, groups), np.float16)
    assert np.array_equal(model.qmm(ones, wc, s1, b0, gs, bits), np.full((1, n), c * groups * covered_per_group, float))
    w0 = np.zeros_like(wc)
    assert np.array_equal(model.qmm(ones, w0, b0, s1, gs, bits), np.full((1, n), groups * covered_per_group, float))
    # a one-hot x at an element without a word gives 0, at a covered one the dequantised weight
    x = np.zeros((1, k))
    x[0, gs - 1] = 1.0  # last element of group 0: never covered at 3 / 6 bits
    s = rng.uniform(0.5, 1.5, size=(n, groups)).astype(np.float16)
    b = rng.uniform(-1, 1, size=(n, groups)).astype(np.float16)
    assert not model.qmm(x, words, s, b, gs, bits).any()
    x[:] = 0
    x[0, gs + 7] = 1.0
    want = s[:, 1].astype(np.float64) * q[:, gs + 7] + b[:, 1].astype(np.float64)
    np.testing.assert_allclose(model.qmm(x, words, s, b, gs, bits)[0], want, rtol=0, atol=0)
