"""Pins the CPU oracle against the reference's own known-answer tests and closed forms.

Each test names the reference test it re-runs (crates/rmlx-core/src/ops/quantized.rs unless
another file is given).  No GPU needed.
"""
import numpy as np
import pytest

from oracle import model, refpath


# ---- nibble / row dequant ------------------------------------------------------------

def test_dequant_q4_nibble_kats():
    # test_dequant_q4_nibble_{low,high,zero,max} (:10578-10599)
    assert refpath.dequant_q4_nibble(0xA7, 0) == 7
    assert refpath.dequant_q4_nibble(0xA7, 1) == 10
    assert refpath.dequant_q4_nibble(0x00, 0) == 0 and refpath.dequant_q4_nibble(0x00, 1) == 0
    assert refpath.dequant_q4_nibble(0xFF, 0) == 15 and refpath.dequant_q4_nibble(0xFF, 1) == 15


def test_dequantize_q4_row_manual():
    # test_dequantize_q4_row_manual (:10601-10624)
    out = refpath.dequantize_q4_row([0x53, 0x1A], [2.0], [0.5], 4, 4)
    assert np.array_equal(out, np.array([6.5, 10.5, 20.5, 2.5], np.float32))
    words = model.bytes_to_words(np.array([[0x53, 0x1A, 0, 0]], np.uint8))
    w = model.dequantize(words, [[2.0, 2.0]], [[0.5, 0.5]], 4, 4)
    assert np.array_equal(w[0, :4], [6.5, 10.5, 20.5, 2.5])


def test_extract_bits_matches_unpack():
    rng = np.random.default_rng(0)
    words = rng.integers(0, 2**32, size=64, dtype=np.uint64).astype(np.uint32)
    for bits in (4, 8):
        vals = model.unpack_u32(words[None, :], bits)[0]
        per = 32 // bits
        for w in range(8):
            for i in range(per):
                assert refpath.extract_bits(int(words[w]), i, bits) == vals[w * per + i]


# ---- packing -------------------------------------------------------------------------

def test_repack_kats():
    # test_repack_q4_simple / test_repack_q8_simple (crates/rmlx-nn/src/safetensors_loader.rs:838-866)
    assert list(refpath.repack_mlx_weight([0x76543210], 4)) == [0x10, 0x32, 0x54, 0x76]
    assert list(refpath.repack_mlx_weight([0x04030201], 8)) == [1, 2, 3, 4]
    assert list(model.words_to_bytes(np.array([[0x76543210]], np.uint32))[0]) == [0x10, 0x32, 0x54, 0x76]
    assert list(model.unpack_u32(np.array([[0x76543210]], np.uint32), 4)[0]) == list(range(8))
    assert list(model.unpack_u32(np.array([[0x04030201]], np.uint32), 8)[0]) == [1, 2, 3, 4]


@pytest.mark.parametrize("bits", [4, 8])
def test_pack_unpack_exhaustive_per_slot(bits):
    per, top = 32 // bits, 1 << bits
    for slot in range(per):
        for v in range(top):
            q = np.zeros(per, np.uint8)
            q[slot] = v
            w = model.pack_u32(q[None, :], bits)
            assert int(w[0, 0]) == v << (bits * slot)
            assert np.array_equal(model.unpack_u32(w, bits)[0], q)
            assert np.array_equal(refpath.pack_u32(q, bits), w[0])


@pytest.mark.parametrize("bits", [4, 8])
def test_pack_roundtrip_random_and_byte_view(bits):
    rng = np.random.default_rng(1)
    q = rng.integers(0, 1 << bits, size=(5, 256), dtype=np.uint8)
    w = model.pack_u32(q, bits)
    assert np.array_equal(model.unpack_u32(w, bits), q)
    assert np.array_equal(refpath.pack_u32(q.reshape(-1), bits), w.reshape(-1))
    by = model.words_to_bytes(w)
    assert np.array_equal(by.reshape(-1), refpath.repack_mlx_weight(w.reshape(-1), bits))
    if bits == 4:  # low nibble = even k
        assert np.array_equal(by & 0xF, q[:, 0::2]) and np.array_equal(by >> 4, q[:, 1::2])
    else:
        assert np.array_equal(by, q)
    assert np.array_equal(model.bytes_to_words(by), w)


# ---- f16 conversion ------------------------------------------------------------------

def test_f32_to_f16_bits_value_list():
    # test_f32_to_f16_bits_correctness (:10480-10513): the `half` crate is IEEE RNE = numpy.float16
    vals = np.array([0.0, 1.0, -1.0, 0.5, -0.5, 0.001, 0.02, -0.005, 65504.0, np.inf, -np.inf, 1e-8],
                    np.float32)
    assert np.array_equal(refpath.f32_to_f16_bits(vals), vals.astype(np.float16).view(np.uint16))
    nan = int(refpath.f32_to_f16_bits(np.array([np.nan], np.float32))[0])
    assert nan & 0x7C00 == 0x7C00 and nan & 0x03FF != 0


def test_f16_roundtrip_exhaustive():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = refpath.f16_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(f), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.array_equal(f[ok].view(np.uint32), ref[ok].view(np.uint32))
    back = refpath.f32_to_f16_bits(f[ok])
    assert np.array_equal(back, bits[ok])


def test_f32_to_f16_random_rne():
    rng = np.random.default_rng(2)
    u = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    f = u.view(np.float32)
    f = f[np.isfinite(f)]
    with np.errstate(over="ignore"):
        ref = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(refpath.f32_to_f16_bits(f), ref)


def test_bf16_helpers():
    x = np.array([1.0, -2.5, 3.140625, 1e-3, 1.00390625, 1.01171875], np.float32)
    b = model.f32_to_bf16_bits(x)
    back = model.bf16_bits_to_f32(b)
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0**-8)
    assert model.f32_to_bf16_bits(np.array([1.00390625], np.float32))[0] == 0x3F80  # tie -> even
    assert model.f32_to_bf16_bits(np.array([1.01171875], np.float32))[0] == 0x3F82  # tie -> even (up)


# ---- LCG -----------------------------------------------------------------------------

def test_lcg_first_values_closed_form():
    # :10743-10747 -- recompute with Python big ints
    s = 42
    exp = []
    for _ in range(5):
        s = (s * 6364136223846793005 + 1) % 2**64
        exp.append(np.float32(np.float32(s >> 33) / np.float32(2147483648.0)) - np.float32(1.0))
    got = refpath.Lcg(42).fill(5)
    assert np.array_equal(got, np.array(exp, np.float32))
    assert np.all(got >= -1.0) and np.all(got < 1.0)


# ---- affine_qmm vs naive (the reference's own assertions) ---------------------------------

def _lcg_case(m, n, k, gs, seed, bits):
    g = refpath.Lcg(seed)
    w = g.fill(n * k).reshape(n, k)   # weights first, then activations (:10750-10753)
    x = g.fill(m * k).reshape(m, k)
    packed, sc, bi = refpath.quantize_rows(w, gs, bits)
    return x, w, packed, sc, bi


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_affine_qmm_matches_naive(gs, bits):
    # test_affine_qmm_matches_naive_group{32,64,128} (:10721-10809), Q8 twin (:11671-11750)
    m, n, k = 8, 4, 128
    x, _, packed, sc, bi = _lcg_case(m, n, k, gs, 42, bits)
    out = refpath.affine_qmm(x, packed, sc, bi, m, n, k, gs, bits)
    naive = refpath.naive_matmul_with_dequant(x, packed, sc, bi, m, n, k, gs, bits)
    assert np.all(np.abs(out - naive) / np.maximum(np.abs(naive), 1.0) < 1e-4)
    words = model.bytes_to_words(packed)
    f64 = model.qmm(x, words, sc, bi, gs, bits)
    assert np.all(np.abs(out - f64) / np.maximum(np.abs(f64), 1.0) < 1e-4)
    assert np.all(np.abs(naive - f64) / np.maximum(np.abs(f64), 1.0) < 1e-4)


@pytest.mark.parametrize("bits", [4, 8])
def test_affine_qmm_large_batch(bits):
    # test_affine_qmm_large_batch (:10933-10998), Q8 twin (:11802-11866)
    m, n, k, gs = 32, 8, 64, 32
    x, _, packed, sc, bi = _lcg_case(m, n, k, gs, 7, bits)
    out = refpath.affine_qmm(x, packed, sc, bi, m, n, k, gs, bits)
    naive = refpath.naive_matmul_with_dequant(x, packed, sc, bi, m, n, k, gs, bits)
    assert np.all(np.abs(out - naive) / np.maximum(np.abs(naive), 1.0) < 1e-4)


@pytest.mark.parametrize("bits,tol", [(4, 0.50), (8, 0.10)])
def test_affine_qmm_vs_float_matmul_tolerance(bits, tol):
    # test_affine_qmm_vs_float_matmul_tolerance (:10815-10889), Q8 twin (:11868-11939)
    m, n, k, gs = 4, 2, 64, 32
    x, w, packed, sc, bi = _lcg_case(m, n, k, gs, 123, bits)
    exact = np.zeros((m, n), np.float32)
    for i in range(m):
        for j in range(n):
            d = np.float32(0)
            for kk in range(k):
                d = np.float32(d + x[i, kk] * w[j, kk])
            exact[i, j] = d
    out = refpath.affine_qmm(x, packed, sc, bi, m, n, k, gs, bits)
    assert np.all(np.abs(exact - out) / np.maximum(np.abs(exact), 0.01) < tol)


def test_closed_forms():
    # test_affine_qmm_m1_reduces_to_qmv (:10895-10931): all nibbles 7, x=1 -> 224
    out = refpath.affine_qmm(np.ones(32), np.full(2 * 16, 0x77, np.uint8), [1, 1], [0, 0], 1, 2, 32, 32)
    assert np.allclose(out, 224.0, atol=1e-4)
    # test_affine_qmm_identity_scale_zero_bias (:11541-11591): nibbles 3, x rows 1 and 2 -> 96 / 192
    x = np.concatenate([np.ones(32), 2 * np.ones(32)])
    out = refpath.affine_qmm(x, np.full(2 * 16, 0x33, np.uint8), [1, 1], [0, 0], 2, 2, 32, 32)
    assert np.allclose(out[0], 96.0, atol=1e-4) and np.allclose(out[1], 192.0, atol=1e-4)
    # test_affine_qmm_q8_identity_scale_zero_bias (:11752-11800): bytes 7 -> 224 / 448
    out = refpath.affine_qmm(x, np.full(2 * 32, 7, np.uint8), [1, 1], [0, 0], 2, 2, 32, 32, bits=8)
    assert np.allclose(out[0], 224.0, atol=1e-4) and np.allclose(out[1], 448.0, atol=1e-4)
    # test_qmv_f16_cpu_reference_consistency (:12069-12095): words 0x11111111, K=512 -> 512
    n, k, gs = 16, 512, 32
    words = np.full((n, k // 8), 0x11111111, np.uint32)
    out = refpath.cpu_qmv_q4_reference(words, np.ones((n, k // gs)), np.zeros((n, k // gs)), np.ones(k), n, k, gs)
    assert np.allclose(out, 512.0, atol=1e-3)
    assert np.allclose(model.qmm(np.ones((1, k)), words, np.ones((n, k // gs)), np.zeros((n, k // gs)), gs, 4), 512.0)


def test_threaded_baseline_is_bit_identical():
    m, n, k, gs = 5, 22, 128, 64
    x, _, packed, sc, bi = _lcg_case(m, n, k, gs, 9, 4)
    a = refpath.affine_qmm(x, packed, sc, bi, m, n, k, gs)
    b = refpath.affine_qmm_threads(x, packed, sc, bi, m, n, k, gs, threads=3)
    assert np.array_equal(a, b)


def test_model_linearity_and_row_independence():
    rng = np.random.default_rng(3)
    n, k, gs = 8, 128, 64
    words = rng.integers(0, 2**32, size=(n, k // 8), dtype=np.uint64).astype(np.uint32)
    s = rng.uniform(0.005, 0.02, (n, k // gs)).astype(np.float16)
    b = (-8 * s.astype(np.float32)).astype(np.float16)
    x1, x2 = rng.standard_normal((2, 3, k))
    f = lambda x: model.qmm(x, words, s, b, gs, 4)
    assert np.allclose(f(x1 + 2 * x2), f(x1) + 2 * f(x2), atol=1e-9)
    assert np.allclose(f(x1)[:, 2:5], model.qmm(x1, words[2:5], s[2:5], b[2:5], gs, 4), atol=1e-12)
    # s*dot + b*xsum identity (:2732)
    q = model.unpack_u32(words, 4).astype(np.float64)
    alt = np.zeros((3, n))
    for g in range(k // gs):
        sl = slice(g * gs, (g + 1) * gs)
        alt += s[:, g].astype(np.float64) * (x1[:, sl] @ q[:, sl].T) + b[:, g].astype(np.float64) * x1[:, sl].sum(1, keepdims=True)
    assert np.allclose(alt, f(x1), atol=1e-9)
