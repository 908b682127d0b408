"""AWQ / GPTQ INT4 dequantisation (crates/rmlx-core/src/ops/quantized.rs:707-783, hosts :2269-2590).

The reference holds no test or vector for these two functions, so the oracle is pinned by what the
format fixes: hand-computed words, agreement of the two formats on one logical matrix packed both ways
(AWQ packs along the columns, GPTQ along the rows with the zero point stored minus one), the g_idx
special cases, and an element-at-a-time walk of the kernels' index arithmetic.  The GPU tests then
require bit-exact agreement with the oracle (one f32 subtraction of small integers, one f32 multiply).
"""
import numpy as np
import pytest

from oracle import model


def _logical(rng, k, n, gs):
    q = rng.integers(0, 16, size=(k, n)).astype(np.uint32)
    z = rng.integers(1, 16, size=(k // gs, n)).astype(np.uint32)  # GPTQ stores z - 1, which must stay >= 0
    s = rng.uniform(0.001, 0.05, size=(k // gs, n)).astype(np.float32)
    return q, z, s


def _pack_awq(q, z):
    return model.pack_u32(q, 4), model.pack_u32(z, 4)


def _pack_gptq(q, z):
    return np.ascontiguousarray(model.pack_u32(q.T, 4).T), model.pack_u32(z - 1, 4)


def test_awq_known_words():
    # nibble c of 0x76543210 is c; every zero nibble of 0x11111111 is 1
    out = model.awq_dequant(np.array([[0x76543210], [0xFEDCBA98]], np.uint32), np.array([[0x11111111]], np.uint32),
                            np.full((1, 8), 2.0, np.float32), 2)
    assert out.tolist() == [[-2, 0, 2, 4, 6, 8, 10, 12], [14, 16, 18, 20, 22, 24, 26, 28]]
    # second group uses its own zero word and scales
    out = model.awq_dequant(np.array([[0x00000005], [0x00000005]], np.uint32),
                            np.array([[0x00000001], [0x00000003]], np.uint32),
                            np.array([[1] * 8, [10] * 8], np.float32), 1)
    assert out[:, 0].tolist() == [4.0, 20.0] and out[0, 1] == 0.0


def test_gptq_known_words():
    # one packed row: nibble r of every word is r; zero word 0x76543210 -> stored zero c, effective c + 1
    qweight = np.full((1, 8), 0x76543210, np.uint32)
    out = model.gptq_dequant(qweight, np.array([[0x76543210]], np.uint32), np.ones((1, 8), np.float32), None, 8)
    want = np.arange(8)[:, None] - (np.arange(8)[None, :] + 1)
    assert np.array_equal(out, want.astype(np.float32))
    # the +1: stored zero 0 and q = 1 give exactly 0
    out = model.gptq_dequant(np.full((1, 8), 0x11111111, np.uint32), np.zeros((1, 1), np.uint32),
                             np.full((1, 8), 3.0, np.float32), None, 8)
    assert not out.any()


@pytest.mark.parametrize("k,n,gs", [(8, 8, 8), (32, 24, 8), (128, 64, 32), (64, 16, 64)])
def test_both_packings_of_one_matrix_agree_with_its_definition(k, n, gs):
    rng = np.random.default_rng(k + n + gs)
    q, z, s = _logical(rng, k, n, gs)
    g = np.arange(k) // gs
    want = s[g].astype(np.float64) * (q.astype(np.float64) - z[g].astype(np.float64))
    awq = model.awq_dequant(*_pack_awq(q, z), s, gs)
    gptq = model.gptq_dequant(*_pack_gptq(q, z), s, None, gs)
    assert np.array_equal(awq, gptq)
    assert np.array_equal(awq, want.astype(np.float32))  # exact: |q - z| <= 15 and one rounding


def test_gptq_g_idx():
    rng = np.random.default_rng(5)
    k, n, gs = 64, 16, 16
    q, z, s = _logical(rng, k, n, gs)
    qw, qz = _pack_gptq(q, z)
    ident = (np.arange(k) // gs).astype(np.int32)
    assert np.array_equal(model.gptq_dequant(qw, qz, s, ident, gs), model.gptq_dequant(qw, qz, s, None, gs))
    perm = rng.integers(0, k // gs, size=k).astype(np.int32)
    want = s[perm].astype(np.float64) * (q.astype(np.float64) - z[perm].astype(np.float64))
    assert np.array_equal(model.gptq_dequant(qw, qz, s, perm, 999), want.astype(np.float32))
    bad = perm.copy()
    bad[3], bad[40] = -1, k // gs
    out = model.gptq_dequant(qw, qz, s, bad, gs)
    assert not out[3].any() and not out[40].any()
    keep = np.ones(k, bool)
    keep[[3, 40]] = False
    assert np.array_equal(out[keep], want.astype(np.float32)[keep])


def test_element_walk_of_the_kernel_index_arithmetic():
    """One element at a time, with the index expressions of quantized.rs:717-732 and :766-782."""
    rng = np.random.default_rng(9)
    rows, cols, gs = 12, 16, 4
    qw = rng.integers(0, 2**32, size=(rows, cols // 8), dtype=np.uint64).astype(np.uint32)
    qz = rng.integers(0, 2**32, size=(rows // gs, cols // 8), dtype=np.uint64).astype(np.uint32)
    sc = rng.standard_normal((rows // gs, cols)).astype(np.float32)
    out = model.awq_dequant(qw, qz, sc, gs)
    flat_w, flat_z, flat_s = qw.reshape(-1), qz.reshape(-1), sc.reshape(-1)
    for row in range(rows):
        for col in range(cols):
            group, pack_idx, pack_off = row // gs, col // 8, col % 8
            nib = (int(flat_w[row * (cols // 8) + pack_idx]) >> (pack_off * 4)) & 0xF
            zero = (int(flat_z[group * (cols // 8) + pack_idx]) >> (pack_off * 4)) & 0xF
            assert out[row, col] == np.float32(flat_s[group * cols + col]) * np.float32(nib - zero)
    k, n, gs = 16, 8, 8
    qw = rng.integers(0, 2**32, size=(k // 8, n), dtype=np.uint64).astype(np.uint32)
    qz = rng.integers(0, 2**32, size=(k // gs, n // 8), dtype=np.uint64).astype(np.uint32)
    sc = rng.standard_normal((k // gs, n)).astype(np.float32)
    g_idx = rng.integers(0, k // gs, size=k).astype(np.int32)
    for gi in (None, g_idx):
        out = model.gptq_dequant(qw, qz, sc, gi, gs)
        flat_w, flat_z, flat_s = qw.reshape(-1), qz.reshape(-1), sc.reshape(-1)
        for row in range(k):
            for col in range(n):
                nib = (int(flat_w[(row // 8) * n + col]) >> ((row % 8) * 4)) & 0xF
                group = int(gi[row]) if gi is not None else row // gs
                zero = ((int(flat_z[group * (n // 8) + col // 8]) >> ((col % 8) * 4)) & 0xF) + 1
                assert out[row, col] == np.float32(flat_s[group * n + col]) * np.float32(nib - zero)


# ---- GPU ------------------------------------------------------------------------------------------


class _View:
    """A device buffer seen from `offset` bytes in (what an `Array` with a byte offset hands over)."""

    def __init__(self, buf, offset):
        self.ptr, self.nbytes, self._keep = buf.ptr + offset, buf.nbytes - offset, buf


def _dev(a):
    from rmlx_amd.runtime import DeviceBuffer
    a = np.ascontiguousarray(a)
    return DeviceBuffer.from_numpy(a.view(np.uint32) if a.dtype == np.int32 else a)


def _offset_dev(a, offset_bytes=4):
    """Upload `a` so that it starts `offset_bytes` into an allocation (not 16-byte aligned)."""
    a = np.ascontiguousarray(a)
    pad = np.zeros(offset_bytes // a.dtype.itemsize, a.dtype)
    return _View(_dev(np.concatenate([pad, a.reshape(-1)])), offset_bytes)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,gs", [(8, 8, 8), (6, 16, 2), (9, 24, 3), (128, 1032, 32), (4096, 4096, 128),
                                          (1001, 8200, 1001)])
def test_awq_dequant_is_bit_exact(hip, rows, cols, gs):
    from rmlx_amd import ops
    rng = np.random.default_rng(rows + cols)
    qw = rng.integers(0, 2**32, size=(rows, cols // 8), dtype=np.uint64).astype(np.uint32)
    qz = rng.integers(0, 2**32, size=(rows // gs, cols // 8), dtype=np.uint64).astype(np.uint32)
    sc = rng.standard_normal((rows // gs, cols)).astype(np.float32)
    print(f"awq rows={rows} cols={cols} gs={gs}", flush=True)
    want = model.awq_dequant(qw, qz, sc, gs)
    got = ops.awq_dequant(_dev(qw), _dev(qz), _dev(sc), rows, cols, gs).numpy()
    assert np.array_equal(got, want)
    if rows * cols <= 1 << 20:  # the any-alignment kernel
        got = ops.awq_dequant(_dev(qw), _dev(qz), _offset_dev(sc), rows, cols, gs).numpy()
        assert np.array_equal(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("k,n,gs,with_idx", [(8, 8, 8, False), (16, 8, 2, True), (24, 40, 3, False), (256, 1032, 64, True),
                                             (4096, 4096, 128, False), (4096, 4096, 128, True), (1000, 8200, 125, False)])
def test_gptq_dequant_is_bit_exact(hip, k, n, gs, with_idx):
    from rmlx_amd import ops
    rng = np.random.default_rng(k + n + int(with_idx))
    groups = k // gs
    qw = rng.integers(0, 2**32, size=(k // 8, n), dtype=np.uint64).astype(np.uint32)
    qz = rng.integers(0, 2**32, size=(groups, n // 8), dtype=np.uint64).astype(np.uint32)
    sc = rng.standard_normal((groups, n)).astype(np.float32)
    g_idx = rng.integers(0, groups, size=k).astype(np.int32) if with_idx else None
    print(f"gptq k={k} n={n} gs={gs} g_idx={with_idx}", flush=True)
    want = model.gptq_dequant(qw, qz, sc, g_idx, gs)
    gi = _dev(g_idx) if with_idx else None
    got = ops.gptq_dequant(_dev(qw), _dev(qz), _dev(sc), gi, k, n, gs).numpy()
    assert np.array_equal(got, want)
    if k * n <= 1 << 20:
        got = ops.gptq_dequant(_offset_dev(qw), _dev(qz), _dev(sc), gi, k, n, gs).numpy()
        assert np.array_equal(got, want)


@pytest.mark.gpu
def test_gptq_g_idx_out_of_range_rows_are_zero_and_identity_matches_none(hip):
    from rmlx_amd import ops
    rng = np.random.default_rng(77)
    k, n, gs = 64, 48, 16
    qw = rng.integers(0, 2**32, size=(k // 8, n), dtype=np.uint64).astype(np.uint32)
    qz = rng.integers(0, 2**32, size=(k // gs, n // 8), dtype=np.uint64).astype(np.uint32)
    sc = rng.standard_normal((k // gs, n)).astype(np.float32)
    base = ops.gptq_dequant(_dev(qw), _dev(qz), _dev(sc), None, k, n, gs).numpy()
    ident = (np.arange(k) // gs).astype(np.int32)
    assert np.array_equal(ops.gptq_dequant(_dev(qw), _dev(qz), _dev(sc), _dev(ident), k, n, gs).numpy(), base)
    bad = ident.copy()
    bad[[0, 9, 63]] = [-5, 4, 2**31 - 1]
    for q in (_dev(qw), _offset_dev(qw)):
        got = ops.gptq_dequant(q, _dev(qz), _dev(sc), _dev(bad), k, n, gs).numpy()
        assert np.array_equal(got, model.gptq_dequant(qw, qz, sc, bad, gs))
        assert not got[[0, 9, 63]].any()


@pytest.mark.gpu
def test_dequant_validation_and_stream(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import Stream
    w, z, s = _dev(np.zeros((16, 2), np.uint32)), _dev(np.zeros((2, 2), np.uint32)), _dev(np.ones((2, 16), np.float32))
    for args, msg in [((w, z, s, 16, 12, 8), r"awq_dequant: cols \(12\) must be a multiple of 8 \(pack factor\)"),
                      ((w, z, s, 16, 16, 0), "awq_dequant: group_size must be > 0"),
                      ((w, z, s, 16, 16, 5), r"awq_dequant: rows \(16\) must be a multiple of group_size \(5\)"),
                      ((w, z, s, 32, 16, 8), "awq_dequant: qweight buffer too small: 128 bytes < expected 256 bytes"),
                      ((w, z, s, 16, 16, 4), "awq_dequant: qzeros buffer too small"),
                      ((w, _dev(np.zeros((4, 2), np.uint32)), s, 16, 16, 4), "awq_dequant: scales buffer too small")]:
        with pytest.raises(ops.KernelError, match=msg) as e:
            ops.awq_dequant(*args)
        assert e.value.code == 1
    gw = _dev(np.zeros((2, 16), np.uint32))
    gi = _dev(np.zeros(16, np.int32))
    for args, msg in [((gw, z, s, None, 12, 16, 8), r"gptq_dequant: in_features \(12\) must be a multiple of 8"),
                      ((gw, z, s, None, 16, 12, 8), r"gptq_dequant: out_features \(12\) must be a multiple of 8 \(pack factor for qzeros\)"),
                      ((gw, z, s, None, 16, 16, 0), "gptq_dequant: group_size must be > 0"),
                      ((gw, z, s, None, 16, 16, 5), "must be a multiple of group_size \\(5\\) when g_idx is not provided"),
                      ((gw, z, s, None, 32, 16, 16), "gptq_dequant: qweight buffer too small"),
                      ((gw, z, s, None, 16, 16, 4), "gptq_dequant: qzeros buffer too small"),
                      ((gw, _dev(np.zeros((4, 2), np.uint32)), s, None, 16, 16, 4), "gptq_dequant: scales buffer too small"),
                      ((gw, z, s, _dev(np.zeros(8, np.int32)), 16, 16, 8), "gptq_dequant: g_idx buffer too small")]:
        with pytest.raises(ops.KernelError, match=msg) as e:
            ops.gptq_dequant(*args)
        assert e.value.code == 1
    # g_idx lifts the divisibility rule (quantized.rs:2434-2438) and the stream twin only enqueues
    stream = Stream()
    out = ops.gptq_dequant(gw, z, s, gi, 16, 16, 5, stream=stream)
    stream.sync()
    assert np.array_equal(out.numpy(), np.full((16, 16), -1.0, np.float32))
    assert ops.awq_dequant(w, z, s, 0, 16, 8).numpy().shape == (0, 16)
