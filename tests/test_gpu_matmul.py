"""GPU parity of qmv / qmm against the float64 dequantize-then-matmul oracle, through the C ABI.

Tolerance everywhere: max|err| <= 1e-2 * RMS(oracle output) on f16 outputs (stated in
helpers.assert_close).  Shapes follow the benchmark configurations plus ragged / edge cases.
"""
import numpy as np
import pytest

from oracle import model, refpath
from tests.helpers import assert_close, make_weight, make_x, x_as_f64

pytestmark = pytest.mark.gpu


def _dev(hip, x, dtype):
    from rmlx_amd.runtime import BF16, DeviceBuffer
    return DeviceBuffer.from_numpy(x, BF16) if dtype == "bf16" else DeviceBuffer.from_numpy(x)


def _run(hip, words, scales, biases, x, bits, gs=64, dtype="f16", kernel=0, qmv_entry=False):
    from rmlx_amd import ops
    qw = ops.QuantizedWeight.from_numpy(words, scales, biases, gs, bits)
    xd = _dev(hip, x, dtype)
    if qmv_entry:
        return ops.affine_quantized_matmul(qw, xd).numpy()[None, :]
    return ops.affine_quantized_matmul_batched(xd, qw, kernel=kernel).numpy()


# ---- closed forms from the reference's tests, on the GPU ------------------------------------------

def test_equal_nibble_closed_forms(hip):
    from rmlx_amd import runtime as rt
    # all nibbles c, scale 1, bias 0, x = 1 (row 0) / 2 (row 1): out = c*K, 2*c*K
    # (quantized.rs:10895-10931, 11541-11591, 12069-12095 scaled to kernel-sized K)
    for kernel, n, k in [(rt.KERNEL_GENERIC, 8, 64), (rt.KERNEL_QMV, 16, 512), (rt.KERNEL_QMM, 64, 512),
                         (rt.KERNEL_QMM_LDS, 64, 512), (rt.KERNEL_QMM, 64, 256)]:
        for c in (1, 3, 7):
            words = np.full((n, k // 8), c * 0x11111111, np.uint32)
            s = np.ones((n, k // 64), np.float16)
            b = np.zeros((n, k // 64), np.float16)
            x = np.concatenate([np.ones((1, k)), 2 * np.ones((1, k))]).astype(np.float16)
            out = _run(hip, words, s, b, x, 4, kernel=kernel)
            assert np.array_equal(out[0], np.full(n, c * k, np.float16)), (kernel, c, out[0][:4])
            assert np.array_equal(out[1], np.full(n, 2 * c * k, np.float16))
    # Q8: all bytes 7 -> 7*K (quantized.rs:11752-11800)
    for n, k, kernels in [(64, 256, (rt.KERNEL_GENERIC, rt.KERNEL_QMM, rt.KERNEL_QMM_LDS)),
                          (64, 512, (rt.KERNEL_QMM, rt.KERNEL_QMM_LDS))]:
        words = np.full((n, k // 4), 0x07070707, np.uint32)
        x = np.ones((2, k), np.float16)
        for kernel in kernels:
            out = _run(hip, words, np.ones((n, k // 64), np.float16), np.zeros((n, k // 64), np.float16), x, 8, kernel=kernel)
            assert np.array_equal(out, np.full((2, n), 7 * k, np.float16)), (kernel, k)


def test_distinct_positions_are_not_mixed_up(hip):
    """One-hot activations pick out single weights: catches any k / row permutation mistake."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(5)
    n, k = 64, 1024
    words, s, b = make_weight(rng, n, k, 4)
    s[:] = 1.0
    b[:] = 0.0
    q = model.unpack_u32(words, 4).astype(np.float64)
    ks = np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 31, 32, 63, 64, 65, 127, 128, 511, 512, 1000, 1023])
    for m0 in range(0, len(ks), 8):
        sel = ks[m0:m0 + 8]
        x = np.zeros((len(sel), k), np.float16)
        x[np.arange(len(sel)), sel] = 1.0
        for kernel in (rt.KERNEL_QMV, rt.KERNEL_QMM, rt.KERNEL_QMM_LDS, rt.KERNEL_GENERIC):
            out = _run(hip, words, s, b, x, 4, kernel=kernel)
            assert np.array_equal(out.astype(np.float64), q[:, sel].T), (kernel, sel)


# ---- configuration shapes ----------------------------------------------------------------------

def test_config1_q4_qmv_4096(hip):
    rng = np.random.default_rng(1001)
    n = k = 4096
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, 1, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    out = _run(hip, words, s, b, x[0], 4, qmv_entry=True)
    assert_close(out, ref, "config1 qmv")
    # the CPU reference path (plumbing): C restatement of affine_qmm on the same inputs
    cpu = refpath.affine_qmm(x.astype(np.float32), model.words_to_bytes(words), s.astype(np.float32),
                             b.astype(np.float32), 1, n, k, 64)
    assert_close(cpu, ref, "config1 cpu reference path")


@pytest.mark.parametrize("m", [1, 4, 8])
def test_config2_q4_qmv_qkv(hip, m):
    rng = np.random.default_rng(1002)
    n, k = 9216, 4096
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    assert_close(_run(hip, words, s, b, x, 4), ref, f"config2 M={m}")


@pytest.mark.parametrize("m", [128, 512])
def test_config3_q4_qmm(hip, m):
    rng = np.random.default_rng(1003)
    n = k = 4096
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    assert_close(_run(hip, words, s, b, x, 4), ref, f"config3 M={m}")
    assert_close(_run(hip, words, s, b, x, 4, kernel=5), ref, f"config3 M={m} (LDS-staged kernel)")


def test_config4_q8_qmm_bf16(hip):
    rng = np.random.default_rng(1004)
    m, n, k = 128, 12288, 4096
    words, s, b = make_weight(rng, n, k, 8)
    x = make_x(rng, m, k, "bf16")
    ref = model.qmm(x_as_f64(x, "bf16"), words, s, b, 64, 8)
    err_auto, tol = assert_close(_run(hip, words, s, b, x, 8, dtype="bf16"), ref, "config4 (f16 MFMA, default)")
    # the bf16 matrix-instruction variant: weights rounded to 8 significant bits, still inside the bar
    err_bf16, _ = assert_close(_run(hip, words, s, b, x, 8, dtype="bf16", kernel=4), ref, "config4 (bf16 MFMA)")
    assert err_auto < err_bf16
    assert_close(_run(hip, words, s, b, x, 8, dtype="bf16", kernel=5), ref, "config4 (LDS-staged kernel)")


@pytest.mark.parametrize("m,n,k,bits", [(33, 64, 512, 4), (100, 128, 1024, 8), (200, 256, 512, 4), (513, 4096, 512, 4),
                                        (64, 2048, 1536, 4), (17, 192, 512, 8), (300, 1024, 2048, 8), (1100, 512, 512, 4)])
def test_qmm_tile_shapes(hip, m, n, k, bits):
    """Shapes that walk through the tile variants of the register-weights GEMM (ragged M, every N step)."""
    rng = np.random.default_rng(m + n + k + bits)
    words, s, b = make_weight(rng, n, k, bits)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, bits)
    assert_close(_run(hip, words, s, b, x, bits, kernel=2), ref, f"qmm M={m} N={n} K={k} bits={bits}")


def test_bf16_mfma_variant_is_only_for_q8_bf16(hip):
    from rmlx_amd import ops
    rng = np.random.default_rng(16)
    words, s, b = make_weight(rng, 64, 256, 8)
    with pytest.raises(ops.KernelError, match="bf16 MFMA GEMM takes Bfloat16"):
        _run(hip, words, s, b, make_x(rng, 32, 256), 8, kernel=4)
    words, s, b = make_weight(rng, 64, 256, 4)
    with pytest.raises(ops.KernelError, match="bf16 MFMA GEMM takes Bfloat16"):
        _run(hip, words, s, b, make_x(rng, 32, 256, "bf16"), 4, dtype="bf16", kernel=4)


# ---- kernel families agree, ragged M, dtypes, other group sizes --------------------------------------

@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 9, 16, 17, 31, 64, 65, 130])
def test_ragged_m_all_kernels(hip, m):
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(100 + m)
    n, k = 128, 1024
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    for kernel in (rt.KERNEL_AUTO, rt.KERNEL_QMV, rt.KERNEL_QMM, rt.KERNEL_QMM_LDS, rt.KERNEL_GENERIC):
        assert_close(_run(hip, words, s, b, x, 4, kernel=kernel), ref, f"M={m} kernel={kernel}")


@pytest.mark.parametrize("k", [512, 1536, 2048, 4608, 8192, 14336])
def test_qmv_k_sweep(hip, k):
    rng = np.random.default_rng(k)
    n, m = 48, 3
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    assert_close(_run(hip, words, s, b, x, 4, kernel=1), ref, f"qmv K={k}")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", ["f16", "f32", "bf16"])
def test_input_dtypes(hip, bits, dtype):
    rng = np.random.default_rng(7)
    n, k = 128, 512
    words, s, b = make_weight(rng, n, k, bits)
    for m in (1, 40):
        x = make_x(rng, m, k, dtype)
        ref = model.qmm(x_as_f64(x, dtype), words, s, b, 64, bits)
        assert_close(_run(hip, words, s, b, x, bits, dtype=dtype), ref, f"bits={bits} {dtype} M={m}")


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_group_sizes_and_odd_shapes_portable_kernel(hip, bits, gs):
    rng = np.random.default_rng(gs + bits)
    n, k, m = 24, 384, 5  # N not a multiple of 16, K not a multiple of 512: no matrix-unit kernel takes it
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, gs, bits)
    # the batched entry point only admits 4 and 8 bits (quantized.rs:7175); 2-bit goes to the portable kernel
    kernel = 3 if bits == 2 else 0
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, kernel=kernel), ref, f"bits={bits} gs={gs}")
    if bits == 2:
        from rmlx_amd import ops
        with pytest.raises(ops.KernelError, match="requires bits==4 or bits==8, got 2"):
            _run(hip, words, s, b, x, bits, gs=gs)


def test_qmv_entry_equals_batched_m1(hip):
    """M=1 qmm == qmv (quantized.rs:10895-10931), bit for bit on the same kernel."""
    rng = np.random.default_rng(11)
    n, k = 256, 2048
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, 1, k)
    a = _run(hip, words, s, b, x[0], 4, qmv_entry=True)
    bb = _run(hip, words, s, b, x, 4)
    assert np.array_equal(a, bb)


def test_linearity_and_row_independence_full_size(hip):
    """Size-independent properties at the full 4096^2 shape."""
    rng = np.random.default_rng(12)
    n = k = 4096
    words, s, b = make_weight(rng, n, k, 4)
    x1 = make_x(rng, 1, k).astype(np.float32)
    x2 = make_x(rng, 1, k).astype(np.float32)
    xs = np.concatenate([x1, x2, (x1 + x2)]).astype(np.float16)
    out = _run(hip, words, s, b, xs, 4).astype(np.float64)
    exact_sum = xs[2].astype(np.float64) - (xs[0].astype(np.float64) + xs[1].astype(np.float64))
    assert np.max(np.abs(exact_sum)) < 0.01  # f16 rounding of the sum only
    tol = 1e-2 * np.sqrt(np.mean(out[2] ** 2))
    assert np.max(np.abs(out[2] - out[0] - out[1])) < 2 * tol
    # rows of W are independent: a sub-block of rows gives the same values
    sub = _run(hip, words[1024:1280], s[1024:1280], b[1024:1280], xs, 4)
    assert np.array_equal(sub, _run(hip, words, s, b, xs, 4)[:, 1024:1280])


def test_quantized_linear_forward(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(13)
    n, k = 256, 1024
    for bits in (4, 8):
        words, s, b = make_weight(rng, n, k, bits)
        layer = ops.QuantizedLinear(model.words_to_bytes(words), s.astype(np.float32), b.astype(np.float32), k, n, 64, bits)
        x = make_x(rng, 6, k)
        ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, bits)
        assert_close(layer.forward(DeviceBuffer.from_numpy(x)).numpy(), ref, "2D")
        out1 = layer.forward(DeviceBuffer.from_numpy(x[0])).numpy()  # 1-D -> [1, out]
        assert out1.shape == (1, n)
        assert_close(out1, ref[:1], "1D")
        bias = rng.standard_normal(n).astype(np.float16)
        outb = layer.forward(DeviceBuffer.from_numpy(x), bias=DeviceBuffer.from_numpy(bias)).numpy()
        assert_close(outb, ref + bias.astype(np.float64)[None, :], "bias")
        with pytest.raises(ops.KernelError, match="1D or 2D"):
            layer.forward(DeviceBuffer.from_numpy(np.zeros((2, 3, k), np.float16)))
        with pytest.raises(ops.KernelError, match="features mismatch"):
            layer.forward(DeviceBuffer.from_numpy(np.zeros((2, k + 64), np.float16)))


def test_async_stream_matches_sync(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer, Stream
    rng = np.random.default_rng(14)
    n, k = 512, 1024
    words, s, b = make_weight(rng, n, k, 4)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    st = Stream()
    for m in (1, 7, 96):
        x = DeviceBuffer.from_numpy(make_x(rng, m, k))
        sync = ops.affine_quantized_matmul_batched(x, qw).numpy()
        out = ops.affine_quantized_matmul_batched(x, qw, stream=st)
        st.sync()
        assert np.array_equal(out.numpy(), sync)


# ---- validation (reference error sites) -------------------------------------------------------------

def test_validation_errors(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer, U32
    rng = np.random.default_rng(15)
    n, k = 64, 512
    words, s, b = make_weight(rng, n, k, 4)
    wb, sb, bb = DeviceBuffer.from_numpy(words), DeviceBuffer.from_numpy(s), DeviceBuffer.from_numpy(b)
    with pytest.raises(ops.KernelError, match="unsupported bit width 5"):
        ops.QuantizedWeight(wb, sb, bb, 64, 5, n, k)
    with pytest.raises(ops.KernelError, match="unsupported group_size 48"):
        ops.QuantizedWeight(wb, sb, bb, 48, 4, n, k)
    with pytest.raises(ops.KernelError, match="multiple of group_size"):
        ops.QuantizedWeight(wb, sb, bb, 128, 4, n, k + 64)
    with pytest.raises(ops.KernelError, match="weights_buf too small"):
        ops.QuantizedWeight(wb, sb, bb, 64, 4, n * 2, k)
    with pytest.raises(ops.KernelError, match="scales_buf too small"):
        ops.QuantizedWeight(wb, DeviceBuffer.from_numpy(s[:10]), bb, 64, 4, n, k)
    with pytest.raises(ops.KernelError, match="biases_buf too small"):
        ops.QuantizedWeight(wb, sb, DeviceBuffer.from_numpy(b[:10]), 64, 4, n, k)
    qw = ops.QuantizedWeight(wb, sb, bb, 64, 4, n, k)
    with pytest.raises(ops.KernelError, match="requires 2D input"):
        ops.affine_quantized_matmul_batched(DeviceBuffer.from_numpy(np.zeros(k, np.float16)), qw)
    with pytest.raises(ops.KernelError, match=r"x.shape\[1\]"):
        ops.affine_quantized_matmul_batched(DeviceBuffer.from_numpy(np.zeros((2, k * 2), np.float16)), qw)
    with pytest.raises(ops.KernelError, match="Float16 or Float32"):
        ops.affine_quantized_matmul_batched(DeviceBuffer((2, k), U32), qw)
    with pytest.raises(ops.KernelError, match=r"vec.numel\(\)"):
        ops.affine_quantized_matmul(qw, DeviceBuffer.from_numpy(np.zeros(k + 1, np.float16)))
    e = None
    try:
        ops.affine_quantized_matmul_batched(DeviceBuffer.from_numpy(np.zeros((2, 3), np.float16)), qw)
    except ops.KernelError as err:
        e = err
    assert e is not None and e.kind == "InvalidShape"
    # M = 0 is legal and returns an empty result
    out = ops.affine_quantized_matmul_batched(DeviceBuffer((0, k), 1), qw)
    assert out.shape == (0, n)


# ---- 8-bit streaming GEMV (affine_qmv_fast_q8, quantized.rs:620-695) -----------------------------------

@pytest.mark.parametrize("m", [1, 2, 7, 16, 17, 40])
@pytest.mark.parametrize("n,k", [(64, 2048), (48, 4096)])
def test_q8_qmv_matches_oracle(hip, m, n, k):
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(m * 7 + n + k)
    words, s, b = make_weight(rng, n, k, 8)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 8)
    assert_close(_run(hip, words, s, b, x, 8, kernel=rt.KERNEL_QMV), ref, f"q8 qmv M={m} N={n} K={k}")
    if m <= 16:  # the ladder sends small M there by itself
        assert_close(_run(hip, words, s, b, x, 8), ref, f"q8 auto M={m}")


def test_q8_qmv_closed_form_and_positions(hip):
    from rmlx_amd import runtime as rt
    n, k = 32, 2048
    words = np.full((n, k // 4), 0x07070707, np.uint32)  # all bytes 7, scale 1, bias 0, x = 1 -> 7*K (quantized.rs:11752-11800)
    out = _run(hip, words, np.ones((n, k // 64), np.float16), np.zeros((n, k // 64), np.float16),
               np.ones((3, k), np.float16), 8, kernel=rt.KERNEL_QMV)
    assert np.array_equal(out, np.full((3, n), 7 * k, np.float16))
    # one-hot activations pick out single weights
    rng = np.random.default_rng(8)
    words, s, b = make_weight(rng, n, k, 8)
    s[:] = 1.0
    b[:] = 0.0
    q = model.unpack_u32(words, 8).astype(np.float64)
    ks = np.array([0, 1, 3, 4, 7, 8, 15, 16, 63, 64, 65, 511, 512, 1023, 2047])
    x = np.zeros((len(ks), k), np.float16)
    x[np.arange(len(ks)), ks] = 1.0
    out = _run(hip, words, s, b, x, 8, kernel=rt.KERNEL_QMV)
    assert np.array_equal(out.astype(np.float64), q[:, ks].T)


# ---- fused store epilogues (qmm_add_residual_into_cb / qmm_swiglu_into_cb, quantized.rs:8227-8452) -------

@pytest.mark.parametrize("m,n,k,bits", [(64, 256, 512, 4), (130, 128, 1024, 4), (40, 128, 512, 8), (4, 64, 512, 4), (9, 24, 128, 4),
                                      (1, 64, 2048, 4), (2, 72, 4096, 4), (1, 32, 1024, 8), (2, 16, 2048, 8),
                                      (64, 256, 640, 4), (130, 128, 1408, 8), (6, 64, 1152, 4), (300, 64, 320, 4), (2, 4104, 512, 4)])
@pytest.mark.parametrize("edtype", ["f16", "f32"])
def test_fused_epilogues(hip, m, n, k, bits, edtype):
    """GEMM and single-row GEMV (fused), multi-row GEMV and portable (separate pass) kernels against the f64
    composition."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(m + n + k + bits)
    words, s, b = make_weight(rng, n, k, bits)
    x = make_x(rng, m, k)
    e = rng.standard_normal((m, n)).astype(np.float16 if edtype == "f16" else np.float32)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, bits)
    base = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, bits)
    e64 = e.astype(np.float64)
    xd, ed = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(e)
    assert_close(ops.qmm_add_residual(xd, qw, ed).numpy(), base + e64, "qmm_add_residual")
    assert_close(ops.qmm_swiglu(xd, qw, ed).numpy(), model.silu(e64) * base, "qmm_swiglu")


def test_fused_epilogue_validation(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(3)
    words, s, b = make_weight(rng, 64, 512, 4)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    xd = DeviceBuffer.from_numpy(make_x(rng, 8, 512))
    with pytest.raises(ops.KernelError, match=r"qmm_add_residual_into_cb: residual shape must be \[8, 64\]"):
        ops.qmm_add_residual(xd, qw, DeviceBuffer.from_numpy(np.zeros((8, 32), np.float16)))
    with pytest.raises(ops.KernelError, match=r"qmm_swiglu_into_cb: gate_result shape must be \[8, 64\]"):
        ops.qmm_swiglu(xd, qw, DeviceBuffer.from_numpy(np.zeros((4, 64), np.float32)))
    with pytest.raises(ops.KernelError, match="gate_result must be Float16 or Float32"):
        ops.qmm_swiglu(xd, qw, DeviceBuffer.from_numpy(np.zeros((8, 64), np.uint32)))


@pytest.mark.parametrize("m,n,k,bits,gs,dtype", [(17, 4096, 4096, 4, 64, "f16"), (33, 1024, 4096, 4, 64, "bf16"),
                                                 (64, 4096, 14336, 4, 64, "f16"), (5, 256, 8192, 8, 64, "f16"),
                                                 (40, 512, 2048, 8, 128, "f16"), (24, 1536, 1024, 4, 32, "f16"),
                                                 (100, 192, 1024, 4, 64, "f32"), (16, 64, 512, 4, 64, "f16")])
def test_qmm_split_k(hip, m, n, k, bits, gs, dtype):
    """Small grids of the register-weights GEMM split K over 2 or 4 workgroups per tile and add the f32
    partial sums in a second kernel (the counterpart of the reference's split-K kernel for 32 <= M < 128,
    quantized.rs:4572-4786, 6927-7103): the split must land on the oracle like the single pass, also
    with the store epilogues, which then run in the reduction kernel."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(m + n + k + bits + gs)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
    print(f"split-k M={m} N={n} K={k} bits={bits} gs={gs} {dtype}", flush=True)
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype, kernel=2), ref, "qmm")
    if m > 16:  # the automatic ladder takes the GEMM here, so the epilogue entry points reach the reduction kernel
        qw = ops.QuantizedWeight.from_numpy(words, s, b, gs, bits)
        xd = _dev(hip, x, dtype)
        for edt in (np.float16, np.float32):
            e = rng.standard_normal((m, n)).astype(edt)
            ed = DeviceBuffer.from_numpy(e)
            assert_close(ops.qmm_add_residual(xd, qw, ed).numpy(), ref + e.astype(np.float64), "qmm_add_residual")
            assert_close(ops.qmm_swiglu(xd, qw, ed).numpy(), model.silu(e.astype(np.float64)) * ref, "qmm_swiglu")


@pytest.mark.parametrize("m,n,k,bits,gs,dtype", [(1, 4096, 4096, 4, 64, "f16"), (2, 1024, 11008, 4, 64, "f16"),
                                                 (1, 512, 18944, 4, 64, "f16"), (1, 256, 2048, 8, 32, "f32"),
                                                 (2, 768, 1024, 8, 128, "bf16"), (5, 1024, 4096, 4, 64, "f16"),
                                                 (40, 512, 2048, 4, 64, "bf16"), (3, 24, 96, 4, 32, "f16"),
                                                 (40, 256, 640, 4, 64, "f16"), (300, 128, 2880, 4, 64, "bf16"), (6, 64, 1408, 4, 64, "f16")])
def test_qmm_norm_prologue(hip, m, n, k, bits, gs, dtype):
    """RMSNorm prologue (`has_norm` of the reference's MMA kernel, quantized.rs:3070-3095): fused into the
    single-row GEMV, a pass of its own in front of the other kernels.  Checked against the oracle, and bit
    for bit against the plain matmul of rows normalised on the host with the same f16 roundings."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(m + n + k + bits)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    nw = rng.uniform(0.5, 1.5, size=k).astype(np.float16)
    inv_rms = rng.uniform(0.3, 3.0, size=m).astype(np.float32)
    xn = model.norm_rows(x_as_f64(x, dtype), inv_rms, nw)
    ref = model.qmm(xn.astype(np.float64), words, s, b, gs, bits)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, gs, bits)
    print(f"qmm_norm M={m} N={n} K={k} bits={bits} gs={gs} {dtype}", flush=True)
    got = ops.qmm_norm(_dev(hip, x, dtype), qw, DeviceBuffer.from_numpy(nw), DeviceBuffer.from_numpy(inv_rms)).numpy()
    assert_close(got, ref, "qmm_norm")
    plain = ops.affine_quantized_matmul_batched(DeviceBuffer.from_numpy(xn), qw).numpy()
    assert np.array_equal(got, plain)


def test_qmm_norm_identity_scaling_and_validation(hip):
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(8)
    n, k = 256, 1024
    words, s, b = make_weight(rng, n, k, 4)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    for m in (1, 6):
        x = make_x(rng, m, k)
        xd = DeviceBuffer.from_numpy(x)
        plain = ops.affine_quantized_matmul_batched(xd, qw).numpy()
        ones_w, ones_r = DeviceBuffer.from_numpy(np.ones(k, np.float16)), DeviceBuffer.from_numpy(np.ones(m, np.float32))
        assert np.array_equal(ops.qmm_norm(xd, qw, ones_w, ones_r).numpy(), plain)
        # a power of two per row scales the activations, hence the f32 sums and the f16 results, exactly
        twos = DeviceBuffer.from_numpy(np.full(m, 2.0, np.float32))
        assert np.array_equal(ops.qmm_norm(xd, qw, ones_w, twos).numpy(), (plain.astype(np.float32) * 2).astype(np.float16))
    xd = DeviceBuffer.from_numpy(make_x(rng, 2, k))
    w16, r32 = DeviceBuffer.from_numpy(np.ones(k, np.float16)), DeviceBuffer.from_numpy(np.ones(2, np.float32))
    with pytest.raises(ops.KernelError, match=r"norm_weight must be Float16 \[1024\]"):
        ops.qmm_norm(xd, qw, DeviceBuffer.from_numpy(np.ones(k, np.float32)), r32)
    with pytest.raises(ops.KernelError, match=r"norm_weight must be Float16 \[1024\]"):
        ops.qmm_norm(xd, qw, DeviceBuffer.from_numpy(np.ones(k - 8, np.float16)), r32)
    with pytest.raises(ops.KernelError, match=r"inv_rms must be Float32 \[2\]"):
        ops.qmm_norm(xd, qw, w16, DeviceBuffer.from_numpy(np.ones(3, np.float32)))
    with pytest.raises(ops.KernelError, match=r"inv_rms must be Float32 \[2\]"):
        ops.qmm_norm(xd, qw, w16, DeviceBuffer.from_numpy(np.ones(2, np.float16)))


@pytest.mark.parametrize("m,n,k", [(3, 512, 256), (16, 1024, 768), (9, 4096, 11008), (5, 64, 2304), (16, 256, 4096)])
def test_q8_multi_row_gemv_any_k_multiple_of_256(hip, m, n, k):
    """The 8-bit streaming GEMV takes K in multiples of 256: waves whose slabs lie past K sit the pass out."""
    rng = np.random.default_rng(m + n + k)
    words, s, b = make_weight(rng, n, k, 8)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 8)
    assert_close(_run(hip, words, s, b, x, 8, kernel=6), ref, f"q8 qmv M={m} N={n} K={k}")


@pytest.mark.parametrize("m", [1, 2, 4, 40])
def test_vocabulary_sized_projection(hip, m):
    """N = 151 936 output rows (a vocabulary projection, 311 MB of 4-bit weights): rows at both ends and a
    random sample are checked against the oracle, every output must be finite."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(151936 + m)
    n, k = 151936, 4096
    words = rng.integers(0, 2**32, size=(n, k // 8), dtype=np.uint64).astype(np.uint32)
    s = rng.uniform(0.005, 0.02, size=(n, k // 64)).astype(np.float16)
    b = (-8 * s.astype(np.float32)).astype(np.float16)
    x = make_x(rng, m, k)
    print(f"vocabulary projection M={m}", flush=True)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    out = ops.affine_quantized_matmul_batched(DeviceBuffer.from_numpy(x), qw).numpy()
    assert out.shape == (m, n) and np.all(np.isfinite(out))
    rows = np.unique(np.concatenate([np.arange(256), np.arange(n - 256, n), rng.integers(0, n, size=512)]))
    ref = model.qmm(x_as_f64(x, "f16"), words[rows], s[rows], b[rows], 64, 4)
    assert_close(out[:, rows], ref, f"M={m}")


@pytest.mark.parametrize("m,n,k", [(3, 1024, 4096), (8, 512, 1536), (13, 9216, 4096), (16, 2048, 512), (5, 64, 2048)])
def test_multi_row_gemv_group_size_128(hip, m, n, k):
    """Group size 128 on the streaming GEMV: one scale per 128-wide slab, applied to both of its halves."""
    rng = np.random.default_rng(m + n + k)
    words, s, b = make_weight(rng, n, k, 4, 128)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 128, 4)
    assert_close(_run(hip, words, s, b, x, 4, gs=128, kernel=1), ref, f"qmv gs128 M={m} N={n} K={k}")
    # group positions: a weight that is non-zero in one group only
    s2, b2 = np.zeros_like(s), np.zeros_like(b)
    s2[:, -1] = s[:, -1]
    ref2 = model.qmm(x_as_f64(x, "f16"), words, s2, b2, 128, 4)
    assert_close(_run(hip, words, s2, b2, x, 4, gs=128, kernel=1), ref2, "last group only")


@pytest.mark.parametrize("m,n,k", [(13, 9216, 4096), (16, 9216, 4096), (16, 8192, 1536), (8, 16384, 512), (9, 8192, 2048)])
def test_qmv_paired_tiles(hip, m, n, k):
    """Shapes whose 8-row chunks take two 16-row tiles per wave (grid still covers the CUs)."""
    rng = np.random.default_rng(m + n + k)
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    assert_close(_run(hip, words, s, b, x, 4, kernel=1), ref, f"qmv paired M={m} N={n} K={k}")


# ---- 3- and 6-bit weights (the reference's portable affine_qmv, quantized.rs:210-291) ---------------------

@pytest.mark.parametrize("bits", [3, 6])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("n,k", [(24, 256), (7, 1024), (130, 384)])
def test_three_and_six_bit_weights(hip, bits, gs, n, k):
    """The bit widths the weight type admits beside 2 / 4 / 8: `affine_quantized_matmul` runs them on the portable
    kernel with the reference's layout (10 / 5 values per word, whole words per group), the batched entry point
    rejects them like the reference's and takes them when the portable kernel is selected."""
    from rmlx_amd import ops, runtime as rt
    if k % gs != 0:
        pytest.skip("group size does not divide K")
    rng = np.random.default_rng(bits * 1000 + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, 5, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, gs, bits)
    assert_close(_run(hip, words, s, b, x[:1], bits, gs=gs, qmv_entry=True), ref[:1], f"qmv bits={bits} gs={gs}")
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, kernel=rt.KERNEL_GENERIC), ref, f"portable bits={bits} gs={gs} M=5")
    with pytest.raises(ops.KernelError, match="affine_quantized_matmul_batched requires bits==4 or bits==8"):
        _run(hip, words, s, b, x, bits, gs=gs)
    # every covered position picks out its value exactly; the positions of a group past its last whole word give 0
    q, covered = model.unpack_grouped(words, gs, bits)
    for kk in sorted({0, 1, 32 // bits - 1, 32 // bits, gs - 1, gs, gs + 9, k - gs, k - 1}):
        x1 = np.zeros((1, k), np.float16)
        x1[0, kk] = 1.0
        out = _run(hip, words, np.ones_like(s), np.zeros_like(b), x1, bits, gs=gs, qmv_entry=True)
        assert np.array_equal(out[0].astype(np.float64), q[:, kk].astype(np.float64) * covered[kk]), f"k={kk}"


# ---- single-row GEMV (decode; affine_qmv_fast_q4 / _q8, quantized.rs:394-695) ---------------------------

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("n,k", [(16, 2048), (24, 4096), (64, 4096), (48, 6144), (32, 8192), (40, 12288), (16, 16384)])
def test_single_row_gemv(hip, bits, gs, n, k):
    """One or two rows (one pass over the weights) at every group size the weight type admits; at group
    sizes 32 / 128 the kernel also takes up to 16 rows in passes of four."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 1000 + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    for m in ((1, 2) if gs == 64 else (1, 3, 16)):
        x = make_x(rng, m, k)
        ref = model.qmm(x_as_f64(x, "f16"), words, s, b, gs, bits)
        assert_close(_run(hip, words, s, b, x, bits, gs=gs), ref, f"auto bits={bits} gs={gs} N={n} K={k} M={m}")
        assert_close(_run(hip, words, s, b, x, bits, gs=gs, kernel=rt.KERNEL_QMV), ref,
                     f"qmv bits={bits} gs={gs} N={n} K={k} M={m}")


@pytest.mark.parametrize("n,k,bits,gs", [(2048, 16384, 4, 64), (1024, 12288, 8, 64), (64, 8192, 4, 32),
                                         (136, 16384, 4, 128), (520, 10240, 8, 128), (8, 16384, 4, 64)])
def test_single_row_split_k(hip, n, k, bits, gs):
    """Long rows of a short matrix (the reference's split-K case `K > 8192 && N <= 2048`, quantized.rs:992-1233,
    7246-7250): two or four waves share a weight row and add their partial sums in workgroup memory.  Against the
    oracle, with one-hot activations in every 1 KB chunk of a row (each lands in another wave), and through the
    fused store epilogues."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(n + k + bits + gs)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, 1, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, gs, bits)
    assert_close(_run(hip, words, s, b, x, bits, gs=gs), ref, f"split-K N={n} K={k} bits={bits} gs={gs}")
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, qmv_entry=True), ref, "through the qmv entry point")
    q = model.unpack_u32(words, bits).astype(np.float64)
    chunk = 8192 // bits
    for kk in sorted({c * chunk + off for c in range(k // chunk) for off in (0, chunk - 1)} | {k - 1}):
        x1 = np.zeros((1, k), np.float16)
        x1[0, kk] = 1.0
        out = _run(hip, words, np.ones_like(s), np.zeros_like(b), x1, bits, gs=gs)
        assert np.array_equal(out[0].astype(np.float64), q[:, kk]), f"k={kk}"
    e = rng.standard_normal((1, n)).astype(np.float32)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, gs, bits)
    xd, ed = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(e)
    assert_close(ops.qmm_add_residual(xd, qw, ed).numpy(), ref + e, "split-K + residual")
    assert_close(ops.qmm_swiglu(xd, qw, ed).numpy(), model.silu(e.astype(np.float64)) * ref, "split-K + SwiGLU")


@pytest.mark.parametrize("n,k,bits,m", [(16400, 2048, 4, 1), (9216, 4096, 4, 1), (24584, 1024, 8, 2), (33000, 2048, 4, 3)])
def test_single_row_gemv_more_row_blocks_than_resident_workgroups(hip, n, k, bits, m):
    """Tall matrices: the grid is sized to the workgroups the chip keeps resident and each of them walks several
    row blocks (an uneven share included); every output row against the oracle, plain and with the residual
    epilogue (whose operand is fetched per block)."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(n + k + bits)
    gs = 128 if m == 3 else 64  # (three rows stay on this kernel because N = 33000 is no multiple of 16, which the multi-row GEMV needs)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, gs, bits)
    assert_close(_run(hip, words, s, b, x, bits, gs=gs), ref, f"looping grid N={n} K={k} bits={bits} M={m}")
    e = rng.standard_normal((m, n)).astype(np.float16)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, gs, bits)
    out = ops.qmm_add_residual(DeviceBuffer.from_numpy(x), qw, DeviceBuffer.from_numpy(e)).numpy()
    assert_close(out, ref + e.astype(np.float64), "looping grid + residual")


@pytest.mark.parametrize("bits", [4, 8])
def test_single_row_gemv_positions_and_multi_row_kernel_agree(hip, bits):
    """One-hot activations pick out single weights exactly (every k position of a lane, chunk borders), and
    the multi-row kernel forced onto one row gives the same numbers within the tolerance."""
    from rmlx_amd import runtime as rt
    n, k = 32, 4096
    rng = np.random.default_rng(40 + bits)
    words, s, b = make_weight(rng, n, k, bits)
    s1, b0 = np.ones_like(s), np.zeros_like(b)
    q = model.unpack_u32(words, bits).astype(np.float64)
    ks = np.array(list(range(40)) + [63, 64, 127, 128, 1023, 1024, 2047, 2048, 2049, 2079, 2080, 4064, 4095])
    for kk in ks:  # one row per call: the single-row kernel
        x = np.zeros((1, k), np.float16)
        x[0, kk] = 1.0
        out = _run(hip, words, s1, b0, x, bits)
        assert np.array_equal(out[0].astype(np.float64), q[:, kk]), f"k={kk}"
    x = make_x(rng, 1, k)
    ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, bits)
    assert_close(_run(hip, words, s, b, x, bits, kernel=rt.KERNEL_QMV_ROWS), ref, "multi-row kernel at M=1")
    assert_close(_run(hip, words, s, b, x, bits, kernel=rt.KERNEL_QMV), ref, "single-row kernel")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 128])
@pytest.mark.parametrize("m,n,k,dtype", [(33, 64, 512, "f16"), (100, 128, 1024, "f16"), (200, 256, 1536, "bf16"),
                                          (64, 192, 2048, "f16"), (17, 64, 512, "f32")])
def test_qmm_group_sizes_32_and_128(hip, bits, gs, m, n, k, dtype):
    """The register-weights GEMM at the other group sizes the weight type admits: same result as the oracle and
    as the portable kernel."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits + gs + m + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype), ref, f"auto bits={bits} gs={gs} M={m}")
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype, kernel=rt.KERNEL_QMM), ref,
                 f"qmm bits={bits} gs={gs} M={m}")
    assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype, kernel=rt.KERNEL_GENERIC), ref,
                 f"portable bits={bits} gs={gs} M={m}")


def test_qmm_group_size_positions(hip):
    """Scales that differ per group and a one-hot row pick out s[n, k / gs] exactly: every lane group, both
    halves of a scale word, block borders."""
    from rmlx_amd import runtime as rt
    for bits in (4, 8):
        for gs in (32, 64, 128):
            n, k, m = 64, 1024, 32
            rng = np.random.default_rng(gs * 10 + bits)
            words = np.full((n, k * bits // 32), 0x11111111 if bits == 4 else 0x01010101, np.uint32)  # q = 1 everywhere
            s = (rng.integers(1, 64, size=(n, k // gs)) / 8.0).astype(np.float16)
            b = np.zeros((n, k // gs), np.float16)
            ks = rng.choice(k, size=m, replace=False)
            x = np.zeros((m, k), np.float16)
            x[np.arange(m), ks] = 1.0
            out = _run(hip, words, s, b, x, bits, gs=gs, kernel=rt.KERNEL_QMM)
            want = s[:, ks // gs].T.astype(np.float64)
            assert np.array_equal(out.astype(np.float64), want), f"bits={bits} gs={gs}"


@pytest.mark.parametrize("bits,gs", [(4, 64), (4, 32), (4, 128), (8, 64), (8, 32), (8, 128)])
@pytest.mark.parametrize("m,n,k,dtype", [(64, 128, 512, "f16"), (130, 256, 1024, "f16"), (512, 1024, 1536, "bf16"), (1, 128, 512, "f16"),
                                         (333, 384, 2048, "f32"), (65, 128, 4096, "f16"), (96, 256, 4608, "f16")])
def test_k_split_gemm(hip, bits, gs, m, n, k, dtype):
    """The K-split GEMM (64 x 128 tiles, 32x32x16 MFMAs; kernel selector 7) on its own: every bit width and group
    size, ragged M (rows past M read as zero), one and several k-block groups, all activation dtypes; at group size 64
    K up to 4096 (scales and biases staged in LDS, rows shorter than a cache line included) and beyond (read from
    global memory as at the other group sizes)."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 1000 + gs + m + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
    assert_close(_run(hip, words, s, b, x, bits, dtype=dtype, gs=gs, kernel=rt.KERNEL_QMM_K2), ref,
                 f"k-split gemm M={m} N={n} K={k} bits={bits} gs={gs} {dtype}")


def test_k_split_gemm_positions_epilogues_and_dispatch(hip):
    """One-hot rows against per-group scales pick out s[n, k / gs] exactly (every lane half, k step, k half and
    scale word); the fused epilogues; and the shapes the ladder sends here agree with the register-weights GEMM."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    for bits in (4, 8):
        for gs in (32, 64, 128):
            n, k, m = 128, 1024, 64
            rng = np.random.default_rng(gs * 10 + bits)
            words = np.full((n, k * bits // 32), 0x11111111 if bits == 4 else 0x01010101, np.uint32)  # q = 1 everywhere
            s = (rng.integers(1, 64, size=(n, k // gs)) / 8.0).astype(np.float16)
            b = np.zeros((n, k // gs), np.float16)
            ks = rng.choice(k, size=m, replace=False)
            x = np.zeros((m, k), np.float16)
            x[np.arange(m), ks] = 1.0
            out = _run(hip, words, s, b, x, bits, gs=gs, kernel=rt.KERNEL_QMM_K2)
            assert np.array_equal(out.astype(np.float64), s[:, ks // gs].T.astype(np.float64)), f"bits={bits} gs={gs}"
    rng = np.random.default_rng(99)
    m, n, k = 400, 4096, 1024  # 7 x 32 = 224 tiles: one round over most of a 256-CU chip -> the ladder picks this kernel
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    base = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    auto = _run(hip, words, s, b, x, 4)
    assert_close(auto, base, "auto")
    assert np.array_equal(auto, _run(hip, words, s, b, x, 4, kernel=rt.KERNEL_QMM_K2))
    assert_close(_run(hip, words, s, b, x, 4, kernel=rt.KERNEL_QMM_RW), base, "register-weights GEMM")
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    xd = DeviceBuffer.from_numpy(x)
    for edtype in (np.float16, np.float32):
        e = rng.standard_normal((m, n)).astype(edtype)
        ed = DeviceBuffer.from_numpy(e)
        assert_close(ops.qmm_add_residual(xd, qw, ed).numpy(), base + e.astype(np.float64), "qmm_add_residual")
        assert_close(ops.qmm_swiglu(xd, qw, ed).numpy(), model.silu(e.astype(np.float64)) * base, "qmm_swiglu")
    with pytest.raises(ops.KernelError, match="register-weights qmm kernels require"):
        _run(hip, *make_weight(rng, 64, 256, 4), make_x(rng, 8, 256), 4, kernel=rt.KERNEL_QMM_K2)


@pytest.mark.parametrize("bits,gs", [(4, 64), (4, 32), (4, 128), (8, 64), (8, 32), (8, 128)])
@pytest.mark.parametrize("m,n,k,dtype", [(128, 128, 512, "f16"), (130, 256, 1024, "f16"), (512, 1024, 1536, "bf16"), (1, 128, 512, "f16"),
                                         (333, 384, 2048, "f32"), (193, 128, 4096, "f16")])
def test_k_split_gemm_tall_tiles(hip, bits, gs, m, n, k, dtype):
    """The same kernel with 128 x 128 tiles (kernel selector 9): every bit width and group size (with one or two
    activation register sets), ragged M with one to four empty 32-row fragments in the last tile, all activation dtypes;
    bit-identical to the 64-row tiles (every output sums the same products in the same order).  8-bit weights at group
    size 32 / 64 with bf16 activations have no such build."""
    from rmlx_amd import ops, runtime as rt
    rng = np.random.default_rng(bits * 1000 + gs + m + n + k + 1)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    if bits == 8 and gs != 128 and dtype == "bf16":
        with pytest.raises(ops.KernelError, match="128 x 128 K-split qmm kernel requires"):
            _run(hip, words, s, b, x, bits, dtype=dtype, gs=gs, kernel=rt.KERNEL_QMM_K2_TALL)
        return
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
    out = _run(hip, words, s, b, x, bits, dtype=dtype, gs=gs, kernel=rt.KERNEL_QMM_K2_TALL)
    assert_close(out, ref, f"k-split gemm, 128-row tiles M={m} N={n} K={k} bits={bits} gs={gs} {dtype}")
    assert np.array_equal(out, _run(hip, words, s, b, x, bits, dtype=dtype, gs=gs, kernel=rt.KERNEL_QMM_K2))


@pytest.mark.parametrize("bits,gs", [(4, 64), (4, 32), (4, 128), (8, 64), (8, 32), (8, 128)])
@pytest.mark.parametrize("m,n,k,dtype", [(32, 128, 512, "f16"), (45, 256, 1024, "f16"), (160, 512, 1536, "bf16"), (1, 128, 512, "f16"),
                                         (97, 384, 2048, "f32"), (64, 128, 8192, "f16")])
def test_k_split_gemm_flat_tiles(hip, bits, gs, m, n, k, dtype):
    """The same kernel with 32 x 128 tiles (kernel selector 10: one activation fragment per wave): every bit width and
    group size, ragged M, all activation dtypes; bit-identical to the 64-row tiles."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 1000 + gs + m + n + k + 2)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
    out = _run(hip, words, s, b, x, bits, dtype=dtype, gs=gs, kernel=rt.KERNEL_QMM_K2_FLAT)
    assert_close(out, ref, f"k-split gemm, 32-row tiles M={m} N={n} K={k} bits={bits} gs={gs} {dtype}")
    assert np.array_equal(out, _run(hip, words, s, b, x, bits, dtype=dtype, gs=gs, kernel=rt.KERNEL_QMM_K2))


@pytest.mark.parametrize("m,n,k,dtype", [(32, 64, 2048, "f16"), (45, 256, 4096, "f16"), (160, 512, 2048, "bf16"), (1, 64, 2048, "f16"),
                                         (97, 384, 6144, "f32"), (128, 128, 14336, "f16")])
def test_gemm_with_k_split_four_ways(hip, m, n, k, dtype):
    """32 x 64 tiles with K split four ways inside the workgroup (kernel selector 11; 4-bit weights, group size 64,
    K a multiple of 2048): ragged M, all activation dtypes, against the oracle; shapes and weights it does not take."""
    from rmlx_amd import ops, runtime as rt
    rng = np.random.default_rng(m + n + k + 11)
    words, s, b = make_weight(rng, n, k, 4, 64)
    x = make_x(rng, m, k, dtype)
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, 64, 4)
    assert_close(_run(hip, words, s, b, x, 4, dtype=dtype, kernel=rt.KERNEL_QMM_K4), ref, f"4-way k-split gemm M={m} N={n} K={k} {dtype}")
    with pytest.raises(ops.KernelError, match="32 x 64 K-split qmm kernel requires"):
        _run(hip, *make_weight(rng, 64, 1024, 4, 64), make_x(rng, 8, 1024), 4, kernel=rt.KERNEL_QMM_K4)  # K % 2048 != 0
    with pytest.raises(ops.KernelError, match="32 x 64 K-split qmm kernel requires"):
        _run(hip, *make_weight(rng, 64, 2048, 8, 64), make_x(rng, 8, 2048), 8, kernel=rt.KERNEL_QMM_K4)  # 8-bit


@pytest.mark.parametrize("bits,gs", [(4, 64), (4, 32), (8, 64), (8, 128)])
@pytest.mark.parametrize("m,n,k,dtype", [(40, 128, 2048, "f16"), (130, 384, 4096, "bf16"), (300, 256, 2048, "f16")])
def test_gemm_layout_gives_identical_results(hip, bits, gs, m, n, k, dtype):
    """The tile-contiguous copy of the weights (rmlx_hip_qweight_set_gemm_layout): every K-split GEMM returns the same bits with
    and without it, the automatic choice lands on the oracle with it, the other kernels ignore it; handles without such a
    layout and buffers that are too small are refused."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits + gs + m + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    x = make_x(rng, m, k, dtype)
    xd = DeviceBuffer.from_numpy(x, rt.BF16) if dtype == "bf16" else DeviceBuffer.from_numpy(x)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, gs, bits)
    ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
    for kernel in (rt.KERNEL_QMM_K2, rt.KERNEL_QMM_K2_TALL, rt.KERNEL_QMM_K2_FLAT, rt.KERNEL_QMM_K4, rt.KERNEL_AUTO, rt.KERNEL_QMV_ROWS):
        try:
            plain = ops.affine_quantized_matmul_batched(xd, qw, kernel=kernel).numpy()
        except ops.KernelError:
            continue  # (the kernel does not take this weight format)
        assert qw.use_gemm_layout(True)
        packed = ops.affine_quantized_matmul_batched(xd, qw, kernel=kernel).numpy()
        qw.use_gemm_layout(False)
        if kernel == rt.KERNEL_AUTO:
            assert_close(packed, ref, f"auto with the GEMM layout, bits={bits} gs={gs} M={m}")
        else:
            assert np.array_equal(plain, packed), (kernel, bits, gs, m)
    odd = ops.QuantizedWeight.from_numpy(*make_weight(rng, 64, 512, 4, 64), 64, 4)  # N % 128 != 0
    assert not odd.use_gemm_layout(True)
    with pytest.raises(ops.KernelError, match="no GEMM layout"):
        rt.check(rt.lib().rmlx_hip_qweight_set_gemm_layout(odd.handle, xd.ptr, 1 << 20, None))
    with pytest.raises(ops.KernelError, match="buffer too small"):
        rt.check(rt.lib().rmlx_hip_qweight_set_gemm_layout(qw.handle, xd.ptr, 16, None))


def test_k_split_gemm_flat_tiles_epilogues_and_dispatch(hip):
    """The fused epilogues on the 32-row tiles and a shape the ladder sends there (one round of 32 x 128 tiles where the
    register-weights GEMM would need tiles larger than 32 x 64)."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(99)
    cus = rt.device_info()["compute_units"]
    n, k = 2048, 1024
    m = 32 * (cus // (n // 128)) - 5  # as many 32 x 128 tiles as fit one round; more 32 x 64 tiles than CUs
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    base = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    auto = _run(hip, words, s, b, x, 4)
    assert_close(auto, base, "auto")
    assert np.array_equal(auto, _run(hip, words, s, b, x, 4, kernel=rt.KERNEL_QMM_K2_FLAT))
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    xd = DeviceBuffer.from_numpy(x)
    for edtype in (np.float16, np.float32):
        e = rng.standard_normal((m, n)).astype(edtype)
        ed = DeviceBuffer.from_numpy(e)
        assert_close(ops.qmm_add_residual(xd, qw, ed).numpy(), base + e.astype(np.float64), "qmm_add_residual")
        assert_close(ops.qmm_swiglu(xd, qw, ed).numpy(), model.silu(e.astype(np.float64)) * base, "qmm_swiglu")
    with pytest.raises(ops.KernelError, match="register-weights qmm kernels require"):
        _run(hip, *make_weight(rng, 64, 512, 4, 64), make_x(rng, 8, 512), 4, kernel=rt.KERNEL_QMM_K2_FLAT)  # N % 128 != 0


def test_k_split_gemm_tall_tiles_positions_epilogues_and_dispatch(hip):
    """One-hot rows against per-group scales (every fragment, lane half, k step, k half and scale word of the 128-row
    tile); the fused epilogues; the shapes the ladder sends to the 128-row tiles; shapes it does not take."""
    from rmlx_amd import ops, runtime as rt
    from rmlx_amd.runtime import DeviceBuffer
    for bits, gs in ((4, 64), (4, 32), (4, 128), (8, 64), (8, 32), (8, 128)):
        n, k, m = 128, 1024, 128
        rng = np.random.default_rng(gs * 10 + bits + 1)
        words = np.full((n, k * bits // 32), 0x11111111 if bits == 4 else 0x01010101, np.uint32)  # q = 1 everywhere
        s = (rng.integers(1, 64, size=(n, k // gs)) / 8.0).astype(np.float16)
        b = np.zeros((n, k // gs), np.float16)
        ks = rng.choice(k, size=m, replace=False)
        x = np.zeros((m, k), np.float16)
        x[np.arange(m), ks] = 1.0
        out = _run(hip, words, s, b, x, bits, gs=gs, kernel=rt.KERNEL_QMM_K2_TALL)
        assert np.array_equal(out.astype(np.float64), s[:, ks // gs].T.astype(np.float64)), f"bits={bits} gs={gs}"
    rng = np.random.default_rng(98)
    cus = rt.device_info()["compute_units"]
    n, k = 2048, 1024
    m = 128 * ((6 * cus + 9) // 10 // (n // 128) + 1) - 28  # 128-row tiles: 0.6 rounds over the chip or more; ragged
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    base = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, 4)
    auto = _run(hip, words, s, b, x, 4)
    assert_close(auto, base, "auto")
    assert np.array_equal(auto, _run(hip, words, s, b, x, 4, kernel=rt.KERNEL_QMM_K2_TALL))
    qw = ops.QuantizedWeight.from_numpy(words, s, b, 64, 4)
    xd = DeviceBuffer.from_numpy(x)
    for edtype in (np.float16, np.float32):
        e = rng.standard_normal((m, n)).astype(edtype)
        ed = DeviceBuffer.from_numpy(e)
        assert_close(ops.qmm_add_residual(xd, qw, ed).numpy(), base + e.astype(np.float64), "qmm_add_residual")
        assert_close(ops.qmm_swiglu(xd, qw, ed).numpy(), model.silu(e.astype(np.float64)) * base, "qmm_swiglu")
    # the large prefill shape (4096 x 4096 weights, 4096 rows; the ladder sends it to the 128-row tiles): rows sampled
    # from every row tile against the oracle, every row against the register-weights GEMM
    m = n = k = 4096
    words, s, b = make_weight(rng, n, k, 4)
    x = make_x(rng, m, k)
    auto = _run(hip, words, s, b, x, 4)
    assert np.array_equal(auto, _run(hip, words, s, b, x, 4, kernel=rt.KERNEL_QMM_K2_TALL))
    rows = (np.arange(32)[:, None] * 128 + rng.integers(0, 128, size=(32, 2))).reshape(-1)
    assert_close(auto[rows], model.qmm(x_as_f64(x[rows], "f16"), words, s, b, 64, 4), "4096 x 4096 x 4096, sampled rows")
    other = _run(hip, words, s, b, x, 4, kernel=rt.KERNEL_QMM_RW).astype(np.float64)
    assert np.abs(auto.astype(np.float64) - other).max() <= 2.0 ** -9 * np.abs(other).max()  # two f16 roundings of one value
    with pytest.raises(ops.KernelError, match="128 x 128 K-split qmm kernel requires"):
        _run(hip, *make_weight(rng, 64, 512, 4, 64), make_x(rng, 8, 512), 4, kernel=rt.KERNEL_QMM_K2_TALL)  # N % 128 != 0


@pytest.mark.parametrize("bits,gs", [(4, 64), (4, 32), (4, 128), (8, 64), (8, 32)])
@pytest.mark.parametrize("n,k", [(16, 11008), (24, 3584), (8, 2560), (16, 1408), (40, 64 * 33), (8, 128)])
def test_single_row_gemv_any_k(hip, bits, gs, n, k):
    """K that is not a multiple of the 1 KB chunk (nor of 512): the tail lanes meet zeros.  Such shapes also
    take a few rows on this kernel, because the multi-row GEMV needs K % 512 == 0."""
    if k % gs != 0:
        pytest.skip("group size does not divide K")
    rng = np.random.default_rng(bits * 7 + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    for m in (1, 2, 5, 16):
        x = make_x(rng, m, k)
        ref = model.qmm(x_as_f64(x, "f16"), words, s, b, gs, bits)
        assert_close(_run(hip, words, s, b, x, bits, gs=gs), ref, f"bits={bits} gs={gs} N={n} K={k} M={m}")
    # the last weight of a row, the first one past the last whole chunk, a group border
    q = model.unpack_u32(words, bits).astype(np.float64)
    for kk in sorted({k - 1, (k // 2048) * 2048 if k >= 2048 else 0, k // 2, gs - 1, min(gs, k - 1)}):
        x = np.zeros((1, k), np.float16)
        x[0, kk] = 1.0
        out = _run(hip, words, np.ones_like(s), np.zeros_like(b), x, bits, gs=gs)
        assert np.array_equal(out[0].astype(np.float64), q[:, kk]), f"bits={bits} gs={gs} K={k} k={kk}"


@pytest.mark.parametrize("bits,n,k", [(4, 16, 18944), (4, 8, 28672), (8, 16, 24576), (8, 8, 28672), (4, 8, 16384 + 64)])
def test_single_row_gemv_long_k(hip, bits, n, k):
    """K beyond 16384: the activation image is staged in more than four rounds (up to the LDS limit; past it
    the multi-row kernels take over)."""
    rng = np.random.default_rng(bits + n + k)
    words, s, b = make_weight(rng, n, k, bits)
    for m in (1, 2):
        x = make_x(rng, m, k)
        ref = model.qmm(x_as_f64(x, "f16"), words, s, b, 64, bits)
        assert_close(_run(hip, words, s, b, x, bits), ref, f"bits={bits} N={n} K={k} M={m}")


@pytest.mark.parametrize("bits,n,k", [(4, 512, 2880), (8, 256, 896), (4, 384, 1152)])
@pytest.mark.parametrize("m", [17, 70, 300])
def test_batches_on_shapes_without_a_gemm(hip, bits, n, k, m):
    """K off the multiples of 256 (hidden sizes such as 2880, 896, 1152): batches beyond 16 rows run on the LDS-staged GEMM
    with padded activations at group size 64, on the single-row kernels in passes at the other group sizes, instead of
    the portable kernel.  Against the oracle."""
    rng = np.random.default_rng(bits + n + k + m)
    words, s, b = make_weight(rng, n, k, bits, 64)
    x = make_x(rng, m, k)
    ref = model.qmm(x.astype(np.float64), words, s, b, 64, bits)
    assert_close(_run(hip, words, s, b, x, bits), ref, f"Q{bits} M={m} N={n} K={k}")


@pytest.mark.parametrize("bits,dtype", [(4, "f16"), (8, "f16"), (8, "bf16"), (4, "f32")])
@pytest.mark.parametrize("n,k", [(64, 320), (128, 448), (192, 2880), (64, 1152)])
def test_staged_gemm_with_k_off_its_unrolled_iteration(hip, bits, dtype, n, k):
    """The LDS-staged GEMM where K is a multiple of 64 but not of 256 (an odd number of groups per row puts a row's scales
    on a 2-byte boundary): the activations are padded with zeros to whole iterations, weight and scale loads stop at the
    row's end.  Scales and biases of the neighbouring rows are large, so a load past the row's end would show.  Against
    the oracle, at one partial tile, whole tiles and 128-row tiles."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 7 + n + k)
    words, s, b = make_weight(rng, n, k, bits, 64)
    for m in (17, 64, 300):
        x = make_x(rng, m, k, dtype)
        ref = model.qmm(x_as_f64(x, dtype), words, s, b, 64, bits)
        for kernel in (rt.KERNEL_QMM_LDS, rt.KERNEL_AUTO) + ((rt.KERNEL_QMM_BF16,) if (bits, dtype) == (8, "bf16") else ()):
            assert_close(_run(hip, words, s, b, x, bits, dtype=dtype, kernel=kernel), ref,
                         f"Q{bits} {dtype} M={m} N={n} K={k} kernel={kernel}")
    # the last row's scales end the buffer: nothing may be read past it (the device allocation ends there too)
    x = make_x(rng, 33, k, dtype)
    s2, b2 = s.copy(), b.copy()
    s2[:, -1] = 0
    b2[:, -1] = 0
    ref = model.qmm(x_as_f64(x, dtype), words, s2, b2, 64, bits)
    assert_close(_run(hip, words, s2, b2, x, bits, dtype=dtype, kernel=rt.KERNEL_QMM_LDS), ref, "last group zeroed")


@pytest.mark.parametrize("bits,gs,n,k", [(bits, gs, n, k) for bits, gs in [(4, 64), (8, 64), (4, 32), (4, 128)]
                                          for n, k in [(128, 576), (192, 1088), (64, 2880), (256, 4160), (64, 2048), (128, 1536)]
                                          if k % gs == 0])
def test_staged_gemm_with_its_k_loop_split(hip, bits, gs, n, k):
    """A launch of few tiles cuts the k loop of the LDS-staged GEMM into two, three or four ranges of whole unrolled iterations
    (K padded up to them: 576 -> two ranges of 8 steps, the second with one step of weights; 1088 -> three of 8; 2880 -> four
    of 12; 4160 -> four of 20; 2048 and 1536 without padding) that leave f32 partial sums, and one pass adds them up.
    Scales and biases grow along the row, so a range that starts at the wrong group shows; the last row's last group is
    zeroed in a second run, so a load past the row's end shows.  Against the oracle, from one row to two tiles of rows."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 13 + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    ramp = (1.0 + np.arange(k // gs) % 5).astype(np.float16)
    s = (s * ramp).astype(np.float16)
    b = (b * ramp[::-1]).astype(np.float16)
    for m, dtype in ((1, "f16"), (9, "f16"), (64, "bf16"), (100, "f32")):
        x = make_x(rng, m, k, dtype)
        ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
        print(f"split staged GEMM Q{bits} gs={gs} {dtype} M={m} N={n} K={k}", flush=True)
        assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype, kernel=rt.KERNEL_QMM_LDS), ref,
                     f"Q{bits} gs={gs} {dtype} M={m} N={n} K={k}")
    x = make_x(rng, 33, k, "f16")
    s2, b2 = s.copy(), b.copy()
    s2[:, -1] = 0
    b2[:, -1] = 0
    ref = model.qmm(x_as_f64(x, "f16"), words, s2, b2, gs, bits)
    assert_close(_run(hip, words, s2, b2, x, bits, gs=gs, kernel=rt.KERNEL_QMM_LDS), ref, "last group zeroed")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 128])
@pytest.mark.parametrize("n,k", [(64, 256), (128, 384), (64, 768), (192, 2944), (64, 1280)])
def test_staged_gemm_at_group_sizes_32_and_128(hip, bits, gs, n, k):
    """The LDS-staged GEMM at the other group sizes (two groups per 64-wide step, or one group per two steps), with K on
    and off whole unrolled iterations: what K not a multiple of 512 runs on at these group sizes.  Every group gets its
    own scale and bias magnitude, so a wrong group index shows.  Against the oracle."""
    from rmlx_amd import runtime as rt
    if k % gs:
        pytest.skip("K is not a multiple of the group size")
    rng = np.random.default_rng(bits * 11 + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    ramp = (1.0 + np.arange(k // gs) % 7).astype(np.float16)
    s = (s * ramp).astype(np.float16)
    b = (b * ramp[::-1]).astype(np.float16)
    for m, dtype in ((17, "f16"), (70, "bf16"), (300, "f32")):
        x = make_x(rng, m, k, dtype)
        ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
        for kernel in (rt.KERNEL_QMM_LDS, rt.KERNEL_AUTO):
            assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype, kernel=kernel), ref,
                         f"Q{bits} gs={gs} {dtype} M={m} N={n} K={k} kernel={kernel}")
    with pytest.raises(Exception, match="group size 64"):
        _run(hip, words, s, b, make_x(rng, 32, k, "bf16"), bits, gs=gs, dtype="bf16", kernel=rt.KERNEL_QMM_BF16)


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32), (8, 32)])
@pytest.mark.parametrize("n,k", [(64, 256), (128, 384), (256, 640), (64, 1408), (128, 2816)])
def test_gemms_and_multi_row_gemv_with_k_in_whole_blocks_of_128(hip, bits, gs, n, k):
    """K a multiple of 128 but not of 512 (11008, 8960, 4864, 6912 in real models): the register-weights GEMM pads its last
    unrolled round with zero activations and clamps weight, scale and bias loads to the row; the 4-bit multi-row GEMV walks
    whole slabs with a shorter last part.  Scales and biases grow along the row so a wrong or repeated group shows.
    Against the oracle through the automatic choice and every kernel that takes the shape, f16 / bf16 / f32 rows."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 13 + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    ramp = (1.0 + np.arange(k // gs) % 5).astype(np.float16)
    s, b = (s * ramp).astype(np.float16), (b * ramp[::-1]).astype(np.float16)
    for m, dtype in ((3, "f16"), (8, "bf16"), (16, "f16"), (17, "f16"), (70, "bf16"), (130, "f32"), (600, "f16")):
        x = make_x(rng, m, k, dtype)
        ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
        kernels = [rt.KERNEL_AUTO, rt.KERNEL_QMM, rt.KERNEL_QMM_LDS]
        if k >= 512:  # (the tail form wants four blocks; shorter rows run on the LDS-staged GEMM)
            kernels.append(rt.KERNEL_QMM_RW)
        if bits == 4 and gs == 64:
            kernels.append(rt.KERNEL_QMV)
        for kernel in kernels:
            assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype, kernel=kernel), ref,
                         f"Q{bits} gs={gs} {dtype} M={m} N={n} K={k} kernel={kernel}")


@pytest.mark.parametrize("bits,n,k", [(4, 9728, 896), (4, 16384, 1024), (4, 6144, 2048), (8, 8192, 512), (4, 4864, 896)])
def test_one_and_two_rows_over_short_rows_of_tall_matrices(hip, bits, n, k):
    """One or two activation rows over a tall matrix of short rows (an up projection from a hidden size of 896, a
    vocabulary head): the automatic choice runs the multi-row GEMV there, the single-row kernel elsewhere.  Both against
    the oracle, and the automatic choice agrees with one of them bit for bit."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits + n + k)
    words, s, b = make_weight(rng, n, k, bits, 64)
    for m in (1, 2):
        x = make_x(rng, m, k)
        ref = model.qmm(x.astype(np.float64), words, s, b, 64, bits)
        auto = _run(hip, words, s, b, x, bits)
        single = _run(hip, words, s, b, x, bits, kernel=rt.KERNEL_QMV)
        rows = _run(hip, words, s, b, x, bits, kernel=rt.KERNEL_QMV_ROWS)
        for got, what in ((auto, "auto"), (single, "single-row"), (rows, "multi-row")):
            assert_close(got, ref, f"Q{bits} M={m} N={n} K={k} {what}")
        assert np.array_equal(auto.view(np.uint16), single.view(np.uint16)) or np.array_equal(auto.view(np.uint16), rows.view(np.uint16))


@pytest.mark.parametrize("bits,gs,n,k", [(4, 64, 4096, 4096), (8, 64, 512, 2048), (4, 32, 256, 1152), (4, 128, 4096, 18944), (8, 128, 4096, 2560)])
def test_bf16_rows_are_converted_inside_the_single_row_kernel(hip, bits, gs, n, k):
    """One or two bf16 (or f32) activation rows: the single-row kernel converts them to f16 while it stages them (no cast
    launch in front of a decoding step's matmuls).  Bit-identical to the same matmul over the rows converted on the host the way
    the cast kernel does (through f32, round to nearest even), and on the oracle; with a fused epilogue as well."""
    from rmlx_amd import ops
    from rmlx_amd.runtime import DeviceBuffer
    rng = np.random.default_rng(bits + gs + n + k)
    words, s, b = make_weight(rng, n, k, bits, gs)
    qw = ops.QuantizedWeight.from_numpy(words, s, b, gs, bits)
    for m in (1, 2, 3, 8, 13, 16):  # (from three rows on: the multi-row GEMVs, which convert inside as well)
        x = make_x(rng, m, k, "bf16")
        x16 = model.bf16_bits_to_f32(x).astype(np.float16)
        got = _run(hip, words, s, b, x, bits, gs=gs, dtype="bf16")
        want = _run(hip, words, s, b, x16, bits, gs=gs)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (m, n, k)
        assert_close(got, model.qmm(x_as_f64(x, "bf16"), words, s, b, gs, bits), f"bf16 M={m} N={n} K={k} Q{bits} gs={gs}")
        if m <= 2:  # f32 rows: rounded to f16 inside the single-row kernel, as the cast kernel rounds them
            x32 = make_x(rng, m, k, "f32")
            got32 = _run(hip, words, s, b, x32, bits, gs=gs, dtype="f32")
            want32 = _run(hip, words, s, b, x32.astype(np.float16), bits, gs=gs)
            assert np.array_equal(got32.view(np.uint16), want32.view(np.uint16)), ("f32", m, n, k)
        e = rng.standard_normal((m, n)).astype(np.float16)
        res = ops.qmm_add_residual(_dev(hip, x, "bf16"), qw, DeviceBuffer.from_numpy(e)).numpy()
        res16 = ops.qmm_add_residual(DeviceBuffer.from_numpy(x16), qw, DeviceBuffer.from_numpy(e)).numpy()
        assert np.array_equal(res.view(np.uint16), res16.view(np.uint16))


def test_random_shapes_through_the_ladder(hip):
    """Sixty seeded random (M, N, K, bits, group size) shapes through the automatic dispatch: whatever kernel
    the ladder picks (single-row, multi-row GEMV, both GEMMs, portable) must land on the oracle."""
    rng = np.random.default_rng(20240607)
    for case in range(60):
        bits = int(rng.choice([4, 8]))
        gs = int(rng.choice([32, 64, 64, 128]))
        n = int(rng.integers(1, 34)) * 8
        k = int(rng.integers(1, 37)) * 128 if rng.random() < 0.6 else int(rng.integers(1, 73)) * gs
        k = (k // gs) * gs or gs
        m = int(rng.choice([1, 2, 3, 5, 8, 16, 17, 33, 70]))
        dtype = str(rng.choice(["f16", "f16", "bf16", "f32"]))
        words, s, b = make_weight(rng, n, k, bits, gs)
        x = make_x(rng, m, k, dtype)
        ref = model.qmm(x_as_f64(x, dtype), words, s, b, gs, bits)
        assert_close(_run(hip, words, s, b, x, bits, gs=gs, dtype=dtype), ref,
                     f"case {case}: M={m} N={n} K={k} bits={bits} gs={gs} {dtype}")


@pytest.mark.parametrize("m", [1, 3, 8, 11, 16])
@pytest.mark.parametrize("n,k", [(48, 512), (512, 4096), (24576, 512)])
def test_q4_group_32_on_the_wave_per_tile_gemv(hip, n, k, m):
    """4-bit weights at group size 32 on the multi-row streaming GEMV (kernel selector 6: a wave per 16-row weight tile,
    two matrix-instruction chains per slab), forced and through the ladder (which takes it for 3 to 8 rows over very wide
    matrices, the single-row kernel up to 4 rows and the GEMM above), against the oracle."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(n + k + m + 32)
    words, s, b = make_weight(rng, n, k, 4, 32)
    x = make_x(rng, m, k)
    ref = model.qmm(x.astype(np.float64), words, s, b, 32, 4)
    assert_close(_run(hip, words, s, b, x, 4, gs=32, kernel=rt.KERNEL_QMV_ROWS), ref, f"Q4 gs32 M={m} N={n} K={k} (wave per tile)")
    assert_close(_run(hip, words, s, b, x, 4, gs=32), ref, f"Q4 gs32 M={m} N={n} K={k} (auto)")


@pytest.mark.parametrize("m", [3, 8, 16])
@pytest.mark.parametrize("n,k", [(512, 1024), (1024, 4096)])
def test_q8_group_128_on_the_streaming_gemv(hip, n, k, m):
    """8-bit weights at group size 128 on the multi-row streaming GEMV (two neighbouring 64-wide slabs share a scale),
    forced and through the ladder, against the oracle."""
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(n + k + m)
    words, s, b = make_weight(rng, n, k, 8, 128)
    x = make_x(rng, m, k)
    ref = model.qmm(x.astype(np.float64), words, s, b, 128, 8)
    assert_close(_run(hip, words, s, b, x, 8, gs=128, kernel=rt.KERNEL_QMV_ROWS), ref, f"Q8 gs128 M={m} N={n} K={k} (streaming GEMV)")
    assert_close(_run(hip, words, s, b, x, 8, gs=128), ref, f"Q8 gs128 M={m} N={n} K={k} (auto)")


@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("n,k", [(256, 4096), (64, 1088 * 2), (4096, 4096), (128, 11008 + 256), (8, 64 * 2)])
def test_two_bit_single_row_kernel(hip, n, k, gs):
    """2-bit weights through affine_quantized_matmul (the reference's affine_qmv takes every bit width,
    quantized.rs:211-290) on the 2-bit single-row kernel: whole and partial chunks of 4096 values, all three group sizes,
    against the oracle and against the portable kernel on the same inputs; one-hot weights pick single activations."""
    from rmlx_amd import ops, runtime as rt
    rng = np.random.default_rng(n + k + gs)
    k = (k // gs) * gs
    words, s, b = make_weight(rng, n, k, 2, gs)
    x = make_x(rng, 1, k)
    ref = model.qmm(x.astype(np.float64), words, s, b, gs, 2)
    got = _run(hip, words, s, b, x[0], 2, gs=gs, qmv_entry=True)
    assert_close(got, ref, f"2-bit N={n} K={k} gs={gs}")
    portable = _run(hip, words, s, b, x, 2, gs=gs, kernel=rt.KERNEL_GENERIC)
    assert_close(portable, ref, f"2-bit N={n} K={k} gs={gs} (portable)")
    # value position: q = 1 at one (row, k) with scale 1 and bias 0 everywhere returns exactly x[k] in that row
    wz = np.zeros_like(words)
    ones, zeros = np.ones_like(s), np.zeros_like(b)
    picks = [(0, 0), (n - 1, k - 1), (n // 2, min(k - 1, 4097)), (3 % n, 23), (5 % n, min(k - 1, 2048 + 40))]
    for r, kk in picks:
        wz[r, kk // 16] |= np.uint32(1) << np.uint32(2 * (kk % 16))
    got = _run(hip, wz, ones, zeros, x[0], 2, gs=gs, qmv_entry=True)[0].astype(np.float64)
    want = np.zeros(n)
    for r, kk in picks:
        want[r] += float(x[0, kk])
    assert np.allclose(got, want.astype(np.float16).astype(np.float64), atol=2e-3), (got[[r for r, _ in picks]], want[[r for r, _ in picks]])
