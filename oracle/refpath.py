"""ctypes bindings of `affine_qmm_ref.c` (TEST INFRASTRUCTURE ONLY, see package docstring).

Each wrapper takes/returns NumPy arrays and forwards to the C restatement; the citation of
the reference lines lives next to each C function.
"""
import ctypes
import os
import subprocess
import threading

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile the C restatement with gcc (`-O2 -ffp-contract=off`)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "affine_qmm_ref.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        sz, vp = ctypes.c_size_t, ctypes.c_void_p
        L.oracle_affine_qmm.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, vp]
        L.oracle_affine_qmm_q8.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, vp]
        L.oracle_affine_qmm_cols.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, ctypes.c_int, sz, sz, vp]
        L.oracle_naive_matmul_with_dequant.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, ctypes.c_int, vp]
        L.oracle_dequantize_q4_row.argtypes = [vp, vp, vp, sz, sz, vp]
        L.oracle_dequant_q4_nibble.argtypes = [ctypes.c_uint8, ctypes.c_uint32]
        L.oracle_dequant_q4_nibble.restype = ctypes.c_uint8
        L.oracle_f32_to_f16_bits.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16_bits.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_f16_bits_array.argtypes = [vp, vp, sz]
        L.oracle_f16_to_f32_array.argtypes = [vp, vp, sz]
        L.oracle_lcg_fill.argtypes = [vp, vp, sz]
        L.oracle_quantize_row.argtypes = [vp, sz, sz, ctypes.c_int, vp, vp, vp]
        L.oracle_repack_mlx_weight.argtypes = [vp, sz, ctypes.c_int, vp]
        L.oracle_pack_u32.argtypes = [vp, sz, ctypes.c_int, vp]
        L.oracle_extract_bits.argtypes = [ctypes.c_uint32] * 3
        L.oracle_extract_bits.restype = ctypes.c_uint32
        L.oracle_cpu_qmv_q4_reference.argtypes = [vp, vp, vp, vp, sz, sz, sz, vp]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def dequant_q4_nibble(byte, nibble_idx):
    return int(lib().oracle_dequant_q4_nibble(byte, nibble_idx))


def extract_bits(word, idx_in_word, bits):
    return int(lib().oracle_extract_bits(word, idx_in_word, bits))


def dequantize_q4_row(w_packed, scales, biases, k, group_size):
    w, s, b = _c(w_packed, np.uint8), _c(scales, np.float32), _c(biases, np.float32)
    out = np.empty(k, np.float32)
    lib().oracle_dequantize_q4_row(_p(w), _p(s), _p(b), k, group_size, _p(out))
    return out


def affine_qmm(x, w_packed, scales, biases, m, n, k, group_size, bits=4):
    """`affine_qmm` (bits=4, bytes [N,K/2]) / `affine_qmm_q8` (bits=8, bytes [N,K]); f32 in/out."""
    x, w = _c(x, np.float32), _c(w_packed, np.uint8)
    s, b = _c(scales, np.float32), _c(biases, np.float32)
    assert x.size == m * k and s.size == n * (k // group_size) == b.size
    assert w.size == (n * k // 2 if bits == 4 else n * k)
    out = np.empty((m, n), np.float32)
    fn = lib().oracle_affine_qmm if bits == 4 else lib().oracle_affine_qmm_q8
    fn(_p(x), _p(w), _p(s), _p(b), m, n, k, group_size, _p(out))
    return out


def affine_qmm_threads(x, w_packed, scales, biases, m, n, k, group_size, bits=4, threads=1):
    """Same scalar loop nest, output columns partitioned over `threads` host threads."""
    x, w = _c(x, np.float32), _c(w_packed, np.uint8)
    s, b = _c(scales, np.float32), _c(biases, np.float32)
    out = np.empty((m, n), np.float32)
    per = -(-n // threads)
    per = -(-per // 4) * 4
    ranges = [(c, min(n, c + per)) for c in range(0, n, per)]

    def run(c0, c1):
        lib().oracle_affine_qmm_cols(_p(x), _p(w), _p(s), _p(b), m, n, k, group_size, bits, c0, c1, _p(out))

    ts = [threading.Thread(target=run, args=r) for r in ranges]
    [t.start() for t in ts]
    [t.join() for t in ts]
    return out


def naive_matmul_with_dequant(x, w_packed, scales, biases, m, n, k, group_size, bits=4):
    x, w = _c(x, np.float32), _c(w_packed, np.uint8)
    s, b = _c(scales, np.float32), _c(biases, np.float32)
    out = np.empty((m, n), np.float32)
    lib().oracle_naive_matmul_with_dequant(_p(x), _p(w), _p(s), _p(b), m, n, k, group_size, bits, _p(out))
    return out


def cpu_qmv_q4_reference(weights_u32, scales, biases, x, n, k, group_size):
    w, s, b, x = _c(weights_u32, np.uint32), _c(scales, np.float32), _c(biases, np.float32), _c(x, np.float32)
    out = np.empty(n, np.float32)
    lib().oracle_cpu_qmv_q4_reference(_p(w), _p(s), _p(b), _p(x), n, k, group_size, _p(out))
    return out


def f32_to_f16_bits(v):
    v = _c(v, np.float32)
    out = np.empty(v.shape, np.uint16)
    lib().oracle_f32_to_f16_bits_array(_p(v), _p(out), v.size)
    return out


def f16_to_f32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().oracle_f16_to_f32_array(_p(bits), _p(out), bits.size)
    return out


class Lcg:
    """The reference tests' PRNG (state update s*6364136223846793005+1, top 31 bits -> [-1,1))."""

    def __init__(self, seed):
        self.state = ctypes.c_uint64(seed)

    def fill(self, n):
        out = np.empty(n, np.float32)
        lib().oracle_lcg_fill(ctypes.byref(self.state), _p(out), n)
        return out


def quantize_rows(weights_f32, group_size, bits):
    """Row-wise `quantize_q4_row` / `quantize_q8_row`: returns (bytes [N,K/2|K], scales, biases)."""
    w = _c(weights_f32, np.float32)
    n, k = w.shape
    packed = np.zeros((n, k // 2 if bits == 4 else k), np.uint8)
    scales = np.empty((n, k // group_size), np.float32)
    biases = np.empty((n, k // group_size), np.float32)
    for j in range(n):
        lib().oracle_quantize_row(_p(w[j]), k, group_size, bits, _p(packed[j]), _p(scales[j]), _p(biases[j]))
    return packed, scales, biases


def repack_mlx_weight(words_u32, bits):
    w = _c(words_u32, np.uint32)
    out = np.empty(w.size * 4, np.uint8)
    lib().oracle_repack_mlx_weight(_p(w), w.size, bits, _p(out))
    return out


def pack_u32(q_values, bits):
    q = _c(q_values, np.uint8)
    per = 32 // bits
    out = np.empty(q.size // per, np.uint32)
    lib().oracle_pack_u32(_p(q), q.size, bits, _p(out))
    return out
