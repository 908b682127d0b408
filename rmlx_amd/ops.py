"""Python view of the C ABI with the reference's names and argument meaning.

Used by the tests and the benchmark; a Rust host would bind the same C symbols directly.
Every function ends in a call into librmlx_hip.so -- there is no NumPy/CPU compute path here.
"""
import ctypes

import numpy as np

from . import runtime as rt
from .runtime import BF16, F16, F32, U32, DeviceBuffer, KernelError  # noqa: F401


def _h(stream):
    return stream.handle if stream is not None else None


class QuantizedWeight:
    """`QuantizedWeight` (crates/rmlx-core/src/ops/quantized.rs:78-177): three device buffers
    in MLX affine layout plus metadata; validated by the library like `QuantizedWeight::new`."""

    def __init__(self, weights_buf, scales_buf, biases_buf, group_size, bits, out_features, in_features,
                 n_experts=1):
        self.weights_buf, self.scales_buf, self.biases_buf = weights_buf, scales_buf, biases_buf
        self.group_size, self.bits = group_size, bits
        self.out_features, self.in_features, self.n_experts = out_features, in_features, n_experts
        h = ctypes.c_void_p()
        rt.check(rt.lib().rmlx_hip_qweight_create(
            weights_buf.ptr, weights_buf.nbytes, scales_buf.ptr, scales_buf.nbytes, biases_buf.ptr,
            biases_buf.nbytes, group_size, bits, out_features, in_features, n_experts, ctypes.byref(h)))
        self.handle = h.value

    @classmethod
    def from_numpy(cls, words, scales, biases, group_size, bits):
        """words u32 [N, K*bits/32] or [E, N, ...]; scales/biases f16 [.., N, K/group_size].  (3 and 6 bits: the
        rows hold whole words per group, K / group_size * (group_size // (32 // bits)) of them.)"""
        words = np.ascontiguousarray(words, np.uint32)
        scales = np.ascontiguousarray(scales, np.float16)
        e = words.shape[0] if words.ndim == 3 else 1
        n = words.shape[-2]
        k = scales.shape[-1] * group_size
        if 32 % bits != 0:
            # the constructor follows the reference's size check, ceil(N * K / (32 // bits)) words, which is more
            # than the rows of this layout occupy: pad the buffer
            need = -(-(e * n * k) // (32 // bits))
            flat = np.zeros(max(need, words.size), np.uint32)
            flat[:words.size] = words.reshape(-1)
            words = flat
        return cls(DeviceBuffer.from_numpy(words), DeviceBuffer.from_numpy(scales),
                   DeviceBuffer.from_numpy(np.ascontiguousarray(biases, np.float16)), group_size, bits, n, k, e)

    def set_expert_gemm_min_rows(self, min_rows):
        """(stacked gate weight) average rows per expert from which the expert projections of the blocks that use
        this handle run on the grouped MFMA GEMM instead of the streaming GEMV (0 = never).  Returns the previous value."""
        return int(rt.lib().rmlx_hip_qweight_set_expert_gemm_min_rows(self.handle, int(min_rows)))

    def set_expert_stream_kernel(self, kind):
        """(stacked gate weight) streaming kernel of decode-sized batches: 0 the library's choice, 1 K split over the
        waves of a workgroup, 2 / 3 a wave per weight tile with chunks of 8 / 16 rows, 4 kernel 1 for gate / up and kernel 2
        for the down projection, 5 as 4 with the gate / up projection in two launches (experts with up to 8 rows on kernel 1,
        the others on kernel 3).  Returns the previous value."""
        return int(rt.lib().rmlx_hip_qweight_set_expert_stream_kernel(self.handle, int(kind)))

    def use_gemm_layout(self, enable=True, stream=None):
        """Give the K-split MFMA GEMMs a tile-contiguous copy of the weights (a second device buffer of the same size,
        owned by this object), or drop it again.  Returns False when the weight has no such layout."""
        if not enable:
            rt.check(rt.lib().rmlx_hip_qweight_set_gemm_layout(self.handle, None, 0, _h(stream)))
            self._gemm_layout = None
            return True
        need = int(rt.lib().rmlx_hip_qweight_gemm_layout_bytes(self.handle))
        if need == 0:
            return False
        buf = DeviceBuffer((need,), rt.U8)
        rt.check(rt.lib().rmlx_hip_qweight_set_gemm_layout(self.handle, buf.ptr, buf.nbytes, _h(stream)))
        self._gemm_layout = buf
        return True

    def groups_per_row(self):
        return self.in_features // self.group_size

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                rt.lib().rmlx_hip_qweight_destroy(self.handle)
        except Exception:
            pass


def affine_quantized_matmul(qw, vec, stream=None):
    """qmv (quantized.rs:1309-1411): vec [K] -> f16 [N]."""
    out = DeviceBuffer((qw.out_features,), F16)
    a = vec.array()
    rt.check(rt.lib().rmlx_hip_affine_quantized_matmul(qw.handle, ctypes.byref(a), out.ptr, out.nbytes, _h(stream)))
    return out


def affine_quantized_matmul_batched(x, qw, stream=None, kernel=rt.KERNEL_AUTO, out=None):
    """qmm (quantized.rs:7149-7782): x [M,K] -> f16 [M,N]."""
    m = x.shape[0] if len(x.shape) == 2 else 0
    if out is None:
        out = DeviceBuffer((m, qw.out_features), F16)
    a = x.array()
    rt.check(rt.lib().rmlx_hip_qmm_select(qw.handle, ctypes.byref(a), kernel, out.ptr, out.nbytes, _h(stream)))
    return out


def qmm_add_residual(x, qw, residual, stream=None):
    """`qmm_add_residual_into_cb` (quantized.rs:8227-8340): QMM(x, qw) + residual, f16 out."""
    out = DeviceBuffer((x.shape[0] if len(x.shape) == 2 else 0, qw.out_features), F16)
    a, r = x.array(), residual.array()
    rt.check(rt.lib().rmlx_hip_qmm_add_residual(qw.handle, ctypes.byref(a), ctypes.byref(r), out.ptr, out.nbytes, _h(stream)))
    return out


def qmm_swiglu(x, qw, gate_result, stream=None):
    """`qmm_swiglu_into_cb` (quantized.rs:8345-8452): silu(gate_result) * QMM(x, qw), f16 out."""
    out = DeviceBuffer((x.shape[0] if len(x.shape) == 2 else 0, qw.out_features), F16)
    a, g = x.array(), gate_result.array()
    rt.check(rt.lib().rmlx_hip_qmm_swiglu(qw.handle, ctypes.byref(a), ctypes.byref(g), out.ptr, out.nbytes, _h(stream)))
    return out


def qmm_norm(x, qw, norm_weight, inv_rms, stream=None, out=None):
    """QMM with the RMSNorm prologue of the reference's MMA kernel (`has_norm`, quantized.rs:2955-2992, 3070-3095):
    x'[m,k] = (half(x[m,k]) * half(inv_rms[m])) * norm_weight[k]; norm_weight f16 [K], inv_rms f32 [M]; f16 out."""
    if out is None:
        out = DeviceBuffer((x.shape[0] if len(x.shape) == 2 else 0, qw.out_features), F16)
    a, w, r = x.array(), norm_weight.array(), inv_rms.array()
    rt.check(rt.lib().rmlx_hip_qmm_norm(qw.handle, ctypes.byref(a), ctypes.byref(w), ctypes.byref(r), out.ptr, out.nbytes,
                                        _h(stream)))
    return out


def qmm_encode_many(qws, x, outs, count, stream=None, kernel=rt.KERNEL_AUTO):
    """Encode `count` matmuls back to back (weights and outputs are cycled) -- see rmlx_hip_qmm_encode_many."""
    qarr = (ctypes.c_void_p * len(qws))(*[q.handle for q in qws])
    oarr = (ctypes.c_void_p * len(outs))(*[o.ptr for o in outs])
    a = x.array()
    rt.check(rt.lib().rmlx_hip_qmm_encode_many(qarr, len(qws), ctypes.byref(a), oarr, len(outs), outs[0].nbytes,
                                               count, kernel, _h(stream)))


class QuantizedLinear:
    """`QuantizedLinear` (crates/rmlx-nn/src/quantized_linear.rs:52-201) with the weights
    uploaded once at construction instead of on every forward."""

    def __init__(self, w_packed, scales, biases, in_features, out_features, group_size, bits):
        w_packed = np.ascontiguousarray(w_packed, np.uint8).reshape(-1)
        scales = np.ascontiguousarray(scales, np.float32).reshape(-1)
        biases = np.ascontiguousarray(biases, np.float32).reshape(-1)
        if group_size not in (32, 64, 128):
            raise KernelError(rt.INVALID_SHAPE, f"QuantizedLinear: group_size must be 32, 64, or 128, got {group_size}")
        if in_features == 0 or out_features == 0:
            raise KernelError(rt.INVALID_SHAPE, "QuantizedLinear: in_features and out_features must be > 0")
        if in_features % group_size != 0:
            raise KernelError(rt.INVALID_SHAPE, f"QuantizedLinear: in_features ({in_features}) must be a multiple "
                                                f"of group_size ({group_size})")
        if bits not in (4, 8):
            raise KernelError(rt.INVALID_SHAPE, f"QuantizedLinear: bits must be 4 or 8, got {bits}")
        expected = out_features * (in_features // 2) if bits == 4 else out_features * in_features
        if w_packed.size != expected:
            raise KernelError(rt.INVALID_SHAPE, f"QuantizedLinear: w_packed length ({w_packed.size}) != expected "
                                                f"({expected}) for [{out_features}, {in_features}] at {bits} bits")
        n_groups = out_features * (in_features // group_size)
        if scales.size != n_groups:
            raise KernelError(rt.INVALID_SHAPE, f"QuantizedLinear: scales length ({scales.size}) != expected ({n_groups})")
        if biases.size != n_groups:
            raise KernelError(rt.INVALID_SHAPE, f"QuantizedLinear: biases length ({biases.size}) != expected ({n_groups})")
        self.in_features, self.out_features, self.group_size, self.bits = in_features, out_features, group_size, bits
        words = w_packed.view("<u4").reshape(out_features, -1)
        self.qw = QuantizedWeight.from_numpy(words, scales.astype(np.float16).reshape(out_features, -1),
                                             biases.astype(np.float16).reshape(out_features, -1), group_size, bits)

    def forward(self, x, bias=None, stream=None):
        batch = 1 if len(x.shape) == 1 else x.shape[0]
        out = DeviceBuffer((batch, self.out_features), F16)
        a = x.array()
        rt.check(rt.lib().rmlx_hip_quantized_linear_forward(self.qw.handle, ctypes.byref(a),
                                                            bias.ptr if bias is not None else None, out.ptr,
                                                            out.nbytes, _h(stream)))
        return out


def gather_qmm(x, w_packed_buf, scales_buf, biases_buf, indices, batch, m_per_batch, n, k, n_experts, group_size,
               stream=None, out=None, kernel=0):
    """gather_qmm (quantized.rs:9404-9599): out[b] = x[b] @ dequant(W[indices[b]])^T, f16 out.  `kernel` forces a
    family (runtime.GATHER_*)."""
    if out is None:
        out = DeviceBuffer((batch, m_per_batch, n), F16)
    xa, ia = x.array(), indices.array()
    rt.check(rt.lib().rmlx_hip_gather_qmm_select(ctypes.byref(xa), w_packed_buf.ptr, w_packed_buf.nbytes, scales_buf.ptr,
                                                 scales_buf.nbytes, biases_buf.ptr, biases_buf.nbytes, ctypes.byref(ia),
                                                 batch, m_per_batch, n, k, n_experts, group_size, kernel, out.ptr,
                                                 out.nbytes, _h(stream)))
    return out


class TopkRouteResult:
    """`TopkRouteResult` (crates/rmlx-core/src/ops/topk_route.rs:396-407)."""

    def __init__(self, expert_indices, expert_weights, expert_counts, dispatch_offsets):
        self.expert_indices, self.expert_weights = expert_indices, expert_weights
        self.expert_counts, self.dispatch_offsets = expert_counts, dispatch_offsets


def gpu_topk_route(gate_logits, top_k, expert_bias=None, stream=None, renormalize=True):
    t = gate_logits.shape[0] if len(gate_logits.shape) == 2 else 0
    e = gate_logits.shape[1] if len(gate_logits.shape) == 2 else 0
    k = max(min(top_k, 8), 0)
    res = TopkRouteResult(DeviceBuffer((t * k,), U32), DeviceBuffer((t * k,), F32), DeviceBuffer((e,), U32),
                          DeviceBuffer((e + 1,), U32))
    la = gate_logits.array()
    ba = expert_bias.array() if expert_bias is not None else None
    rt.check(rt.lib().rmlx_hip_topk_route(ctypes.byref(la), top_k, ctypes.byref(ba) if ba is not None else None,
                                          1 if renormalize else 0, res.expert_indices.ptr, res.expert_weights.ptr,
                                          res.expert_counts.ptr, res.dispatch_offsets.ptr, _h(stream)))
    return res


def moe_sort(expert_indices, n_experts, stream=None):
    n = expert_indices.shape[0]
    sorted_assign, offsets = DeviceBuffer((n,), U32), DeviceBuffer((n_experts + 1,), U32)
    rt.check(rt.lib().rmlx_hip_moe_sort(expert_indices.ptr, n, n_experts, sorted_assign.ptr, offsets.ptr, _h(stream)))
    return sorted_assign, offsets


def index_gather(src, indices, stream=None):
    n, d = indices.shape[0], src.shape[1]
    dst = DeviceBuffer((n, d), F16)
    rt.check(rt.lib().rmlx_hip_index_gather(src.ptr, src.shape[0], d, indices.ptr, n, dst.ptr, _h(stream)))
    return dst


def scatter_weighted_add(src, output, tok_indices, weights, stream=None):
    rt.check(rt.lib().rmlx_hip_scatter_weighted_add(src.ptr, src.shape[0], src.shape[1], tok_indices.ptr, weights.ptr,
                                                    output.ptr, output.shape[0], _h(stream)))


def silu_gate(gate_in, up_in, stream=None):
    out = DeviceBuffer(gate_in.shape, F16)
    n = int(np.prod(gate_in.shape))
    rt.check(rt.lib().rmlx_hip_silu_gate(gate_in.ptr, up_in.ptr, out.ptr, n, _h(stream)))
    return out


def awq_dequant(qweight, qzeros, scales, rows, cols, group_size, stream=None, out=None):
    """`awq_dequant` (crates/rmlx-core/src/ops/quantized.rs:2269-2383): qweight u32 [rows, cols/8], qzeros u32
    [rows/group_size, cols/8], scales f32 [rows/group_size, cols] -> f32 [rows, cols]."""
    if out is None:
        out = DeviceBuffer((rows, cols), F32)
    rt.check(rt.lib().rmlx_hip_awq_dequant(qweight.ptr, qweight.nbytes, qzeros.ptr, qzeros.nbytes, scales.ptr,
                                           scales.nbytes, rows, cols, group_size, out.ptr, out.nbytes, _h(stream)))
    return out


def gptq_dequant(qweight, qzeros, scales, g_idx, in_features, out_features, group_size, stream=None, out=None):
    """`gptq_dequant` (crates/rmlx-core/src/ops/quantized.rs:2407-2590): qweight u32 [in/8, out], qzeros u32
    [groups, out/8], scales f32 [groups, out], g_idx (None or i32 [in], carried as its u32 bit pattern)
    -> f32 [in, out]."""
    if out is None:
        out = DeviceBuffer((in_features, out_features), F32)
    rt.check(rt.lib().rmlx_hip_gptq_dequant(qweight.ptr, qweight.nbytes, qzeros.ptr, qzeros.nbytes, scales.ptr,
                                            scales.nbytes, g_idx.ptr if g_idx is not None else None,
                                            g_idx.nbytes if g_idx is not None else 0, in_features, out_features,
                                            group_size, out.ptr, out.nbytes, _h(stream)))
    return out


class ExpertGroup:
    """`ExpertGroup` (crates/rmlx-nn/src/expert_group.rs) over stacked quantized expert weights."""

    def __init__(self, gate, up, down):
        self.gate, self.up, self.down = gate, up, down
        self.hidden_dim = gate.in_features
        self.num_experts = gate.n_experts

    def grouped_forward(self, expert_inputs, stream=None):
        """expert_inputs: list of (expert_idx, DeviceBuffer [batch_i, D]) -> list of (expert_idx, f16 ndarray)."""
        if not expert_inputs:
            return []
        for _, buf in expert_inputs:
            if len(buf.shape) != 2:
                raise KernelError(rt.INVALID_SHAPE, f"ExpertGroup: input must be 2D [batch, D], got {len(buf.shape)}D")
            if buf.shape[1] != self.hidden_dim:
                raise KernelError(rt.INVALID_SHAPE, f"ExpertGroup: input dim {buf.shape[1]} != hidden_dim {self.hidden_dim}")
        sizes = np.array([b.shape[0] for _, b in expert_inputs], np.uint32)
        idx = np.array([e for e, _ in expert_inputs], np.uint32)
        total = int(sizes.sum())
        dt = expert_inputs[0][1].dtype
        packed = DeviceBuffer((total, self.hidden_dim), dt)
        row = 0
        for (_, b), sz in zip(expert_inputs, sizes):
            rt.check(rt.lib().rmlx_hip_memcpy_d2d(packed.ptr + row * self.hidden_dim * (2 if dt != F32 else 4), b.ptr,
                                                  b.nbytes, None))
            row += int(sz)
        out = DeviceBuffer((total, self.hidden_dim), F16)
        pa = packed.array()
        rt.check(rt.lib().rmlx_hip_expert_group_grouped_forward(
            self.gate.handle, self.up.handle if self.up is not None else None, self.down.handle, len(idx),
            idx.ctypes.data, sizes.ctypes.data, ctypes.byref(pa), out.ptr, out.nbytes, _h(stream)))
        host = out.numpy()
        res, row = [], 0
        for e, sz in zip(idx, sizes):
            res.append((int(e), host[row:row + int(sz)]))
            row += int(sz)
        return res


def moe_forward_grouped(gate, up, down, x, expert_indices, expert_weights, top_k, stream=None, out=None):
    if out is None:
        out = DeviceBuffer((x.shape[0], x.shape[1]), F16)
    xa = x.array()
    rt.check(rt.lib().rmlx_hip_moe_forward_grouped(gate.handle, up.handle if up is not None else None, down.handle,
                                                   ctypes.byref(xa), expert_indices.ptr, expert_weights.ptr, top_k,
                                                   out.ptr, out.nbytes, _h(stream)))
    return out


def moe_forward(gate, up, down, x, gate_logits, top_k, expert_bias=None, stream=None, out=None, noalloc=False):
    """Routing + routed expert block.  `noalloc=True` takes the entry point that carves every intermediate from the
    library's static workspace (the caller must pass `out`: this wrapper would otherwise allocate it)."""
    if out is None:
        out = DeviceBuffer((x.shape[0], x.shape[1]), F16)
    xa, la = x.array(), gate_logits.array()
    ba = expert_bias.array() if expert_bias is not None else None
    fn = rt.lib().rmlx_hip_moe_forward_noalloc if noalloc else rt.lib().rmlx_hip_moe_forward
    rt.check(fn(gate.handle, up.handle if up is not None else None, down.handle,
                                           ctypes.byref(xa), ctypes.byref(la), top_k,
                                           ctypes.byref(ba) if ba is not None else None, out.ptr, out.nbytes,
                                           _h(stream)))
    return out
