"""Float64 NumPy model of the reference's semantics (TEST INFRASTRUCTURE ONLY).

Restates *what* the reference computes (not its kernels): MLX affine dequantisation,
dequantize-then-matmul, top-k routing, stable expert grouping, SwiGLU expert FFN and the
weighted combine.  File:line citations are relative to the reference checkout.
"""
import numpy as np

# --------------------------------------------------------------------------------------
# Packing (bit-exact)
# --------------------------------------------------------------------------------------


def pack_u32(q, bits):
    """Value i of a row sits in word i // (32/bits) at bit offset bits * (i % (32/bits)).

    Follows `word |= q << (k * bits)` (crates/rmlx-nn/src/attention.rs:4853-4862) and
    `extract_bits` (crates/rmlx-core/src/ops/quantized.rs:206-208).
    Pinned by: 0x76543210 / 0x04030201 known answers (safetensors_loader.rs:838-866), the
    0x11111111 rows (quantized.rs:12069-12095) and exhaustive per-slot round trips in tests/.
    """
    q = np.asarray(q, dtype=np.uint32)
    per = 32 // bits
    assert q.shape[-1] % per == 0
    qq = q.reshape(q.shape[:-1] + (q.shape[-1] // per, per))
    shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
    return np.bitwise_or.reduce(qq << shifts, axis=-1).astype(np.uint32)


def unpack_u32(words, bits):
    """Inverse of `pack_u32`: returns uint8 values, last axis expanded by 32/bits."""
    words = np.asarray(words, dtype=np.uint32)
    per = 32 // bits
    shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
    vals = (words[..., None] >> shifts) & np.uint32((1 << bits) - 1)
    return vals.reshape(words.shape[:-1] + (words.shape[-1] * per,)).astype(np.uint8)


def words_per_group(group_size, bits):
    """`u32s_per_group = group_size / (32 / bits)` of the reference's portable kernel `affine_qmv`
    (crates/rmlx-core/src/ops/quantized.rs:232-236), both divisions rounding down: 3 / 6 / 12 words of 10 values at
    3 bits, 6 / 12 / 25 words of 5 values at 6 bits (group sizes 32 / 64 / 128)."""
    return group_size // (32 // bits)


def pack_grouped(q, group_size, bits):
    """Row layout `affine_qmv` reads (quantized.rs:232-270): the words of group 0, then of group 1, ...; value k of word w
    of group g is element g * group_size + w * (32 / bits) + k.  Elements of a group past its last whole word get no
    word.  Equal to `pack_u32` at 2, 4 and 8 bits.  q [..., K] -> u32 [..., K / group_size * words_per_group]."""
    q = np.asarray(q, dtype=np.uint32)
    per, wpg = 32 // bits, words_per_group(group_size, bits)
    g = q.reshape(q.shape[:-1] + (q.shape[-1] // group_size, group_size))[..., : wpg * per]
    g = g.reshape(g.shape[:-1] + (wpg, per))
    shifts = np.arange(per, dtype=np.uint32) * np.uint32(bits)
    w = np.bitwise_or.reduce(g << shifts, axis=-1).astype(np.uint32)
    return w.reshape(w.shape[:-2] + (w.shape[-2] * wpg,))


def unpack_grouped(words, group_size, bits):
    """Inverse of `pack_grouped`: (values [..., K] with zeros where a group has no word, covered [K] bool)."""
    words = np.asarray(words, dtype=np.uint32)
    per, wpg = 32 // bits, words_per_group(group_size, bits)
    groups = words.shape[-1] // wpg
    vals = unpack_u32(words, bits).reshape(words.shape[:-1] + (groups, wpg * per))
    q = np.zeros(words.shape[:-1] + (groups, group_size), np.uint8)
    q[..., : wpg * per] = vals
    covered = np.zeros((groups, group_size), bool)
    covered[:, : wpg * per] = True
    return q.reshape(words.shape[:-1] + (groups * group_size,)), covered.reshape(-1)


def words_to_bytes(words):
    """Byte image the reference's CPU path consumes: for Q4 low nibble = even k, for Q8 one
    byte per value; equal to the little-endian bytes of the u32 words
    (crates/rmlx-nn/src/safetensors_loader.rs:562-628)."""
    w = np.ascontiguousarray(words, dtype="<u4")
    return w.view(np.uint8).reshape(w.shape[:-1] + (w.shape[-1] * 4,))


def bytes_to_words(b):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    return b.view("<u4").reshape(b.shape[:-1] + (b.shape[-1] // 4,))


# --------------------------------------------------------------------------------------
# bf16 helpers (NumPy has no bfloat16)
# --------------------------------------------------------------------------------------


def f32_to_bf16_bits(x):
    """Round-to-nearest-even f32 -> bf16 bit pattern (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


# --------------------------------------------------------------------------------------
# Dequantize-then-matmul (tolerance oracle)
# --------------------------------------------------------------------------------------


def dequantize(words, scales, biases, group_size, bits):
    """w[n,k] = scale[n,k//gs] * q[n,k] + bias[n,k//gs], evaluated exactly in float64.

    Semantics of `dequantize_q4_row` (crates/rmlx-core/src/ops/quantized.rs:2602-2622) and of
    the QuantizedWeight doc (`w_i = scale_g * q_i + bias_g`, :69-77).  Pinned by the
    [3,5,10,1] -> [6.5,10.5,20.5,2.5] known answer (:10601-10624) and by agreement with the C
    restatement of `dequantize_q4_row`.
    """
    s = np.repeat(np.asarray(scales, dtype=np.float64), group_size, axis=-1)
    b = np.repeat(np.asarray(biases, dtype=np.float64), group_size, axis=-1)
    if 32 % bits != 0:
        # 3 and 6 bits, layout and coverage of `affine_qmv` (quantized.rs:232-270, the only kernel of the reference
        # that takes them): an element without a word adds nothing to `scale * sum(q x) + bias * sum(x)`, i.e. its
        # weight is 0.  No test or fixture of the reference holds such a weight; pinned in tests/ by a loop-for-loop
        # restatement of the kernel on small shapes and by the closed forms its coverage fixes.
        q, covered = unpack_grouped(words, group_size, bits)
        return np.where(covered, s * q.astype(np.float64) + b, 0.0)
    q = unpack_u32(words, bits).astype(np.float64)
    return s * q + b


def qmm(x, words, scales, biases, group_size, bits):
    """out[m,n] = sum_k x[m,k] * dequant(W)[n,k] in float64 (the reference's
    `naive_matmul_with_dequant`, quantized.rs:10681-10719, with exact arithmetic).
    Pinned by: equal-nibble closed forms 224/96/192/448/512 (:10922, :11575, :11784, :12088),
    agreement with the C restatement of `affine_qmm` (1e-4 relative, the bar the reference
    itself uses at :10794-10808)."""
    w = dequantize(words, scales, biases, group_size, bits)
    return np.asarray(x, dtype=np.float64) @ w.T


def norm_rows(x, inv_rms, norm_weight):
    """x'[m,k] = (half(x[m,k]) * half(inv_rms[m])) * norm_weight[k], each product rounded to f16: the A loader of
    the reference's Q4 MMA kernel under `has_norm` (crates/rmlx-core/src/ops/quantized.rs:3070-3095).  No host
    entry point or test of the reference exercises it; pinned in tests/ by what the formula fixes (unit
    inv_rms and norm_weight leave x unchanged bit for bit, powers of two scale exactly, the result equals
    qmm of the separately normalised rows) -- numpy's float16 product is the IEEE round-to-nearest-even one."""
    xh = np.asarray(x).astype(np.float16)
    rs = np.asarray(inv_rms, dtype=np.float32).astype(np.float16)[:, None]
    return ((xh * rs).astype(np.float16) * np.asarray(norm_weight, dtype=np.float16)[None, :]).astype(np.float16)


def gather_qmm(x, words, scales, biases, indices, group_size, bits=4):
    """out[b] = x[b] @ dequant(W[indices[b]])^T for stacked expert weights [E,N,K*bits/32]
    (crates/rmlx-core/src/ops/quantized.rs:9279-9290, 9300-9368).  x is [batch, M_b, K] or
    [batch, K]."""
    x = np.asarray(x, dtype=np.float64)
    outs = []
    for b, e in enumerate(np.asarray(indices)):
        outs.append(qmm(np.atleast_2d(x[b]), words[e], scales[e], biases[e], group_size, bits))
    out = np.stack(outs) if outs else np.zeros((0, 1, words.shape[1]))
    return out if x.ndim == 3 else out[:, 0, :]


def tolerance(ref):
    """The acceptance bar: max|err| <= 1e-2 * RMS(reference output)."""
    ref = np.asarray(ref, dtype=np.float64)
    return 1e-2 * float(np.sqrt(np.mean(ref * ref)))


# --------------------------------------------------------------------------------------
# Routing
# --------------------------------------------------------------------------------------


def exp_neg_exact(x):
    """exp(x) for x <= 0 as a fixed sequence of f32 multiplies and adds, each rounded once: Cody-Waite reduction
    x = n ln2 + r, the degree-5 polynomial of Cephes' expf for (e^r - 1 - r) / r^2, scaling by 2^n; arguments
    below -80 give 0.  The reference evaluates Metal's `fast::exp` here (topk_route.rs:256-257, 294), whose bits
    no other machine reproduces; this routine is a definition both the library's routing kernel and this model
    follow operation by operation, so they see the same ties.  Pinned in tests/ against float64 `exp` (a few
    ulp) and by exact powers of two at multiples of ln 2 being monotone."""
    x = np.asarray(x, dtype=np.float32)
    f = np.float32
    with np.errstate(invalid="ignore", over="ignore"):
        n = np.rint(x * f(1.44269504))
        r = x - n * f(0.693359375)
        r = r - n * f(-2.12194440e-4)
        p = np.full(x.shape, f(1.9875691500e-4), np.float32)
        for c in (1.3981999507e-3, 8.3334519073e-3, 4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1):
            p = p * r + f(c)
        p = p * (r * r)
        p = p + r
        p = p + f(1.0)
        ni = np.where(np.isfinite(n) & (n >= -126), n, 0).astype(np.int64)
        two_n = ((ni + 127).astype(np.uint32) << np.uint32(23)).view(np.float32)
        out = (p * two_n).astype(np.float32)
    return np.where(x < f(-80.0), f(0.0), out).astype(np.float32)


def _pairwise_sum_f32(v):
    """Balanced pairwise tree over a power-of-two number of f32 values: ((v0+v1)+(v2+v3))+..."""
    v = np.asarray(v, dtype=np.float32)
    while v.size > 1:
        v = (v[0::2] + v[1::2]).astype(np.float32)
    return np.float32(v[0])


def topk_route(logits, top_k, bias=None, renormalize=True, rank_by="softmax"):
    """softmax over E -> top-k by repeated argmax (strict >, ties -> lowest index) ->
    weights / sum(top-k) -> histogram -> exclusive scan.

    Restates `moe_topk_route_f32` + `moe_prefix_scan_u32`
    (crates/rmlx-core/src/ops/topk_route.rs:212-388).  Softmax is evaluated in f32 like the
    kernel: `exp(l - max) * (1 / sum)` (:294), the experts ranked by that f32 value with strict `>`
    over ascending index and selected ones skipped (:283-300), so equal values -- an underflowing
    tail, two logits that collapse after exp -- go to the lower index.  `exp` is `exp_neg_exact`;
    the sum adds experts j, j+64, j+128, j+192 in that order for j = 0..63 and then the 64 partial
    sums as a balanced pairwise tree (the reference's order is its threadgroup reduction, which
    its tests do not pin).  `rank_by="logit"` ranks the (biased) logits instead: the same order
    wherever the softmax values are distinct.
    Pinned in tests/ by the reference's behavioural tests (:674-751, :764-783, :815-840), a
    brute-force stable argsort, hand-written picks on underflowing rows, and the weights against
    float64 softmax closed forms (renormalised top-k weights = softmax over the selected logits).
    Returns (indices u32 [T*K], weights f32 [T*K], counts u32 [E], offsets u32 [E+1]).
    """
    lg = np.asarray(logits, dtype=np.float32)
    T, E = lg.shape
    if bias is not None:
        lg = (lg + np.asarray(bias, dtype=np.float32)[None, :]).astype(np.float32)
    idx = np.zeros((T, top_k), np.uint32)
    wts = np.zeros((T, top_k), np.float32)
    for t in range(T):
        row = lg[t]
        mx = np.float32(row.max()) if E else np.float32(0)
        ex = exp_neg_exact((row - mx).astype(np.float32))
        lanes = np.zeros((4, 64), np.float32)
        lanes.reshape(-1)[:E] = ex
        part = np.zeros(64, np.float32)
        for j in range(4):
            part = (part + lanes[j]).astype(np.float32)
        inv = np.float32(1.0) / _pairwise_sum_f32(part)
        sm = (ex * inv).astype(np.float32)
        key = sm if rank_by == "softmax" else row
        taken = np.zeros(E, bool)
        for k in range(top_k):
            best, best_i = None, 0
            for i in range(E):
                if taken[i]:
                    continue
                if best is None or key[i] > best:
                    best, best_i = key[i], i
            taken[best_i] = True
            idx[t, k] = best_i
            wts[t, k] = sm[best_i]
        if renormalize:
            ssum = np.float32(0)
            for k in range(top_k):
                ssum = np.float32(ssum + wts[t, k])
            invw = np.float32(1.0) / ssum if ssum > 0 else np.float32(0)
            wts[t] = (wts[t] * invw).astype(np.float32)
    counts = np.bincount(idx.reshape(-1), minlength=E).astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    return idx.reshape(-1), wts.reshape(-1), counts, offsets


def expert_dispatch(indices, weights, seq_len, top_k, num_experts):
    """`expert_dispatch[e] = [(tok, w), ...]` in (tok, k) order
    (crates/rmlx-nn/src/moe.rs:1439-1447), as plain loops."""
    disp = [[] for _ in range(num_experts)]
    for tok in range(seq_len):
        for k in range(top_k):
            flat = tok * top_k + k
            disp[int(indices[flat])].append((tok, float(weights[flat])))
    return disp


def moe_sort(indices, num_experts):
    """Stable sort of flat assignment ids (tok*K+k) by expert id.  Returns
    (sorted_assign u32 [A], offsets u32 [E+1]); segment e of sorted_assign lists the flat
    ids routed to expert e in ascending order -- the same order `expert_dispatch` produces."""
    indices = np.asarray(indices, dtype=np.uint32)
    order = np.argsort(indices, kind="stable").astype(np.uint32)
    counts = np.bincount(indices, minlength=num_experts).astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    return order, offsets


# --------------------------------------------------------------------------------------
# Expert FFN + combine
# --------------------------------------------------------------------------------------


def silu(x):
    x = np.asarray(x, dtype=np.float64)
    return x / (1.0 + np.exp(-x))


def scatter_weighted_add(src, tok_indices, weights, num_tokens):
    """out[tok_indices[a], :] += weights[a] * src[a, :] over the assignments a in ascending order, out zero-initialised
    (`scatter_weighted_add`, crates/rmlx-core/src/ops/moe_kernels.rs:306-363; the reference accumulates in the
    array dtype, this model in float64).  Pinned by the reference's known answer (:420-450)."""
    src = np.asarray(src, dtype=np.float64)
    out = np.zeros((num_tokens, src.shape[1]), np.float64)
    for a in range(src.shape[0]):
        out[int(tok_indices[a])] += float(weights[a]) * src[a]
    return out


def combine_cpu(expert_outputs, weights, indices, batch_size, top_k, hidden_dim):
    """out[t, :] = sum_k weights[t*K+k] * expert_outputs[indices[t*K+k]][t, :] with out-of-range experts skipped
    (`MoeCombineExchange::combine_cpu`, crates/rmlx-distributed/src/moe_exchange.rs:2288-2320).  Pinned by the
    reference's known answers (crates/rmlx-distributed/tests/moe_tests.rs:115-135, 660-687)."""
    out = np.zeros((batch_size, hidden_dim), np.float64)
    for t in range(batch_size):
        for k in range(top_k):
            flat = t * top_k + k
            e = int(indices[flat])
            if e < len(expert_outputs):
                eo = np.asarray(expert_outputs[e], dtype=np.float64).reshape(-1)
                if (t + 1) * hidden_dim <= eo.size:
                    out[t] += float(weights[flat]) * eo[t * hidden_dim:(t + 1) * hidden_dim]
    return out


def expert_ffn(x, gate_w, up_w, down_w, round_h=np.float16):
    """y = (silu(x Wg^T) * (x Wu^T)) Wd^T for dequantised [out, in] weight matrices: `Expert::forward`
    (crates/rmlx-nn/src/moe.rs:188-200) / the per-expert body of `ExpertGroup::grouped_forward`
    (crates/rmlx-nn/src/expert_group.rs:445-524).  The hidden activation is rounded to `round_h` (the reference
    stores it in the input dtype, expert_group.rs:380-383); everything else is float64."""
    x = np.asarray(x, dtype=np.float64)
    h = silu(x @ gate_w.T) * (x @ up_w.T)
    if round_h is not None:
        h = h.astype(round_h).astype(np.float64)
    return h @ down_w.T


def moe_forward(x, indices, weights, gate, up, down, group_size, top_k, round_h=np.float16, bits=4):
    """out[t] = sum_k w[t,k] * down_e( silu(gate_e x_t) * up_e x_t ), e = indices[t,k].

    Composition of `ExpertGroup::grouped_forward` (crates/rmlx-nn/src/expert_group.rs:445-524:
    gate GEMM, up GEMM, silu_gate, down GEMM) and the weighted scatter-add
    (crates/rmlx-nn/src/moe.rs:1851-1932; `scatter_weighted_add`,
    crates/rmlx-core/src/ops/moe_kernels.rs:306-363), with expert weights in the stacked Q4
    layout of `gather_qmv_fast_f16_q4` (quantized.rs:9605-9620).  `gate`, `up`, `down` are
    (words, scales, biases) triples with a leading expert axis.  Assignments are grouped by expert
    in (token, k) order (`moe_sort`), every group runs `expert_ffn`, and the rows go back through
    `scatter_weighted_add` with the token of each sorted position.
    Pinned in tests/: the combine step by the reference's known answers for `scatter_weighted_add`
    and `combine_cpu`; the whole function by a brute per-(token, k) loop that dequantises with the C
    restatement of `dequantize_q4_row` and shares no code with this one, on small shapes with
    top_k > 1 and repeated experts, and by one-hot / identity closed forms.
    """
    x = np.asarray(x, dtype=np.float64)
    T, D = x.shape
    idx = np.asarray(indices).reshape(-1)
    wts = np.asarray(weights, dtype=np.float64).reshape(-1)
    E = gate[0].shape[0]
    order, offsets = moe_sort(idx, E)
    tok = order // top_k
    y = np.zeros((order.size, D), np.float64)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if lo == hi:
            continue
        wg, wu, wd = (dequantize(t[0][e], t[1][e], t[2][e], group_size, bits) for t in (gate, up, down))
        y[lo:hi] = expert_ffn(x[tok[lo:hi]], wg, wu, wd, round_h)
    return scatter_weighted_add(y, tok, wts[order], T)


# --------------------------------------------------------------------------------------
# AWQ / GPTQ INT4 dequantisation (float32, bit-exact: one subtraction of small integers and
# one multiplication per element)
# --------------------------------------------------------------------------------------


def awq_dequant(qweight, qzeros, scales, group_size):
    """out[r, c] = scales[g, c] * (nibble(qweight[r, c/8], c%8) - nibble(qzeros[g, c/8], c%8)), g = r / group_size.

    Follows `awq_dequant_f32` (crates/rmlx-core/src/ops/quantized.rs:707-733): packing along the
    columns.  The reference holds no test or vector for it; pinned in tests/ by hand-computed words
    (0x76543210 against zero word 0x11111111), by agreement with `gptq_dequant` on one logical matrix
    packed both ways (the two index paths share nothing but `unpack_u32`, itself pinned above), and
    by an element-at-a-time walk of the kernel's index arithmetic on small shapes.
    """
    qweight = np.asarray(qweight, dtype=np.uint32)
    rows = qweight.shape[0]
    nib = unpack_u32(qweight, 4).astype(np.float32)
    zero = unpack_u32(np.asarray(qzeros, dtype=np.uint32), 4).astype(np.float32)
    g = np.arange(rows) // group_size
    return (np.asarray(scales, dtype=np.float32)[g] * (nib - zero[g])).astype(np.float32)


def gptq_dequant(qweight, qzeros, scales, g_idx, group_size):
    """out[r, c] = scales[g, c] * (nibble(qweight[r/8, c], r%8) - (nibble(qzeros[g, c/8], c%8) + 1)),
    g = g_idx[r] if given else r / group_size.

    Follows `gptq_dequant_f32` (crates/rmlx-core/src/ops/quantized.rs:749-783): packing along the rows
    and the zero point stored minus one.  Rows whose g_idx is outside [0, groups) give zeros (the
    reference reads out of bounds there; the library defines the result instead).  Pinned as
    `awq_dequant`, plus: identity g_idx == no g_idx, and a permuted g_idx against the logical matrices.
    """
    qweight = np.asarray(qweight, dtype=np.uint32)
    packed_rows, n = qweight.shape
    k = packed_rows * 8
    shifts = (np.arange(8, dtype=np.uint32) * np.uint32(4))[None, :, None]
    nib = ((qweight[:, None, :] >> shifts) & np.uint32(15)).reshape(k, n).astype(np.float32)
    zero = (unpack_u32(np.asarray(qzeros, dtype=np.uint32), 4).astype(np.float32) + np.float32(1))
    scales = np.asarray(scales, dtype=np.float32)
    groups = scales.shape[0]
    if g_idx is None:
        g = np.arange(k, dtype=np.int64) // group_size
    else:
        g = np.asarray(g_idx).astype(np.int32).view(np.uint32).astype(np.int64)  # the kernel's uint(g_idx[row])
    valid = g < groups
    gc = np.where(valid, g, 0)
    out = scales[gc] * (nib - zero[gc])
    out[~valid] = 0
    return out.astype(np.float32)
