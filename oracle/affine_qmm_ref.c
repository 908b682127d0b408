/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's scalar CPU path.
 *
 * This file is the checker (and the timed "cpu_baseline" leg of bench.py); it is never
 * linked into, loaded by or called from the shipped library.  Build with
 *   gcc -O2 -ffp-contract=off -fPIC -shared   (no FMA contraction: plain IEEE f32)
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout).  The reference is a Rust crate that cannot be built in this
 * image (no rustc/cargo, hard dependency on objc2-metal), so parity of this file is
 * pinned by the reference's own known-answer tests re-run against it from tests/ and
 * by closed forms / a float64 model, not by linking the original.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>

/* crates/rmlx-core/src/ops/quantized.rs:2586-2592 -- low nibble = even column. */
static inline uint8_t dequant_q4_nibble(uint8_t packed_byte, size_t nibble_idx) {
    return nibble_idx == 0 ? (uint8_t)(packed_byte & 0x0F) : (uint8_t)((packed_byte >> 4) & 0x0F);
}

uint8_t oracle_dequant_q4_nibble(uint8_t packed_byte, uint32_t nibble_idx) {
    return dequant_q4_nibble(packed_byte, nibble_idx);
}

/* crates/rmlx-core/src/ops/quantized.rs:2602-2622 */
void oracle_dequantize_q4_row(const uint8_t* w_packed, const float* scales, const float* biases,
                              size_t k, size_t group_size, float* out) {
    for (size_t col = 0; col < k; ++col) {
        float q = (float)dequant_q4_nibble(w_packed[col / 2], col % 2);
        size_t group = col / group_size;
        out[col] = scales[group] * q + biases[group];
    }
}

/* crates/rmlx-core/src/ops/quantized.rs:2649-2741 -- same 4x4 tiling, same loop nest,
 * same accumulation order: out[i,j] += scale*dot + bias*xsum once per group. */
void oracle_affine_qmm(const float* x, const uint8_t* w_packed, const float* scales,
                       const float* biases, size_t m, size_t n, size_t k, size_t group_size,
                       float* output) {
    const size_t TILE_M = 4, TILE_N = 4;
    const size_t groups_per_row = k / group_size;
    for (size_t i = 0; i < m * n; ++i) output[i] = 0.0f;
    for (size_t row = 0; row < m; row += TILE_M) {
        size_t rm = (m - row < TILE_M) ? m - row : TILE_M;
        for (size_t col = 0; col < n; col += TILE_N) {
            size_t rn = (n - col < TILE_N) ? n - col : TILE_N;
            for (size_t g = 0; g < groups_per_row; ++g) {
                size_t k_start = g * group_size, k_end = k_start + group_size;
                for (size_t jj = 0; jj < rn; ++jj) {
                    size_t j = col + jj;
                    float scale = scales[j * groups_per_row + g];
                    float bias = biases[j * groups_per_row + g];
                    const uint8_t* w_row = w_packed + j * (k / 2);
                    for (size_t ii = 0; ii < rm; ++ii) {
                        size_t i = row + ii;
                        const float* x_row = x + i * k;
                        float dot = 0.0f, xsum = 0.0f;
                        for (size_t kk = k_start; kk < k_end; ++kk) {
                            float q = (float)dequant_q4_nibble(w_row[kk / 2], kk % 2);
                            float xv = x_row[kk];
                            dot += q * xv;
                            xsum += xv;
                        }
                        output[i * n + j] += scale * dot + bias * xsum;
                    }
                }
            }
        }
    }
}

/* crates/rmlx-core/src/ops/quantized.rs:2755-2836 -- byte weights [N,K]. */
void oracle_affine_qmm_q8(const float* x, const uint8_t* w_packed, const float* scales,
                          const float* biases, size_t m, size_t n, size_t k, size_t group_size,
                          float* output) {
    const size_t TILE_M = 4, TILE_N = 4;
    const size_t groups_per_row = k / group_size;
    for (size_t i = 0; i < m * n; ++i) output[i] = 0.0f;
    for (size_t row = 0; row < m; row += TILE_M) {
        size_t rm = (m - row < TILE_M) ? m - row : TILE_M;
        for (size_t col = 0; col < n; col += TILE_N) {
            size_t rn = (n - col < TILE_N) ? n - col : TILE_N;
            for (size_t g = 0; g < groups_per_row; ++g) {
                size_t k_start = g * group_size, k_end = k_start + group_size;
                for (size_t jj = 0; jj < rn; ++jj) {
                    size_t j = col + jj;
                    float scale = scales[j * groups_per_row + g];
                    float bias = biases[j * groups_per_row + g];
                    const uint8_t* w_row = w_packed + j * k;
                    for (size_t ii = 0; ii < rm; ++ii) {
                        size_t i = row + ii;
                        const float* x_row = x + i * k;
                        float dot = 0.0f, xsum = 0.0f;
                        for (size_t kk = k_start; kk < k_end; ++kk) {
                            float q = (float)w_row[kk];
                            float xv = x_row[kk];
                            dot += q * xv;
                            xsum += xv;
                        }
                        output[i * n + j] += scale * dot + bias * xsum;
                    }
                }
            }
        }
    }
}

/* crates/rmlx-core/src/ops/quantized.rs:10681-10719 (Q4) and :11640-11669 (Q8):
 * the test-side "naive" dequantize-then-matmul, f32, k-ascending accumulation. */
void oracle_naive_matmul_with_dequant(const float* x, const uint8_t* w_packed, const float* scales,
                                      const float* biases, size_t m, size_t n, size_t k,
                                      size_t group_size, int bits, float* output) {
    size_t gpr = k / group_size;
    for (size_t j = 0; j < n; ++j) {
        for (size_t i = 0; i < m; ++i) {
            float dot = 0.0f;
            for (size_t kk = 0; kk < k; ++kk) {
                float q = bits == 4 ? (float)dequant_q4_nibble(w_packed[j * (k / 2) + kk / 2], kk % 2)
                                    : (float)w_packed[j * k + kk];
                float w = scales[j * gpr + kk / group_size] * q + biases[j * gpr + kk / group_size];
                if (bits == 4) dot += x[i * k + kk] * w;  /* :10712 x*w */
                else dot += x[i * k + kk] * w;             /* :11662 x*w */
            }
            output[i * n + j] = dot;
        }
    }
}

/* crates/rmlx-core/src/ops/quantized.rs:8464-8515 -- f32 -> f16 bits, RNE, quiet NaN 0x7E00. */
uint16_t oracle_f32_to_f16_bits(float val) {
    uint32_t bits;
    memcpy(&bits, &val, 4);
    uint32_t sign = (bits >> 16) & 0x8000u;
    int32_t exponent = (int32_t)((bits >> 23) & 0xFF);
    uint32_t mantissa = bits & 0x007FFFFFu;
    if (exponent == 0xFF) return (uint16_t)(mantissa == 0 ? (sign | 0x7C00u) : (sign | 0x7E00u));
    int32_t new_exp = exponent - 127 + 15;
    if (new_exp >= 31) return (uint16_t)(sign | 0x7C00u);
    if (new_exp <= 0) {
        if (new_exp < -10) return (uint16_t)sign;
        uint32_t shift = (uint32_t)(1 - new_exp);
        uint32_t mm = (mantissa | 0x00800000u) >> (13 + shift);
        uint32_t round_bit = 1u << (12 + shift);
        uint32_t remainder = (mantissa | 0x00800000u) & ((round_bit << 1) - 1);
        if (remainder > round_bit || (remainder == round_bit && (mm & 1))) return (uint16_t)(sign | (mm + 1));
        return (uint16_t)(sign | mm);
    }
    uint32_t mm = mantissa >> 13;
    uint32_t round_bit = 1u << 12;
    uint32_t remainder = mantissa & ((round_bit << 1) - 1);
    uint32_t half_val = sign | ((uint32_t)new_exp << 10) | mm;
    if (remainder > round_bit || (remainder == round_bit && (mm & 1))) return (uint16_t)(half_val + 1);
    return (uint16_t)half_val;
}

/* crates/rmlx-nn/src/quantized_linear.rs:304-336 -- exact f16 bits -> f32. */
float oracle_f16_to_f32(uint16_t bits) {
    uint32_t sign = (bits >> 15) & 1u, exp = (bits >> 10) & 0x1Fu, mant = bits & 0x3FFu, out;
    if (exp == 0) {
        if (mant == 0) out = sign << 31;
        else {
            uint32_t mm = mant; int32_t e = 0;
            while ((mm & 0x400u) == 0) { mm <<= 1; e -= 1; }
            mm &= 0x3FFu;
            out = (sign << 31) | ((uint32_t)(127 - 15 + 1 + e) << 23) | (mm << 13);
        }
    } else if (exp == 31) out = (sign << 31) | (0xFFu << 23) | (mant << 13);
    else out = (sign << 31) | ((exp - 15 + 127) << 23) | (mant << 13);
    float f; memcpy(&f, &out, 4); return f;
}

void oracle_f32_to_f16_bits_array(const float* in, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = oracle_f32_to_f16_bits(in[i]);
}
void oracle_f16_to_f32_array(const uint16_t* in, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = oracle_f16_to_f32(in[i]);
}

/* Test PRNG of the reference: crates/rmlx-core/src/ops/quantized.rs:10743-10747.
 * seed = seed*6364136223846793005 + 1 (wrapping u64); v = ((seed>>33) as f32 / 2^31) - 1.
 * `u32::MAX as f32 / 2.0` is exactly 2^31; the u64->f32 cast rounds to nearest even. */
void oracle_lcg_fill(uint64_t* seed, float* out, size_t n) {
    uint64_t s = *seed;
    for (size_t i = 0; i < n; ++i) {
        s = s * 6364136223846793005ULL + 1ULL;
        out[i] = ((float)(s >> 33) / 2147483648.0f) - 1.0f;
    }
    *seed = s;
}

/* Rust f32::round = half away from zero; C roundf has the same definition. */
/* crates/rmlx-core/src/ops/quantized.rs:10638-10676 (bits=4, byte packing lo|hi<<4)
 * and :11605-11636 (bits=8, one byte per value). */
void oracle_quantize_row(const float* weights, size_t k, size_t group_size, int bits,
                         uint8_t* packed, float* scales, float* biases) {
    float maxq = bits == 4 ? 15.0f : 255.0f;
    size_t num_groups = k / group_size;
    if (bits == 4) memset(packed, 0, k / 2);
    for (size_t g = 0; g < num_groups; ++g) {
        size_t start = g * group_size;
        float mn = INFINITY, mx = -INFINITY;
        for (size_t i = 0; i < group_size; ++i) {
            float w = weights[start + i];
            mn = fminf(mn, w); mx = fmaxf(mx, w);
        }
        float range = mx - mn;
        float scale = range < 1e-10f ? 1.0f : range / maxq;
        float bias = mn;
        scales[g] = scale; biases[g] = bias;
        for (size_t i = 0; i < group_size; ++i) {
            float r = roundf((weights[start + i] - bias) / scale);
            if (r < 0.0f) r = 0.0f;
            if (r > maxq) r = maxq;
            uint8_t q = (uint8_t)r;
            size_t col = start + i;
            if (bits == 4) {
                if (col % 2 == 0) packed[col / 2] = q; else packed[col / 2] |= (uint8_t)(q << 4);
            } else packed[col] = q;
        }
    }
}

/* crates/rmlx-nn/src/safetensors_loader.rs:562-628 -- MLX u32 words -> byte stream.
 * For both widths the result equals the little-endian byte image of the words. */
void oracle_repack_mlx_weight(const uint32_t* words, size_t num_u32, int bits, uint8_t* packed) {
    for (size_t i = 0; i < num_u32; ++i) {
        uint32_t word = words[i];
        for (int j = 0; j < 4; ++j) {
            if (bits == 4) {
                uint8_t lo = (uint8_t)((word >> (j * 8)) & 0xF), hi = (uint8_t)((word >> (j * 8 + 4)) & 0xF);
                packed[i * 4 + j] = (uint8_t)(lo | (hi << 4));
            } else packed[i * 4 + j] = (uint8_t)((word >> (j * 8)) & 0xFF);
        }
    }
}

/* crates/rmlx-nn/src/attention.rs:4853-4862 -- packer: word |= q << (k*bits). */
void oracle_pack_u32(const uint8_t* q, size_t n_values, int bits, uint32_t* words) {
    size_t per = 32 / (size_t)bits;
    for (size_t w = 0; w < n_values / per; ++w) {
        uint32_t word = 0;
        for (size_t kk = 0; kk < per; ++kk) word |= (uint32_t)q[w * per + kk] << (kk * (size_t)bits);
        words[w] = word;
    }
}

/* crates/rmlx-core/src/ops/quantized.rs:206-208 -- extract_bits. */
uint32_t oracle_extract_bits(uint32_t word, uint32_t idx_in_word, uint32_t bits) {
    return (word >> (idx_in_word * bits)) & ((1u << bits) - 1u);
}

/* crates/rmlx-core/src/ops/quantized.rs:12018-12049 -- u32-word Q4 qmv, f32, k ascending. */
void oracle_cpu_qmv_q4_reference(const uint32_t* weights_u32, const float* scales, const float* biases,
                                 const float* x, size_t n, size_t k, size_t group_size, float* output) {
    size_t u32s_per_row = k / 8, gpr = k / group_size;
    for (size_t row = 0; row < n; ++row) {
        float acc = 0.0f;
        for (size_t col = 0; col < k; ++col) {
            uint32_t word = weights_u32[row * u32s_per_row + col / 8];
            float q = (float)((word >> ((col % 8) * 4)) & 0xF);
            float w = scales[row * gpr + col / group_size] * q + biases[row * gpr + col / group_size];
            acc += w * x[col];
        }
        output[row] = acc;
    }
}

/* Multi-threaded driver used only by the bench's cpu_baseline leg: output columns are
 * partitioned into contiguous 4-aligned ranges, each range runs the scalar loop nest above
 * unchanged (so every out[i,j] is computed by exactly the same operation sequence). */
void oracle_affine_qmm_cols(const float* x, const uint8_t* w_packed, const float* scales,
                            const float* biases, size_t m, size_t n, size_t k, size_t group_size,
                            int bits, size_t col_begin, size_t col_end, float* output) {
    /* output is the full [m,n] buffer; this call fills columns [col_begin, col_end). */
    const size_t gpr = k / group_size;
    const size_t wrow = bits == 4 ? k / 2 : k;
    for (size_t row = 0; row < m; row += 4) {
        size_t rm = (m - row < 4) ? m - row : 4;
        for (size_t col = col_begin; col < col_end; col += 4) {
            size_t rn = (col_end - col < 4) ? col_end - col : 4;
            for (size_t ii = 0; ii < rm; ++ii)
                for (size_t jj = 0; jj < rn; ++jj) output[(row + ii) * n + col + jj] = 0.0f;
            for (size_t g = 0; g < gpr; ++g) {
                size_t k_start = g * group_size, k_end = k_start + group_size;
                for (size_t jj = 0; jj < rn; ++jj) {
                    size_t j = col + jj;
                    float scale = scales[j * gpr + g], bias = biases[j * gpr + g];
                    const uint8_t* w_row = w_packed + j * wrow;
                    for (size_t ii = 0; ii < rm; ++ii) {
                        const float* x_row = x + (row + ii) * k;
                        float dot = 0.0f, xsum = 0.0f;
                        for (size_t kk = k_start; kk < k_end; ++kk) {
                            float q = bits == 4 ? (float)dequant_q4_nibble(w_row[kk / 2], kk % 2)
                                                : (float)w_row[kk];
                            float xv = x_row[kk];
                            dot += q * xv;
                            xsum += xv;
                        }
                        output[(row + ii) * n + j] += scale * dot + bias * xsum;
                    }
                }
            }
        }
    }
}
