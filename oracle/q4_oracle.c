/*
 * q4_oracle.c — CPU restatement of lattice's Q4 block-quantized matmul semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP path is compared
 * against; nothing in the shipped library links, loads or calls it.  Build with
 * `make -C oracle` (flags matter: -ffp-contract=off keeps `acc += x*w` as a
 * separate multiply and add, exactly as the Rust reference evaluates it).
 *
 * Every function cites the reference span it restates (paths relative to the
 * lattice repository root).  How each one is pinned (golden bytes, closed
 * forms, brute force vs hardware conversions) is listed in tests/test_oracle_*.py.
 *
 * Parity status: every function in this file is pinned by at least one
 * reference-held vector or a mathematical identity; none is "parity unpinned".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LQ4_BLOCK_BYTES 20 /* crates/inference/src/weights/q4_weights.rs:84 */
#define LQ4_BLOCK_WEIGHTS 32 /* crates/inference/src/weights/q4_weights.rs:92 */

/* ------------------------------------------------------------------------- */
/* f16 <-> f32 bit conversion                                                 */
/* ------------------------------------------------------------------------- */

static float bits_to_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static uint32_t f32_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* crates/inference/src/weights/half_bits.rs:24-53 — exact widening, subnormals
 * normalised, NaN payload shifted into the f32 mantissa. */
float lq4o_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h >> 15) & 1u;
    uint32_t exp = (uint32_t)(h >> 10) & 0x1fu;
    uint32_t frac = (uint32_t)h & 0x3ffu;
    uint32_t out;
    if (exp == 0 && frac == 0) {
        out = sign << 31;
    } else if (exp == 0) {
        int e = -14;
        uint32_t mant = frac;
        while ((mant & 0x400u) == 0) {
            mant <<= 1;
            e -= 1;
        }
        mant &= 0x3ffu;
        out = (sign << 31) | ((uint32_t)(e + 127) << 23) | (mant << 13);
    } else if (exp == 0x1f && frac == 0) {
        out = (sign << 31) | 0x7f800000u;
    } else if (exp == 0x1f) {
        out = (sign << 31) | 0x7f800000u | (frac << 13);
    } else {
        out = (sign << 31) | ((uint32_t)((int)exp - 15 + 127) << 23) | (frac << 13);
    }
    return bits_to_f32(out);
}

/* crates/inference/src/weights/f16_encode.rs:4-23 */
static uint32_t round_shift_right_even(uint32_t value, uint32_t shift) {
    if (shift == 0) return value;
    if (shift >= 32) return 0;
    uint32_t base = value >> shift;
    uint32_t mask = (1u << shift) - 1u;
    uint32_t rem = value & mask;
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (base & 1u) != 0)) return base + 1;
    return base;
}

/* crates/inference/src/weights/f16_encode.rs:27-84 — round-to-nearest-even,
 * overflow -> inf, f32 subnormal input -> signed zero, NaN quieted. */
uint16_t lq4o_f32_to_f16(float v) {
    uint32_t bits = f32_to_bits(v);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int exp = (int)((bits >> 23) & 0xffu);
    uint32_t frac = bits & 0x007fffffu;

    if (exp == 0xff) {
        if (frac == 0) return sign | 0x7c00u;
        uint16_t payload = (uint16_t)(frac >> 13);
        if (payload == 0) payload = 1;
        payload |= 0x0200u;
        return sign | 0x7c00u | (payload & 0x03ffu);
    }
    if (exp == 0) return sign;

    int exp32 = exp - 127;
    if (exp32 > 15) return sign | 0x7c00u;

    if (exp32 >= -14) {
        uint16_t exp16 = (uint16_t)(exp32 + 15);
        uint16_t frac16 = (uint16_t)round_shift_right_even(frac, 13);
        if (frac16 == 0x0400u) {
            frac16 = 0;
            exp16 += 1;
            if (exp16 >= 0x1f) return sign | 0x7c00u;
        }
        return sign | (uint16_t)(exp16 << 10) | frac16;
    }

    uint32_t mant = frac | 0x00800000u;
    uint32_t shift = (uint32_t)(-exp32 - 1);
    if (shift >= 32) return sign;
    uint16_t frac16 = (uint16_t)round_shift_right_even(mant, shift);
    if (frac16 == 0) return sign;
    if (frac16 == 0x0400u) return sign | 0x0400u;
    return sign | frac16;
}

/* crates/inference/src/weights/half_bits.rs:55-63 */
float lq4o_bf16_to_f32(uint16_t b) { return bits_to_f32((uint32_t)b << 16); }

/* Array forms of the two conversions (inputs/outputs are raw bit patterns). */
void lq4o_f16_to_f32_array(const uint16_t* in, uint32_t* out_bits, size_t n) {
    for (size_t i = 0; i < n; ++i) out_bits[i] = f32_to_bits(lq4o_f16_to_f32(in[i]));
}
void lq4o_f32_to_f16_array(const uint32_t* in_bits, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = lq4o_f32_to_f16(bits_to_f32(in_bits[i]));
}

/* ------------------------------------------------------------------------- */
/* Block quantizer                                                            */
/* ------------------------------------------------------------------------- */

/* crates/inference/src/weights/q4_weights.rs:161-165 */
static int scale_survives_f16(float scale) {
    float s = lq4o_f16_to_f32(lq4o_f32_to_f16(scale));
    return isfinite(s) && s > 0.0f;
}

/* crates/inference/src/weights/q4_weights.rs:210-216 */
static float degenerate_safe_scale(float candidate) {
    if (candidate < 1.0f && !scale_survives_f16(candidate)) return 1.0f;
    return candidate;
}

/* Rust `f32::clamp(0.0, 15.0) as u8`: NaN saturates to 0 in the cast. */
static uint8_t clamp_nibble(float v) {
    if (v != v) return 0;
    if (v < 0.0f) v = 0.0f;
    if (v > 15.0f) v = 15.0f;
    return (uint8_t)v;
}

/* Error codes shared by the quantizer entry points. */
#define LQ4O_OK 0
#define LQ4O_ERR_VALID_LEN 1  /* valid_len outside 1..=32 */
#define LQ4O_ERR_NONFINITE 2  /* a source weight is NaN/inf */
#define LQ4O_ERR_SCALE 3      /* scale not a finite, strictly positive f16 */
#define LQ4O_ERR_BIAS 4       /* bias not a finite f16 */

/* crates/inference/src/weights/q4_weights.rs:239-295 (+ metadata rule :166-181).
 * `vals` holds 32 floats (caller zero-pads the tail); writes one 20-byte block. */
int lq4o_quantize_block(const float* vals, int valid_len, int symmetric, uint8_t* out) {
    if (valid_len < 1 || valid_len > 32) return LQ4O_ERR_VALID_LEN;
    for (int i = 0; i < 32; ++i)
        if (!isfinite(vals[i])) return LQ4O_ERR_NONFINITE;

    float scale, bias, sub;
    if (symmetric) {
        float abs_max = 0.0f;
        for (int i = 0; i < 32; ++i) {
            float a = fabsf(vals[i]);
            if (a > abs_max) abs_max = a;
        }
        scale = degenerate_safe_scale(abs_max / 7.0f);
        bias = -8.0f * scale;
        sub = 0.0f;
    } else {
        float mn = INFINITY, mx = -INFINITY;
        for (int i = 0; i < valid_len; ++i) {
            if (vals[i] < mn) mn = vals[i];
            if (vals[i] > mx) mx = vals[i];
        }
        scale = degenerate_safe_scale((mx - mn) / 15.0f);
        bias = mn;
        sub = mn;
    }
    uint16_t scale_bits = lq4o_f32_to_f16(scale);
    uint16_t bias_bits = lq4o_f32_to_f16(bias);
    if (!scale_survives_f16(scale)) return LQ4O_ERR_SCALE;
    if (!isfinite(lq4o_f16_to_f32(bias_bits))) return LQ4O_ERR_BIAS;

    float inv_scale = 1.0f / scale;
    out[0] = (uint8_t)(scale_bits & 0xff);
    out[1] = (uint8_t)(scale_bits >> 8);
    out[2] = (uint8_t)(bias_bits & 0xff);
    out[3] = (uint8_t)(bias_bits >> 8);
    for (int b = 0; b < 16; ++b) {
        uint8_t q0, q1;
        if (symmetric) {
            q0 = clamp_nibble(roundf(vals[2 * b] * inv_scale) + 8.0f);
            q1 = clamp_nibble(roundf(vals[2 * b + 1] * inv_scale) + 8.0f);
        } else {
            q0 = clamp_nibble(roundf((vals[2 * b] - sub) * inv_scale));
            q1 = clamp_nibble(roundf((vals[2 * b + 1] - sub) * inv_scale));
        }
        out[4 + b] = (uint8_t)((q1 << 4) | (q0 & 0x0f));
    }
    return LQ4O_OK;
}

/* Flat blocking over `n` values, last block zero-padded:
 * quantize_row_q4_0 (q4_weights.rs:312-328, asymmetric) and
 * quantize_f32_to_q4 / quantize_f64_to_q4_mode (q4_weights.rs:470-556).
 * `out` must hold ceil(n/32)*20 bytes. */
int lq4o_quantize_flat(const float* src, size_t n, int symmetric, uint8_t* out) {
    size_t nb = (n + 31) / 32;
    for (size_t blk = 0; blk < nb; ++blk) {
        float vals[32];
        size_t base = blk * 32;
        int len = (int)((n - base) < 32 ? (n - base) : 32);
        for (int i = 0; i < 32; ++i) vals[i] = i < len ? src[base + i] : 0.0f;
        int rc = lq4o_quantize_block(vals, len, symmetric, out + blk * LQ4_BLOCK_BYTES);
        if (rc) return rc;
    }
    return LQ4O_OK;
}

/* quantize_tensor_q4_0 (q4_weights.rs:364-388): each row blocked on its own. */
int lq4o_quantize_rows(const float* src, size_t rows, size_t cols, int symmetric, uint8_t* out) {
    size_t bpr = (cols + 31) / 32;
    for (size_t r = 0; r < rows; ++r) {
        int rc = lq4o_quantize_flat(src + r * cols, cols, symmetric, out + r * bpr * LQ4_BLOCK_BYTES);
        if (rc) return rc;
    }
    return LQ4O_OK;
}

/* ------------------------------------------------------------------------- */
/* Dequantize                                                                 */
/* ------------------------------------------------------------------------- */

/* dequantize_row_q4_0 (q4_weights.rs:340-353): complete blocks only, output
 * truncated to n_weights; returns the number of floats written. */
size_t lq4o_dequantize(const uint8_t* data, size_t nbytes, size_t n_weights, float* out) {
    size_t nb = nbytes / LQ4_BLOCK_BYTES;
    size_t w = 0;
    for (size_t blk = 0; blk < nb && w < n_weights; ++blk) {
        const uint8_t* c = data + blk * LQ4_BLOCK_BYTES;
        float scale = lq4o_f16_to_f32((uint16_t)(c[0] | (c[1] << 8)));
        float bias = lq4o_f16_to_f32((uint16_t)(c[2] | (c[3] << 8)));
        for (int b = 0; b < 16 && w < n_weights; ++b) {
            uint8_t byte = c[4 + b];
            out[w++] = (float)(byte & 0x0f) * scale + bias;
            if (w < n_weights) out[w++] = (float)(byte >> 4) * scale + bias;
        }
    }
    return w;
}

/* Per-block metadata rule (weights/ingress.rs:542-559 through
 * q4_weights.rs:876-918): scale finite and > 0, bias finite.  Returns the index
 * of the first offending block, or -1 when every block passes.  `*why` gets
 * 1 for a bad scale, 2 for a bad bias. */
long lq4o_validate_blocks(const uint8_t* payload, size_t nbytes, int* why) {
    size_t nb = nbytes / LQ4_BLOCK_BYTES;
    for (size_t blk = 0; blk < nb; ++blk) {
        const uint8_t* c = payload + blk * LQ4_BLOCK_BYTES;
        float scale = lq4o_f16_to_f32((uint16_t)(c[0] | (c[1] << 8)));
        float bias = lq4o_f16_to_f32((uint16_t)(c[2] | (c[3] << 8)));
        if (!isfinite(scale) || scale <= 0.0f) {
            if (why) *why = 1;
            return (long)blk;
        }
        if (!isfinite(bias)) {
            if (why) *why = 2;
            return (long)blk;
        }
    }
    if (why) *why = 0;
    return -1;
}

/* ------------------------------------------------------------------------- */
/* Matmul oracle:  Y[M,N] = X[M,K] . dequant(W_q4[N,K])^T                      */
/* ------------------------------------------------------------------------- */

/* Composition the reference's own GPU tests use as ground truth:
 * dequantize_row_q4_0 per weight row, then cpu_matmul_ref — sequential f32
 * `acc += x*w`, k ascending (forward/metal_qwen35.rs:22850-22899).
 * W is N rows of (K/32) blocks, row stride (K/32)*20 bytes. */
int lq4o_gemm_f32(const float* x, const uint8_t* wq, float* y, size_t m, size_t n, size_t k) {
    if (k == 0 || k % 32 != 0) return 1;
    size_t row_bytes = (k / 32) * LQ4_BLOCK_BYTES;
    float* wrow = (float*)malloc(k * sizeof(float));
    if (!wrow) return 2;
    for (size_t ni = 0; ni < n; ++ni) {
        lq4o_dequantize(wq + ni * row_bytes, row_bytes, k, wrow);
        for (size_t mi = 0; mi < m; ++mi) {
            const float* xr = x + mi * k;
            float acc = 0.0f;
            for (size_t ki = 0; ki < k; ++ki) acc += xr[ki] * wrow[ki];
            y[mi * n + ni] = acc;
        }
    }
    free(wrow);
    return 0;
}

/* Same contraction accumulated in f64 (products of two f32 are exact in f64):
 * separates a kernel's error from the f32 oracle's own summation error.  This
 * is the form quarot_rotated_q4_forward_matches_f64_reference uses
 * (weights/q4_weights.rs:2487-2672). */
int lq4o_gemm_f64(const float* x, const uint8_t* wq, double* y, size_t m, size_t n, size_t k) {
    if (k == 0 || k % 32 != 0) return 1;
    size_t row_bytes = (k / 32) * LQ4_BLOCK_BYTES;
    float* wrow = (float*)malloc(k * sizeof(float));
    if (!wrow) return 2;
    for (size_t ni = 0; ni < n; ++ni) {
        lq4o_dequantize(wq + ni * row_bytes, row_bytes, k, wrow);
        for (size_t mi = 0; mi < m; ++mi) {
            const float* xr = x + mi * k;
            double acc = 0.0;
            for (size_t ki = 0; ki < k; ++ki) acc += (double)xr[ki] * (double)wrow[ki];
            y[mi * n + ni] = acc;
        }
    }
    free(wrow);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* LoRA delta:  y[row] += scale * B . (A . x[row])                             */
/* ------------------------------------------------------------------------- */

/* apply_lora (crates/tune/src/lora/apply.rs:48-98): t[r] = sum_k A[r,k]*x[k]
 * (sequential f32), then y[n] += scale * sum_j B[n,j]*t[j].  A is [rank,d_in],
 * B is [d_out,rank], both row-major f32.  Applied independently to each of
 * `m` rows, as apply_lora_rows does (crates/inference/src/lora_hook.rs). */
void lq4o_lora_apply(const float* a, const float* b, size_t rank, size_t d_in, size_t d_out,
                     float scale, const float* x, float* y, size_t m) {
    float* t = (float*)malloc((rank ? rank : 1) * sizeof(float));
    for (size_t mi = 0; mi < m; ++mi) {
        const float* xr = x + mi * d_in;
        float* yr = y + mi * d_out;
        for (size_t r = 0; r < rank; ++r) {
            float acc = 0.0f;
            for (size_t kk = 0; kk < d_in; ++kk) acc += a[r * d_in + kk] * xr[kk];
            t[r] = acc;
        }
        for (size_t nn = 0; nn < d_out; ++nn) {
            float acc = 0.0f;
            for (size_t j = 0; j < rank; ++j) acc += b[nn * rank + j] * t[j];
            yr[nn] += scale * acc;
        }
    }
    free(t);
}

/* f64 twin of the above (A, B, x widened exactly), y accumulated in f64. */
void lq4o_lora_apply_f64(const float* a, const float* b, size_t rank, size_t d_in, size_t d_out,
                         float scale, const float* x, double* y, size_t m) {
    double* t = (double*)malloc((rank ? rank : 1) * sizeof(double));
    for (size_t mi = 0; mi < m; ++mi) {
        const float* xr = x + mi * d_in;
        double* yr = y + mi * d_out;
        for (size_t r = 0; r < rank; ++r) {
            double acc = 0.0;
            for (size_t kk = 0; kk < d_in; ++kk) acc += (double)a[r * d_in + kk] * (double)xr[kk];
            t[r] = acc;
        }
        for (size_t nn = 0; nn < d_out; ++nn) {
            double acc = 0.0;
            for (size_t j = 0; j < rank; ++j) acc += (double)b[nn * rank + j] * t[j];
            yr[nn] += (double)scale * acc;
        }
    }
    free(t);
}

/* ------------------------------------------------------------------------- */
/* MoE routing and routed-expert accumulation                                 */
/* ------------------------------------------------------------------------- */

/* compute_router_probs (crates/inference/src/model/qwen35/moe.rs:39-95), from the
 * logits row on (the router GEMV itself is not on this path): softmax over all
 * E with the max subtracted; a non-finite max, or a denominator that is not
 * > 0 (NaN included), zeroes the whole row. */
void lq4o_router_softmax(const float* logits, int num_experts, float* probs) {
    float mx = -INFINITY;
    for (int e = 0; e < num_experts; ++e) {
        /* Rust f32::max returns the other operand when one is NaN. */
        if (logits[e] > mx || mx != mx) mx = logits[e];
    }
    if (!isfinite(mx)) {
        for (int e = 0; e < num_experts; ++e) probs[e] = 0.0f;
        return;
    }
    float denom = 0.0f;
    for (int e = 0; e < num_experts; ++e) {
        probs[e] = expf(logits[e] - mx);
        denom += probs[e];
    }
    if (denom > 0.0f) {
        for (int e = 0; e < num_experts; ++e) probs[e] /= denom;
    } else {
        for (int e = 0; e < num_experts; ++e) probs[e] = 0.0f;
    }
}

/* select_top_k (moe.rs:97-116): insertion by strict `>` against slots seeded
 * with -inf, so equal probabilities keep the lower expert id first and a slot
 * nothing beats stays unfilled (id -1 here, usize::MAX there). */
void lq4o_select_top_k(const float* probs, int num_experts, int top_k, int32_t* ids, float* vals) {
    for (int r = 0; r < top_k; ++r) {
        ids[r] = -1;
        vals[r] = -INFINITY;
    }
    for (int e = 0; e < num_experts; ++e) {
        float p = probs[e];
        for (int r = 0; r < top_k; ++r) {
            if (p > vals[r]) {
                for (int s = top_k - 1; s > r; --s) {
                    ids[s] = ids[s - 1];
                    vals[s] = vals[s - 1];
                }
                ids[r] = e;
                vals[r] = p;
                break;
            }
        }
    }
}

/* renormalize_selected (moe.rs:118-125): divide by the sequential f32 sum of
 * the selected values when that sum is positive. */
void lq4o_renormalize_selected(float* vals, int top_k) {
    float top_sum = 0.0f;
    for (int r = 0; r < top_k; ++r) top_sum += vals[r];
    if (top_sum > 0.0f)
        for (int r = 0; r < top_k; ++r) vals[r] /= top_sum;
}

/* The three steps in the order moe_ffn_step runs them (moe.rs:25-31). */
void lq4o_moe_route(const float* logits, int num_experts, int top_k, float* probs, int32_t* ids,
                    float* weights) {
    lq4o_router_softmax(logits, num_experts, probs);
    lq4o_select_top_k(probs, num_experts, top_k, ids, weights);
    lq4o_renormalize_selected(weights, top_k);
}

/* silu_inplace_scalar (crates/inference/src/forward/cpu/elementwise.rs:140-144) */
static float silu_f32(float v) { return v * (1.0f / (1.0f + expf(-v))); }

/* accumulate_routed_experts (moe.rs:127-190) with the expert tensors held as Q4
 * blocks instead of f32: gate_up is [E, 2I, H] (gate rows first, then up rows),
 * down is [E, H, I]; out[t,:] = sum over the token's selected experts of
 * w * W_down . (silu(W_gate . x) * (W_up . x)).  Slots with id outside
 * [0, E) are skipped, as the reference does for unfilled slots.  Each GEMV is
 * dequantize -> sequential f32 dot.  H and I must be multiples of 32. */
int lq4o_moe_ffn_f32(const uint8_t* gate_up_q4, const uint8_t* down_q4, int num_experts, int inter,
                     int hidden, const float* x, int tokens, const int32_t* ids,
                     const float* weights, int top_k, float* out) {
    if (hidden % 32 || inter % 32) return 1;
    size_t gu_bytes = (size_t)2 * inter * (hidden / 32) * LQ4_BLOCK_BYTES;
    size_t dn_bytes = (size_t)hidden * (inter / 32) * LQ4_BLOCK_BYTES;
    float* gu = (float*)malloc((size_t)2 * inter * sizeof(float));
    float* o = (float*)malloc((size_t)hidden * sizeof(float));
    for (int t = 0; t < tokens; ++t) {
        const float* xt = x + (size_t)t * hidden;
        float* ot = out + (size_t)t * hidden;
        for (int i = 0; i < hidden; ++i) ot[i] = 0.0f;
        for (int s = 0; s < top_k; ++s) {
            int e = ids[t * top_k + s];
            float w = weights[t * top_k + s];
            if (e < 0 || e >= num_experts) continue;
            lq4o_gemm_f32(xt, gate_up_q4 + (size_t)e * gu_bytes, gu, 1, (size_t)2 * inter, hidden);
            for (int i = 0; i < inter; ++i) gu[i] = silu_f32(gu[i]) * gu[inter + i];
            lq4o_gemm_f32(gu, down_q4 + (size_t)e * dn_bytes, o, 1, hidden, inter);
            for (int i = 0; i < hidden; ++i) ot[i] += w * o[i];
        }
    }
    free(gu);
    free(o);
    return 0;
}

/* f64 twin: every dot, the SiLU and the weighted sum carried in f64. */
int lq4o_moe_ffn_f64(const uint8_t* gate_up_q4, const uint8_t* down_q4, int num_experts, int inter,
                     int hidden, const float* x, int tokens, const int32_t* ids,
                     const float* weights, int top_k, double* out) {
    if (hidden % 32 || inter % 32) return 1;
    size_t gu_row = (size_t)(hidden / 32) * LQ4_BLOCK_BYTES;
    size_t dn_row = (size_t)(inter / 32) * LQ4_BLOCK_BYTES;
    size_t gu_bytes = (size_t)2 * inter * gu_row;
    size_t dn_bytes = (size_t)hidden * dn_row;
    float* wrow = (float*)malloc((size_t)(hidden > inter ? hidden : inter) * sizeof(float));
    double* gu = (double*)malloc((size_t)2 * inter * sizeof(double));
    for (int t = 0; t < tokens; ++t) {
        const float* xt = x + (size_t)t * hidden;
        double* ot = out + (size_t)t * hidden;
        for (int i = 0; i < hidden; ++i) ot[i] = 0.0;
        for (int s = 0; s < top_k; ++s) {
            int e = ids[t * top_k + s];
            double w = (double)weights[t * top_k + s];
            if (e < 0 || e >= num_experts) continue;
            const uint8_t* gw = gate_up_q4 + (size_t)e * gu_bytes;
            for (int r = 0; r < 2 * inter; ++r) {
                lq4o_dequantize(gw + (size_t)r * gu_row, gu_row, hidden, wrow);
                double acc = 0.0;
                for (int kk = 0; kk < hidden; ++kk) acc += (double)xt[kk] * (double)wrow[kk];
                gu[r] = acc;
            }
            for (int i = 0; i < inter; ++i) gu[i] = gu[i] / (1.0 + exp(-gu[i])) * gu[inter + i];
            const uint8_t* dw = down_q4 + (size_t)e * dn_bytes;
            for (int r = 0; r < hidden; ++r) {
                lq4o_dequantize(dw + (size_t)r * dn_row, dn_row, inter, wrow);
                double acc = 0.0;
                for (int kk = 0; kk < inter; ++kk) acc += gu[kk] * (double)wrow[kk];
                ot[r] += w * acc;
            }
        }
    }
    free(wrow);
    free(gu);
    return 0;
}

/* apply_shared_expert (moe.rs:194-250) with the shared expert's tensors held as Q4
 * blocks: gate_up is [2*SI, H] (gate_proj rows, then up_proj rows), down is [H, SI].
 * Per token: g = 1 / (1 + exp(-dot(x, shared_gate))) with the dot summed
 * sequentially in f32 (the iterator .sum() of moe.rs:201-206), then
 * out[i] += g * (W_down . (silu(W_gate . x) * (W_up . x)))[i] (moe.rs:242-244):
 * `out` is accumulated into, as the reference adds onto the routed experts' sum. */
int lq4o_moe_shared_expert_f32(const uint8_t* gate_up_q4, const uint8_t* down_q4,
                               const float* shared_gate, int shared_inter, int hidden,
                               const float* x, int tokens, float* out) {
    if (hidden % 32 || shared_inter % 32) return 1;
    float* gu = (float*)malloc((size_t)2 * shared_inter * sizeof(float));
    float* o = (float*)malloc((size_t)hidden * sizeof(float));
    for (int t = 0; t < tokens; ++t) {
        const float* xt = x + (size_t)t * hidden;
        float* ot = out + (size_t)t * hidden;
        float logit = 0.0f;
        for (int i = 0; i < hidden; ++i) logit += xt[i] * shared_gate[i];
        const float g = 1.0f / (1.0f + expf(-logit));
        lq4o_gemm_f32(xt, gate_up_q4, gu, 1, (size_t)2 * shared_inter, hidden);
        for (int i = 0; i < shared_inter; ++i) gu[i] = silu_f32(gu[i]) * gu[shared_inter + i];
        lq4o_gemm_f32(gu, down_q4, o, 1, hidden, shared_inter);
        for (int i = 0; i < hidden; ++i) ot[i] += g * o[i];
    }
    free(gu);
    free(o);
    return 0;
}

/* f64 twin: gate logit, sigmoid, every dot, the SiLU and the scaled add in f64. */
int lq4o_moe_shared_expert_f64(const uint8_t* gate_up_q4, const uint8_t* down_q4,
                               const float* shared_gate, int shared_inter, int hidden,
                               const float* x, int tokens, double* out) {
    if (hidden % 32 || shared_inter % 32) return 1;
    size_t gu_row = (size_t)(hidden / 32) * LQ4_BLOCK_BYTES;
    size_t dn_row = (size_t)(shared_inter / 32) * LQ4_BLOCK_BYTES;
    float* wrow = (float*)malloc((size_t)(hidden > shared_inter ? hidden : shared_inter) * sizeof(float));
    double* gu = (double*)malloc((size_t)2 * shared_inter * sizeof(double));
    for (int t = 0; t < tokens; ++t) {
        const float* xt = x + (size_t)t * hidden;
        double* ot = out + (size_t)t * hidden;
        double logit = 0.0;
        for (int i = 0; i < hidden; ++i) logit += (double)xt[i] * (double)shared_gate[i];
        const double g = 1.0 / (1.0 + exp(-logit));
        for (int r = 0; r < 2 * shared_inter; ++r) {
            lq4o_dequantize(gate_up_q4 + (size_t)r * gu_row, gu_row, hidden, wrow);
            double acc = 0.0;
            for (int kk = 0; kk < hidden; ++kk) acc += (double)xt[kk] * (double)wrow[kk];
            gu[r] = acc;
        }
        for (int i = 0; i < shared_inter; ++i) gu[i] = gu[i] / (1.0 + exp(-gu[i])) * gu[shared_inter + i];
        for (int r = 0; r < hidden; ++r) {
            lq4o_dequantize(down_q4 + (size_t)r * dn_row, dn_row, shared_inter, wrow);
            double acc = 0.0;
            for (int kk = 0; kk < shared_inter; ++kk) acc += gu[kk] * (double)wrow[kk];
            ot[r] += g * acc;
        }
    }
    free(wrow);
    free(gu);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* `.q4` file header                                                          */
/* ------------------------------------------------------------------------- */

/* read_q4_header + validate_q4_header_payload_bounds
 * (weights/q4_weights.rs:709-812): "KHQ4", u32 version (1 = legacy, rejected;
 * only 2 accepted), u32 ndim, u64 shape[ndim], u64 original_len, then exactly
 * ceil(original_len/32) blocks and nothing after them.
 * Returns 0 and fills the outputs, or: 1 short/bad magic, 2 legacy v1,
 * 3 unsupported version, 4 header truncated / ndim beyond max_dims,
 * 5 payload truncated, 6 trailing bytes, 7 shape product != original_len. */
int lq4o_parse_q4_file(const uint8_t* file, size_t file_len, uint64_t* shape, int max_dims,
                       int* ndim_out, uint64_t* original_len, uint64_t* payload_offset) {
    if (file_len < 12 || memcmp(file, "KHQ4", 4) != 0) return 1;
    uint32_t ver, ndim;
    memcpy(&ver, file + 4, 4);
    memcpy(&ndim, file + 8, 4);
    if (ver == 1) return 2;
    if (ver != 2) return 3;
    if ((int)ndim > max_dims || (uint64_t)ndim * 8 + 20 > file_len) return 4;
    uint64_t prod = 1;
    for (uint32_t i = 0; i < ndim; ++i) {
        memcpy(&shape[i], file + 12 + 8 * (size_t)i, 8);
        prod *= shape[i];
    }
    uint64_t olen;
    memcpy(&olen, file + 12 + 8 * (size_t)ndim, 8);
    uint64_t off = 20 + 8 * (uint64_t)ndim;
    uint64_t need = off + ((olen + 31) / 32) * LQ4_BLOCK_BYTES;
    if (file_len < need) return 5;
    if (file_len > need) return 6;
    if (prod != olen) return 7;
    *ndim_out = (int)ndim;
    *original_len = olen;
    *payload_offset = off;
    return 0;
}

/* ---- Q8_0 sibling format -------------------------------------------------------------
 * Block = [u16 f16 scale d, little endian][32 x i8], 34 bytes, 32 weights; w = q * f16(d).
 * quantize_row_q8_0 (forward/metal_qwen35.rs:2323-2346): per block amax = max|v|, d = amax / 127,
 * id = 1 / d (0 if d == 0), q = clamp(round(v * id), -127, 127) with round-half-away-from-zero;
 * the stored scale is f16(d) while the quotient uses the f32 d.  Returns 0, or -(1 + index of the
 * first block holding a non-finite value): the reference rejects such rows. */
#define LQ8_BLOCK_BYTES 34
long lq4o_q8_quantize_row(const float* src, size_t len, uint8_t* out) {
    if (len % 32 != 0) return -1;
    for (size_t b = 0; b < len / 32; ++b) {
        const float* blk = src + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) {
            if (!isfinite(blk[i])) return -(long)(1 + b);
            const float a = fabsf(blk[i]);
            if (a > amax) amax = a;
        }
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const uint16_t bits = lq4o_f32_to_f16(d);
        uint8_t* o = out + b * LQ8_BLOCK_BYTES;
        o[0] = (uint8_t)(bits & 0xff);
        o[1] = (uint8_t)(bits >> 8);
        for (int i = 0; i < 32; ++i) {
            float r = roundf(blk[i] * id);
            if (r < -127.0f) r = -127.0f;
            if (r > 127.0f) r = 127.0f;
            o[2 + i] = (uint8_t)(int8_t)r;
        }
    }
    return 0;
}

/* The dequantisation the reference's Q8_0 tests use as ground truth
 * (forward/metal_qwen35.rs:23255-23262): f32(i8) * f32(f16 scale). */
size_t lq4o_q8_dequantize(const uint8_t* data, size_t n_weights, float* out) {
    const size_t nb = n_weights / 32;
    for (size_t b = 0; b < nb; ++b) {
        const uint8_t* blk = data + b * LQ8_BLOCK_BYTES;
        const float d = lq4o_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        for (int i = 0; i < 32; ++i) out[b * 32 + i] = (float)(int8_t)blk[2 + i] * d;
    }
    return nb * 32;
}

/* Y[M,N] = X[M,K] . W_q8[N,K]^T in the arithmetic of gemv_q8_decode (shaders/qwen35.metal:133-190):
 * per block sumq = sum_i f32(q_i) * x_i, y += sumq * f32(d); blocks in ascending order, f32. */
int lq4o_q8_gemm_f32(const float* x, const uint8_t* wq, float* y, size_t m, size_t n, size_t k) {
    if (k == 0 || k % 32 != 0) return 1;
    const size_t nb = k / 32, row_bytes = nb * LQ8_BLOCK_BYTES;
    for (size_t ni = 0; ni < n; ++ni)
        for (size_t mi = 0; mi < m; ++mi) {
            const float* xr = x + mi * k;
            float acc = 0.0f;
            for (size_t b = 0; b < nb; ++b) {
                const uint8_t* blk = wq + ni * row_bytes + b * LQ8_BLOCK_BYTES;
                const float d = lq4o_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
                float sumq = 0.0f;
                for (int i = 0; i < 32; ++i) sumq += (float)(int8_t)blk[2 + i] * xr[b * 32 + i];
                acc += sumq * d;
            }
            y[mi * n + ni] = acc;
        }
    return 0;
}

/* The same contraction over the dequantised weights in f64. */
int lq4o_q8_gemm_f64(const float* x, const uint8_t* wq, double* y, size_t m, size_t n, size_t k) {
    if (k == 0 || k % 32 != 0) return 1;
    const size_t nb = k / 32, row_bytes = nb * LQ8_BLOCK_BYTES;
    for (size_t ni = 0; ni < n; ++ni)
        for (size_t mi = 0; mi < m; ++mi) {
            const float* xr = x + mi * k;
            double acc = 0.0;
            for (size_t b = 0; b < nb; ++b) {
                const uint8_t* blk = wq + ni * row_bytes + b * LQ8_BLOCK_BYTES;
                const double d = (double)lq4o_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
                for (int i = 0; i < 32; ++i) acc += (double)(int8_t)blk[2 + i] * d * (double)xr[b * 32 + i];
            }
            y[mi * n + ni] = acc;
        }
    return 0;
}

/* ---- Q3 sibling format ---------------------------------------------------------------
 * Block = [u16 f16 scale][u16 f16 bias][8 bytes low-2-bit plane][4 bytes high-1-bit plane],
 * 16 bytes, 32 weights, w = q * scale + bias with q = low2 | hi << 2
 * (weights/q3_weights.rs:13-52, pack_plane_split :148-167, unpack_plane_split :170-175). */
#define LQ3_BLOCK_BYTES 16
static void lq3_pack(const uint8_t q[32], uint8_t packed[12]) {
    memset(packed, 0, 12);
    for (int b = 0; b < 8; ++b)
        packed[b] = (uint8_t)((q[4 * b] & 3) | ((q[4 * b + 1] & 3) << 2) | ((q[4 * b + 2] & 3) << 4) | ((q[4 * b + 3] & 3) << 6));
    for (int b = 0; b < 4; ++b)
        for (int k = 0; k < 8; ++k) packed[8 + b] |= (uint8_t)(((q[8 * b + k] >> 2) & 1) << k);
}

static uint8_t lq3_unpack(const uint8_t* packed, int i) {
    const uint8_t low2 = (packed[i / 4] >> ((i % 4) * 2)) & 3;
    const uint8_t hi = (packed[8 + i / 8] >> (i % 8)) & 1;
    return (uint8_t)(low2 | (hi << 2));
}

/* quantize_block_with_mode_len (weights/q3_weights.rs:199-262).  Returns 0, 1 for a bad
 * valid_len, 2 for a non-finite value. */
int lq4o_q3_quantize_block(const float* vals, int valid_len, int symmetric, uint8_t* out) {
    if (valid_len < 1 || valid_len > 32) return 1;
    for (int i = 0; i < 32; ++i)
        if (!isfinite(vals[i])) return 2;
    uint8_t q[32];
    float scale, bias;
    if (symmetric) {
        float abs_max = 0.0f;
        for (int i = 0; i < 32; ++i) abs_max = fmaxf(abs_max, fabsf(vals[i]));
        scale = abs_max == 0.0f ? 1.0f : abs_max / 3.5f;
        const float inv = 1.0f / scale;
        bias = -4.0f * scale;
        for (int i = 0; i < 32; ++i) {
            float r = roundf(vals[i] * inv) + 4.0f;
            r = r < 0.0f ? 0.0f : r > 7.0f ? 7.0f : r;
            q[i] = (uint8_t)r;
        }
    } else {
        float mn = INFINITY, mx = -INFINITY;
        for (int i = 0; i < valid_len; ++i) {
            mn = fminf(mn, vals[i]);
            mx = fmaxf(mx, vals[i]);
        }
        const float range = mx - mn;
        scale = range == 0.0f ? 1.0f : range / 7.0f;
        const float inv = 1.0f / scale;
        bias = mn;
        for (int i = 0; i < 32; ++i) {
            float r = roundf((vals[i] - mn) * inv);
            r = r < 0.0f ? 0.0f : r > 7.0f ? 7.0f : r;
            q[i] = (uint8_t)r;
        }
    }
    const uint16_t sb = lq4o_f32_to_f16(scale), bb = lq4o_f32_to_f16(bias);
    out[0] = (uint8_t)(sb & 0xff);
    out[1] = (uint8_t)(sb >> 8);
    out[2] = (uint8_t)(bb & 0xff);
    out[3] = (uint8_t)(bb >> 8);
    lq3_pack(q, out + 4);
    return 0;
}

/* quantize_row_q3_0 (weights/q3_weights.rs:279-299): 32 at a time, zero-padded tail block whose
 * range comes from the real values only. */
int lq4o_q3_quantize_row(const float* src, size_t len, int symmetric, uint8_t* out) {
    for (size_t b = 0; b * 32 < len; ++b) {
        float vals[32] = {0};
        const size_t take = len - b * 32 < 32 ? len - b * 32 : 32;
        memcpy(vals, src + b * 32, take * sizeof(float));
        const int rc = lq4o_q3_quantize_block(vals, (int)take, symmetric, out + b * LQ3_BLOCK_BYTES);
        if (rc) return rc;
    }
    return 0;
}

/* dequantize_row_q3_0 (weights/q3_weights.rs:306-319). */
size_t lq4o_q3_dequantize(const uint8_t* data, size_t nbytes, size_t n_weights, float* out) {
    size_t done = 0;
    for (size_t b = 0; (b + 1) * LQ3_BLOCK_BYTES <= nbytes && done < n_weights; ++b) {
        const uint8_t* blk = data + b * LQ3_BLOCK_BYTES;
        const float scale = lq4o_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        const float bias = lq4o_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        for (int i = 0; i < 32 && done < n_weights; ++i) out[done++] = (float)lq3_unpack(blk + 4, i) * scale + bias;
    }
    return done;
}

/* gemm_q3_reference / gemv_q3_reference (weights/q3_weights.rs:784-838): dequantise the row, then a
 * sequential f32 sum of products, k ascending. */
int lq4o_q3_gemm_f32(const float* x, const uint8_t* wq, float* y, size_t m, size_t n, size_t k) {
    if (k == 0 || k % 32 != 0) return 1;
    const size_t row_bytes = (k / 32) * LQ3_BLOCK_BYTES;
    float* wrow = (float*)malloc(k * sizeof(float));
    if (!wrow) return 2;
    for (size_t ni = 0; ni < n; ++ni) {
        lq4o_q3_dequantize(wq + ni * row_bytes, row_bytes, k, wrow);
        for (size_t mi = 0; mi < m; ++mi) {
            float acc = 0.0f;
            for (size_t ki = 0; ki < k; ++ki) acc += x[mi * k + ki] * wrow[ki];
            y[mi * n + ni] = acc;
        }
    }
    free(wrow);
    return 0;
}

int lq4o_q3_gemm_f64(const float* x, const uint8_t* wq, double* y, size_t m, size_t n, size_t k) {
    if (k == 0 || k % 32 != 0) return 1;
    const size_t row_bytes = (k / 32) * LQ3_BLOCK_BYTES;
    float* wrow = (float*)malloc(k * sizeof(float));
    if (!wrow) return 2;
    for (size_t ni = 0; ni < n; ++ni) {
        lq4o_q3_dequantize(wq + ni * row_bytes, row_bytes, k, wrow);
        for (size_t mi = 0; mi < m; ++mi) {
            double acc = 0.0;
            for (size_t ki = 0; ki < k; ++ki) acc += (double)x[mi * k + ki] * (double)wrow[ki];
            y[mi * n + ni] = acc;
        }
    }
    free(wrow);
    return 0;
}

/* ---- elementwise steps either side of the decode GEMVs ---------------------------------
 * Shifted RMSNorm of Qwen3.5, qwen35_rms_norm (crates/inference/src/model/qwen35/norm.rs:6-23):
 * per row a sequential f32 sum of squares, rms = sqrt(sum / hidden + eps), inv = 1 / rms,
 * out = x * inv * (1 + gamma), evaluated left to right in f32. */
void lq4o_shifted_rms_norm(float* x, const float* gamma, size_t hidden, size_t rows, float eps) {
    for (size_t t = 0; t < rows; ++t) {
        float* row = x + t * hidden;
        float sum_sq = 0.0f;
        for (size_t i = 0; i < hidden; ++i) sum_sq += row[i] * row[i];
        const float rms = sqrtf(sum_sq / (float)hidden + eps);
        const float inv_rms = 1.0f / rms;
        for (size_t i = 0; i < hidden; ++i) row[i] = row[i] * inv_rms * (1.0f + gamma[i]);
    }
}

/* fused_residual_add_norm / fused_residual_add_norm_batch (shaders/qwen35.metal:739-767,
 * 2219-2249): residual_out = base + delta, normed_out = shifted RMSNorm of residual_out. */
void lq4o_residual_add_norm(const float* base, const float* delta, const float* gamma, size_t hidden,
                            size_t rows, float eps, float* residual_out, float* normed_out) {
    for (size_t i = 0; i < hidden * rows; ++i) {
        residual_out[i] = base[i] + delta[i];
        normed_out[i] = residual_out[i];
    }
    lq4o_shifted_rms_norm(normed_out, gamma, hidden, rows, eps);
}

/* silu_mul_fused (shaders/qwen35.metal:712-722) per row of [gate(count) | up(count)]:
 * out[i] = gate / (1 + exp(-gate)) * up. */
void lq4o_silu_mul(const float* gate_up, size_t count, size_t rows, float* out) {
    for (size_t r = 0; r < rows; ++r)
        for (size_t i = 0; i < count; ++i) {
            const float gate = gate_up[r * 2 * count + i], up = gate_up[r * 2 * count + count + i];
            const float s = gate / (1.0f + expf(-gate));
            out[r * count + i] = s * up;
        }
}

/* add_and_copy (shaders/qwen35.metal:2255-2266): residual += src; dst = residual. */
void lq4o_add_and_copy(const float* src, float* residual, float* dst, size_t count) {
    for (size_t i = 0; i < count; ++i) {
        const float r = residual[i] + src[i];
        residual[i] = r;
        dst[i] = r;
    }
}

/* ---- lm_head top-k selection ----------------------------------------------------
 * The ordering of the reference's GPU top-k (shaders/qwen35.metal:1688-1703):
 * candidate = (logit, token_id); a ranks before b if it has the higher logit, ties go
 * to the lower token id; a NaN logit becomes the sentinel (-inf, UINT32_MAX) before it
 * enters the selection (qwen35.metal:1916, 1966) and so ranks last.  The two-stage
 * tile/merge scheme is exact by construction (qwen35.metal:1868-1892), so its result is
 * the first k entries of the fully sorted candidate list, which is what this computes.
 * Slots beyond the number of logits hold sentinels. */
static int lq4o_topk_better(float al, uint32_t ai, float bl, uint32_t bi) {
    if (al != al) return 0;
    if (bl != bl) return 1;
    if (al != bl) return al > bl;
    return ai < bi;
}

void lq4o_topk(const float* logits, uint32_t n, uint32_t k, float* out_logits, uint32_t* out_ids) {
    for (uint32_t r = 0; r < k; ++r) {
        out_logits[r] = -INFINITY;
        out_ids[r] = UINT32_MAX;
    }
    for (uint32_t i = 0; i < n; ++i) {
        float l = logits[i];
        uint32_t id = i;
        if (l != l) {
            l = -INFINITY;
            id = UINT32_MAX;
        }
        /* insertion into the sorted list of the best k so far */
        if (k == 0 || !lq4o_topk_better(l, id, out_logits[k - 1], out_ids[k - 1])) continue;
        uint32_t pos = k - 1;
        while (pos > 0 && lq4o_topk_better(l, id, out_logits[pos - 1], out_ids[pos - 1])) {
            out_logits[pos] = out_logits[pos - 1];
            out_ids[pos] = out_ids[pos - 1];
            --pos;
        }
        out_logits[pos] = l;
        out_ids[pos] = id;
    }
}
