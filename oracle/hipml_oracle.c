/*
 * CPU oracle for the hipml full-attention hot path.  TEST INFRASTRUCTURE ONLY:
 * see hipml_oracle.h.  Each function names the reference file:line it restates
 * and keeps that code's evaluation order (no fused multiply-add, no reordering).
 */
#include "hipml_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- format constants: crates/hipml-core/src/kv.rs:47-91 ---------------- */

size_t orc_block_bytes(int dtype) { return dtype == ORC_Q8 ? 34 : 18; }

size_t orc_row_bytes(int dtype, size_t head_dim)
{
    return head_dim / ORC_BLOCK * orc_block_bytes(dtype);
}

size_t orc_token_bytes(int dtype, size_t n_kv, size_t head_dim, size_t n_layers)
{
    return 2 * n_kv * n_layers * orc_row_bytes(dtype, head_dim);
}

/* ---- binary16 <-> binary32: kv.rs:94-165 -------------------------------- */

static float bits_f32(uint32_t b)
{
    float f;
    memcpy(&f, &b, 4);
    return f;
}

static uint32_t f32_bits(float f)
{
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)(h & 0x8000u)) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t mant = h & 0x03ff;
    if (exp == 0) {
        if (mant == 0)
            return bits_f32(sign);
        /* subnormal: mant * 2^-24 */
        float two_m24 = bits_f32((127u - 24u) << 23);
        float mag = (float)mant * two_m24;
        return sign ? -mag : mag;
    }
    if (exp == 0x1f)
        return bits_f32(sign | 0x7f800000u | (mant << 13));
    return bits_f32(sign | ((exp + 127 - 15) << 23) | (mant << 13));
}

uint16_t orc_f32_to_f16(float v)
{
    uint32_t x = f32_bits(v);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    int32_t exp = (int32_t)((x >> 23) & 0xff);
    uint32_t mant = x & 0x007fffffu;

    if (exp == 0xff) {
        uint16_t m = mant == 0 ? 0 : (uint16_t)((mant >> 13) | 1);
        return sign | 0x7c00 | m;
    }
    exp -= 127 - 15;
    if (exp >= 0x1f)
        return sign | 0x7c00;
    if (exp <= 0) {
        if (exp < -10)
            return sign;
        mant |= 0x00800000u;
        uint32_t shift = (uint32_t)(14 - exp);
        uint32_t half = 1u << (shift - 1);
        uint32_t m = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1);
        if (rem > half || (rem == half && (m & 1) == 1))
            m += 1;
        return sign | (uint16_t)m;
    }
    uint32_t half = 1u << 12;
    uint32_t m = mant >> 13;
    uint32_t rem = mant & 0x1fff;
    if (rem > half || (rem == half && (m & 1) == 1)) {
        m += 1;
        if (m == 0x400) {
            m = 0;
            exp += 1;
            if (exp >= 0x1f)
                return sign | 0x7c00;
        }
    }
    return sign | (uint16_t)((uint32_t)exp << 10) | (uint16_t)m;
}

/* ---- block encode: kv.rs:176-235 ---------------------------------------- */

/* Rust `f32::clamp` keeps NaN and `as i8` / `as u8` turn NaN into 0 and
 * saturate; both are spelled out so the corner cases match. */
static float clampf_keep_nan(float x, float lo, float hi)
{
    if (x < lo)
        return lo;
    if (x > hi)
        return hi;
    return x;
}

static int sat_cast_i(float x, int lo, int hi)
{
    if (x != x)
        return 0;
    if (x <= (float)lo)
        return lo;
    if (x >= (float)hi)
        return hi;
    return (int)x;
}

void orc_quantize_block(int dtype, const float *xs, uint8_t *out)
{
    if (dtype == ORC_Q8) {
        float amax = 0.0f;
        for (int j = 0; j < ORC_BLOCK; j++)
            amax = fmaxf(amax, fabsf(xs[j]));
        float d = amax / 127.0f;
        float id = d > 0.0f ? 1.0f / d : 0.0f;
        uint16_t hd = orc_f32_to_f16(d);
        out[0] = (uint8_t)(hd & 0xff);
        out[1] = (uint8_t)(hd >> 8);
        for (int j = 0; j < ORC_BLOCK; j++) {
            float r = clampf_keep_nan(roundf(xs[j] * id), -127.0f, 127.0f);
            out[2 + j] = (uint8_t)(int8_t)sat_cast_i(r, -128, 127);
        }
    } else {
        /* ggml q4_0: the scale carries the sign of the largest-magnitude value. */
        float vmax = 0.0f;
        for (int j = 0; j < ORC_BLOCK; j++)
            if (fabsf(xs[j]) > fabsf(vmax))
                vmax = xs[j];
        float d = -vmax / 8.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        uint16_t hd = orc_f32_to_f16(d);
        out[0] = (uint8_t)(hd & 0xff);
        out[1] = (uint8_t)(hd >> 8);
        uint8_t q[ORC_BLOCK];
        for (int j = 0; j < ORC_BLOCK; j++) {
            float r = clampf_keep_nan(roundf(xs[j] * id) + 8.0f, 0.0f, 15.0f);
            q[j] = (uint8_t)sat_cast_i(r, 0, 255);
        }
        for (int j = 0; j < ORC_BLOCK / 2; j++)
            out[2 + j] = (uint8_t)(q[j] | (q[j + ORC_BLOCK / 2] << 4));
    }
}

void orc_quantize(int dtype, const float *values, size_t n_values, uint8_t *out)
{
    size_t bb = orc_block_bytes(dtype);
    for (size_t b = 0; b < n_values / ORC_BLOCK; b++)
        orc_quantize_block(dtype, values + b * ORC_BLOCK, out + b * bb);
}

/* ---- block decode: kv.rs:238-290 ---------------------------------------- */

void orc_block_f32(int dtype, const uint8_t *src, float *out)
{
    float d = orc_f16_to_f32((uint16_t)(src[0] | (src[1] << 8)));
    if (dtype == ORC_Q8) {
        for (int j = 0; j < ORC_BLOCK; j++)
            out[j] = d * (float)(int8_t)src[2 + j];
    } else {
        for (int j = 0; j < ORC_BLOCK / 2; j++) {
            uint8_t byte = src[2 + j];
            out[j] = d * ((float)(byte & 0x0f) - 8.0f);
            out[j + ORC_BLOCK / 2] = d * ((float)(byte >> 4) - 8.0f);
        }
    }
}

void orc_dequantize(int dtype, const uint8_t *bytes, size_t n_bytes, float *out)
{
    size_t bb = orc_block_bytes(dtype);
    for (size_t b = 0; b < n_bytes / bb; b++)
        orc_block_f32(dtype, bytes + b * bb, out + b * ORC_BLOCK);
}

/* ---- bench filler: kv.rs:306-329 ---------------------------------------- */

static uint64_t xorshift_star(uint64_t *state)
{
    uint64_t x = *state;
    x ^= x >> 12;
    x ^= x << 25;
    x ^= x >> 27;
    *state = x;
    return x * 0x2545F4914F6CDD1DULL;
}

void orc_synthetic_blocks(int dtype, size_t n_blocks, uint64_t seed, uint8_t *out)
{
    size_t bb = orc_block_bytes(dtype);
    uint64_t s = seed | 1;
    for (size_t b = 0; b < n_blocks; b++) {
        size_t base = b * bb;
        float d = 0.01f + (float)(xorshift_star(&s) % 1000) * 0.00004f;
        uint16_t hd = orc_f32_to_f16(d);
        out[base] = (uint8_t)(hd & 0xff);
        out[base + 1] = (uint8_t)(hd >> 8);
        for (size_t j = 0; j < bb - 2; j++)
            out[base + 2 + j] = (uint8_t)(xorshift_star(&s) >> 24);
    }
}

/* ---- RNG: crates/hipml-core/src/rng.rs:9-50 ------------------------------ */

void orc_rng_new(orc_rng *r, uint64_t seed) { r->state = seed | 1; }

uint64_t orc_rng_next_u64(orc_rng *r) { return xorshift_star(&r->state); }

float orc_rng_uniform(orc_rng *r)
{
    return (float)(orc_rng_next_u64(r) >> 40) / (float)(1u << 24);
}

float orc_rng_normal(orc_rng *r)
{
    float u1 = fmaxf(orc_rng_uniform(r), 1e-7f);
    float u2 = orc_rng_uniform(r);
    const float tau = 6.28318530717958647692528676655900577f;
    return sqrtf(-2.0f * logf(u1)) * cosf(tau * u2);
}

void orc_rng_fill_normal(orc_rng *r, float *out, size_t n, float std)
{
    for (size_t i = 0; i < n; i++)
        out[i] = orc_rng_normal(r) * std;
}

void orc_rng_fill_uniform(orc_rng *r, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++)
        out[i] = orc_rng_uniform(r);
}

/* ---- elementwise: ops.rs:62-64, 354-360 ---------------------------------- */

void orc_sigmoid_f32(const float *x, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++)
        out[i] = 1.0f / (1.0f + expf(-x[i]));
}

void orc_q_gate_f32(const float *q, const float *gate, float *y, size_t n)
{
    for (size_t i = 0; i < n; i++)
        y[i] = q[i] * (1.0f / (1.0f + expf(-gate[i])));
}

/* ---- attention front end: ops.rs:178-187, 315-349 ------------------------------ */

/* ops.rs:181-187: mean of squares summed in index order (Rust's f32 `sum()` is a left fold),
 * scale = 1/sqrt(mean + eps), then the two multiplies x*scale*w left to right. */
void orc_rmsnorm_f32(const float *x, const float *w, float *y, size_t n, float eps)
{
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++)
        sum += x[i] * x[i];
    float mean_sq = sum / (float)n;
    float scale = 1.0f / sqrtf(mean_sq + eps);
    for (size_t i = 0; i < n; i++)
        y[i] = x[i] * scale * w[i];
}

/* ops.rs:337-349: every head row normalised with the shared weight row. */
void orc_head_rmsnorm_f32(const float *x, const float *w, float *y, size_t n_heads, size_t head_dim,
                          float eps)
{
    for (size_t h = 0; h < n_heads; h++)
        orc_rmsnorm_f32(x + h * head_dim, w, y + h * head_dim, head_dim, eps);
}

/* The summation order of the reference's GPU kernels (attn_front_f32.hip:79-103,
 * attn_chunk_f32.hip:68-81) at head_dim == block size: thread t holds x[t]^2 (its fma chain has
 * one link), then the shared-memory tree red[t] += red[t + off] for off = n/2 .. 1.  n must be a
 * power of two <= 256.  Everything else as orc_rmsnorm_f32. */
void orc_rmsnorm_tree_f32(const float *x, const float *w, float *y, size_t n, float eps)
{
    float red[256];
    for (size_t i = 0; i < n; i++)
        red[i] = x[i] * x[i];
    for (size_t off = n / 2; off > 0; off >>= 1)
        for (size_t t = 0; t < off; t++)
            red[t] += red[t + off];
    float mean_sq = red[0] / (float)n;
    float scale = 1.0f / sqrtf(mean_sq + eps);
    for (size_t i = 0; i < n; i++)
        y[i] = x[i] * scale * w[i];
}

/* ops.rs:315-330: joint projection [n_heads][2*head_dim] -> q [n_heads][head_dim], gate likewise. */
void orc_qg_split_f32(const float *qg, float *q, float *gate, size_t n_heads, size_t head_dim)
{
    for (size_t h = 0; h < n_heads; h++) {
        memcpy(q + h * head_dim, qg + h * 2 * head_dim, head_dim * sizeof(float));
        memcpy(gate + h * head_dim, qg + h * 2 * head_dim + head_dim, head_dim * sizeof(float));
    }
}

/* ---- RoPE: ops.rs:195-224, 260-309 --------------------------------------- */

static void rotate_pair(const float *x, float *y, size_t lo, size_t hi, size_t p, double freq)
{
    double ang = (double)p * freq;
    float sn = (float)sin(ang);
    float cs = (float)cos(ang);
    float x1 = x[lo];
    float x2 = x[hi];
    y[lo] = x1 * cs - x2 * sn;
    y[hi] = x1 * sn + x2 * cs;
}

void orc_rope_neox_f32(const float *x, float *y, size_t n_heads, size_t head_dim, size_t pos,
                       float theta_base)
{
    size_t half = head_dim / 2;
    if (y != x)
        memcpy(y, x, n_heads * head_dim * sizeof(float));
    for (size_t h = 0; h < n_heads; h++) {
        size_t base = h * head_dim;
        for (size_t i = 0; i < half; i++) {
            double freq = pow((double)theta_base, -2.0 * (double)i / (double)head_dim);
            rotate_pair(x, y, base + i, base + half + i, pos, freq);
        }
    }
}

void orc_rope_multi_f32(const float *x, float *y, size_t n_heads, size_t head_dim, size_t n_rot,
                        const size_t sections[4], const size_t pos[4], float theta_base)
{
    size_t half = n_rot / 2;
    size_t sect = sections[0] + sections[1] + sections[2] + sections[3];
    if (y != x)
        memcpy(y, x, n_heads * head_dim * sizeof(float));
    for (size_t h = 0; h < n_heads; h++) {
        size_t base = h * head_dim;
        for (size_t k = 0; k < half; k++) {
            size_t p;
            if (sect == 0) {
                p = pos[0];
            } else {
                size_t s = k % sect;
                if (s < sections[0])
                    p = pos[0];
                else if (s < sections[0] + sections[1])
                    p = pos[1];
                else if (s < sections[0] + sections[1] + sections[2])
                    p = pos[2];
                else
                    p = pos[3];
            }
            double freq = pow((double)theta_base, -2.0 * (double)k / (double)n_rot);
            rotate_pair(x, y, base + k, base + half + k, p, freq);
        }
    }
}

/* ---- f32 cache append: ops.rs:366-386 ------------------------------------ */

void orc_kv_append_f32(float *k_cache, float *v_cache, const float *k, const float *v, size_t off,
                       size_t width)
{
    memcpy(k_cache + off * width, k, width * sizeof(float));
    memcpy(v_cache + off * width, v, width * sizeof(float));
}

/* ---- two-pass causal attention, position-major f32 cache:
 *      crates/hipml-core/src/attention.rs:56-102 --------------------------- */

void orc_attn_causal_f32(const float *q, const float *k_cache, const float *v_cache,
                         size_t n_heads, size_t n_kv, size_t head_dim, size_t seq, float scale,
                         float *out)
{
    size_t width = n_kv * head_dim;
    size_t group = n_heads / n_kv;
    float *scores = (float *)malloc((seq ? seq : 1) * sizeof(float));
    memset(out, 0, n_heads * head_dim * sizeof(float));

    for (size_t h = 0; h < n_heads; h++) {
        size_t kvh = h / group;
        const float *qh = q + h * head_dim;
        float max = -INFINITY;
        for (size_t t = 0; t < seq; t++) {
            const float *kr = k_cache + t * width + kvh * head_dim;
            float dot = 0.0f;
            for (size_t d = 0; d < head_dim; d++)
                dot += qh[d] * kr[d];
            float s = dot * scale;
            scores[t] = s;
            max = fmaxf(max, s);
        }
        float sum = 0.0f;
        for (size_t t = 0; t < seq; t++) {
            float w = expf(scores[t] - max);
            scores[t] = w;
            sum += w;
        }
        float inv = 1.0f / sum;
        float *ob = out + h * head_dim;
        for (size_t t = 0; t < seq; t++) {
            float w = scores[t] * inv;
            const float *vr = v_cache + t * width + kvh * head_dim;
            for (size_t d = 0; d < head_dim; d++)
                ob[d] += w * vr[d];
        }
    }
    free(scores);
}

/* ---- two-pass decode attention, head-major f32 cache: ops.rs:535-588 ----- */

void orc_attn_decode_f32(const float *q, const float *k, const float *v, size_t n_heads,
                         size_t n_kv, size_t head_dim, size_t seq, float scale, float *out)
{
    size_t group = n_heads / n_kv;
    float *scores = (float *)malloc((seq ? seq : 1) * sizeof(float));
    memset(out, 0, n_heads * head_dim * sizeof(float));
    for (size_t h = 0; h < n_heads; h++) {
        size_t kvh = h / group;
        const float *qh = q + h * head_dim;
        size_t kbase = kvh * seq * head_dim;
        float max = -INFINITY;
        for (size_t row = 0; row < seq; row++) {
            const float *kr = k + kbase + row * head_dim;
            float dot = 0.0f;
            for (size_t d = 0; d < head_dim; d++)
                dot += qh[d] * kr[d];
            float s = dot * scale;
            scores[row] = s;
            max = fmaxf(max, s);
        }
        float sum = 0.0f;
        for (size_t row = 0; row < seq; row++) {
            float w = expf(scores[row] - max);
            scores[row] = w;
            sum += w;
        }
        float inv = 1.0f / sum;
        for (size_t row = 0; row < seq; row++) {
            float w = scores[row] * inv;
            const float *vr = v + kbase + row * head_dim;
            for (size_t d = 0; d < head_dim; d++)
                out[h * head_dim + d] += w * vr[d];
        }
    }
    free(scores);
}

/* ---- online-softmax decode over a quantized cache: ops.rs:449-518 -------- */

void orc_attn_decode_kv(const float *q, const uint8_t *k, const uint8_t *v, size_t n_heads,
                        size_t n_kv, size_t head_dim, size_t seq, size_t stride, float scale,
                        int dtype, float *out)
{
    size_t nb = head_dim / ORC_BLOCK;
    size_t bb = orc_block_bytes(dtype);
    size_t row = nb * bb;
    size_t group = n_heads / n_kv;
    float *acc = (float *)malloc(head_dim * sizeof(float));
    float blk[ORC_BLOCK];

    for (size_t h = 0; h < n_heads; h++) {
        size_t kvh = h / group;
        const float *qh = q + h * head_dim;
        size_t kbase = kvh * stride * row;
        for (size_t d = 0; d < head_dim; d++)
            acc[d] = 0.0f;
        float m = -INFINITY;
        float l = 0.0f;

        for (size_t pos = 0; pos < seq; pos++) {
            size_t at = kbase + pos * row;
            float dot = 0.0f;
            for (size_t c = 0; c < nb; c++) {
                orc_block_f32(dtype, k + at + c * bb, blk);
                const float *qc = qh + c * ORC_BLOCK;
                for (int j = 0; j < ORC_BLOCK; j++)
                    dot += qc[j] * blk[j];
            }
            float s = dot * scale;
            float m_new = fmaxf(m, s);
            float corr = expf(m - m_new);
            float p = expf(s - m_new);
            l = l * corr + p;
            m = m_new;
            for (size_t c = 0; c < nb; c++) {
                orc_block_f32(dtype, v + at + c * bb, blk);
                float *a = acc + c * ORC_BLOCK;
                for (int j = 0; j < ORC_BLOCK; j++)
                    a[j] = a[j] * corr + p * blk[j];
            }
        }
        float inv = 1.0f / l;
        for (size_t d = 0; d < head_dim; d++)
            out[h * head_dim + d] = acc[d] * inv;
    }
    free(acc);
}

/* ---- one token through the attention core: attention.rs:140-161 ---------- */

void orc_attn_core_token_f32(float *q, float *k, const float *v, const float *gate,
                             float *k_cache, float *v_cache, size_t n_ctx, size_t n_heads,
                             size_t n_kv, size_t head_dim, size_t n_rot,
                             const size_t sections[4], size_t pos, float theta_base, float *out)
{
    (void)n_ctx;
    size_t p[4] = { pos, pos, pos, pos };
    size_t width = n_kv * head_dim;
    orc_rope_multi_f32(q, q, n_heads, head_dim, n_rot, sections, p, theta_base);
    orc_rope_multi_f32(k, k, n_kv, head_dim, n_rot, sections, p, theta_base);
    orc_kv_append_f32(k_cache, v_cache, k, v, pos, width);
    float scale = 1.0f / sqrtf((float)head_dim);
    orc_attn_causal_f32(q, k_cache, v_cache, n_heads, n_kv, head_dim, pos + 1, scale, out);
    for (size_t i = 0; i < n_heads * head_dim; i++) {
        float g = 1.0f / (1.0f + expf(-gate[i]));
        out[i] *= g;
    }
}

/* ---- chunk-prefill expectation: hipml-cli/src/attn_chunk_parity.rs:127-210 */

void orc_attn_chunk_kv(const float *q, const uint8_t *k, const uint8_t *v, size_t n_heads,
                       size_t n_kv, size_t head_dim, size_t pos0, size_t tokens, size_t stride,
                       float scale, int dtype, const int32_t *rows, size_t n_rows, int n_threads,
                       float *out)
{
    size_t nb = head_dim / ORC_BLOCK;
    size_t bb = orc_block_bytes(dtype);
    size_t row = nb * bb;
    size_t width = n_kv * head_dim;
    size_t nhd = n_heads * head_dim;
    size_t live = pos0 + tokens;
    if (rows == NULL)
        n_rows = tokens;
    /* head-major quantized rows -> position-major f32, as the reference case does */
    float *kq = (float *)malloc(live * width * sizeof(float));
    float *vq = (float *)malloc(live * width * sizeof(float));
    for (size_t h = 0; h < n_kv; h++) {
        for (size_t p = 0; p < live; p++) {
            const uint8_t *ks = k + (h * stride + p) * row;
            const uint8_t *vs = v + (h * stride + p) * row;
            for (size_t c = 0; c < nb; c++) {
                orc_block_f32(dtype, ks + c * bb, kq + p * width + h * head_dim + c * ORC_BLOCK);
                orc_block_f32(dtype, vs + c * bb, vq + p * width + h * head_dim + c * ORC_BLOCK);
            }
        }
    }
    if (n_threads < 1)
        n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 1)
    for (size_t i = 0; i < n_rows; i++) {
        size_t t = rows ? (size_t)rows[i] : i;
        orc_attn_causal_f32(q + t * nhd, kq, vq, n_heads, n_kv, head_dim, pos0 + t + 1, scale,
                            out + i * nhd);
    }
    free(kq);
    free(vq);
}

/* ---- comparison: crates/hipml-core/src/parity.rs:44-80 ------------------- */

int orc_compare(const float *expected, const float *actual, size_t n, float abs_tol,
                float rel_tol, float *max_abs_out, float *max_rel_out)
{
    float max_abs = 0.0f;
    float max_rel = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float abs = fabsf(expected[i] - actual[i]);
        float denom = fmaxf(fabsf(expected[i]), 1e-12f);
        max_abs = fmaxf(max_abs, abs);
        max_rel = fmaxf(max_rel, abs / denom);
    }
    if (max_abs_out)
        *max_abs_out = max_abs;
    if (max_rel_out)
        *max_rel_out = max_rel;
    return (max_abs <= abs_tol || max_rel <= rel_tol) ? 1 : 0;
}

/* ---- Q8_0 weight matrices: quant.rs:433-443, 653-675, 785-796, 846-854; ops.rs:102-104, 136-176 -- */

void orc_dequant_q8_0(const uint8_t *block, float *out)
{
    const float d = orc_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
    for (int i = 0; i < 32; i++)
        out[i] = d * (float)(int8_t)block[2 + i];
}

void orc_gemv_q8_0(const uint8_t *w, const float *x, size_t m, size_t k, float *y)
{
    const size_t nb = k / 32, row_bytes = nb * 34;
    float tmp[32];
    for (size_t row = 0; row < m; row++) {
        const uint8_t *rd = w + row * row_bytes;
        float acc = 0.0f;
        for (size_t b = 0; b < nb; b++) {
            orc_dequant_q8_0(rd + b * 34, tmp);
            const float *xb = x + b * 32;
            for (int l = 0; l < 32; l++)
                acc += tmp[l] * xb[l];
        }
        y[row] = acc;
    }
}

void orc_gemm_q8_0(const uint8_t *w, const float *x, size_t tokens, size_t m, size_t k,
                   int n_threads, float *y)
{
    const size_t nb = k / 32, row_bytes = nb * 34;
#pragma omp parallel for schedule(static) num_threads(n_threads > 1 ? n_threads : 1)
    for (long r = 0; r < (long)m; r++) {
        float *row = (float *)malloc(k * sizeof(float));
        const uint8_t *rd = w + (size_t)r * row_bytes;
        for (size_t b = 0; b < nb; b++)
            orc_dequant_q8_0(rd + b * 34, row + b * 32);
        for (size_t t = 0; t < tokens; t++) {
            const float *xr = x + t * k;
            float acc = 0.0f;
            for (size_t j = 0; j < k; j++)
                acc += row[j] * xr[j];
            y[t * m + (size_t)r] = acc;
        }
        free(row);
    }
}

void orc_random_q8_0_bytes(orc_rng *r, size_t nblocks, uint8_t *out)
{
    for (size_t blk = 0; blk < nblocks; blk++) {
        uint8_t *b = out + blk * 34;
        size_t i = 0;
        while (i + 8 <= 34) {
            uint64_t v = orc_rng_next_u64(r);
            for (int j = 0; j < 8; j++)
                b[i + j] = (uint8_t)(v >> (8 * j));
            i += 8;
        }
        uint64_t tail = orc_rng_next_u64(r);
        for (int j = 0; i + j < 34; j++)
            b[i + j] = (uint8_t)(tail >> (8 * j));
        b[0] = 0x00;
        b[1] = 0x14;
    }
}
