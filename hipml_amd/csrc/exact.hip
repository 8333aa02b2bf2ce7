// Bit-exact and elementwise kernels of the attention path for gfx950:
// q8_0 KV quantize-and-append, M-RoPE, sigmoid output gate.
//
// This translation unit is compiled with -ffp-contract=off: the CPU definitions
// these kernels must reproduce bit for bit evaluate x1*c - x2*s and x*id with
// separately rounded multiplies (crates/hipml-core/src/ops.rs:296-305,
// crates/hipml-core/src/kv.rs:191-200 in the reference).

#include "common.h"

#include <hip/hip_fp16.h>

namespace hipml {

// ---- q8_0 quantize + append ---------------------------------------------------
//
// One workgroup per (kv head, unit); thread t owns value t of the head row.  A
// wave64 holds two 32-value blocks, so the absolute-maximum butterfly stays
// inside each 32-lane half (xor masks 16..1 never cross bit 5).
//
// unit u reads source row (src0 + u) of a position-major f32 [.][n_kv*head_dim]
// buffer and writes cache position pos[u*pos_stride] (or start + u when pos is
// null) of the cache at base + u*slot_bytes.

__device__ __forceinline__ float half_wave_amax(float x)
{
    float m = fabsf(x);
#pragma unroll
    for (int bit = 16; bit > 0; bit >>= 1)
        m = fmaxf(m, __shfl_xor(m, bit));
    return m;
}

__device__ __forceinline__ void q8_encode_store(float x, uint8_t *dst_block, int lane32)
{
    const float amax = half_wave_amax(x);
    const float d = amax / 127.0f;                    // IEEE division
    const float id = d > 0.0f ? 1.0f / d : 0.0f;
    const float t = roundf(x * id);                   // half away from zero
    // NaN (0 * inf when d is subnormal) encodes as 0, like Rust's `as i8`.
    const float c = fminf(127.0f, fmaxf(-127.0f, t));
    const int q = (t != t) ? 0 : (int)c;
    if (lane32 == 0)
        *reinterpret_cast<__half *>(dst_block) = __float2half_rn(d);
    dst_block[2 + lane32] = (uint8_t)(int8_t)q;
}

__global__ void __launch_bounds__(256) kv_encode_q8_kernel(
    const float *__restrict__ k, const float *__restrict__ v, uint8_t *__restrict__ kc,
    uint8_t *__restrict__ vc, int n_kv, int head_dim, int stride, const int32_t *__restrict__ pos,
    int pos_stride, size_t slot_bytes, int start, int src0)
{
    const int h = blockIdx.x;
    const int u = blockIdx.y;
    const int t = threadIdx.x;
    if (t >= head_dim)
        return;
    const int chunk = t >> 5;
    const int lane32 = t & 31;
    const int nchunk = head_dim >> 5;
    const int p = pos ? pos[(size_t)u * pos_stride] : start + u;
    const size_t src = ((size_t)(src0 + u) * n_kv + h) * head_dim + t;
    const size_t off = (size_t)u * slot_bytes +
                       (((size_t)h * stride + p) * nchunk + chunk) * kQ8BlockBytes;
    q8_encode_store(k[src], kc + off, lane32);
    q8_encode_store(v[src], vc + off, lane32);
}

// ---- q4_0 quantize + append (crates/hipml-core/src/kv.rs:201-218) ---------------------------
//
// The scale takes the sign of the value of largest magnitude, the FIRST such value when several
// tie (the reference folds left with a strict `>`; NaN never wins that comparison); d = -vmax/8,
// id = 1/d or 0, q = clamp(round(x*id) + 8, 0, 15); byte j of the block holds q[j] in its low and
// q[j+16] in its high nibble.  Same thread layout as the q8_0 kernel: 32 lanes per block.

__device__ __forceinline__ float half_wave_vmax(float x, int lane32)
{
    float mag = fabsf(x);
    if (!(mag == mag))
        mag = -1.0f; // NaN: below every real magnitude, like a failed `>`
    float val = x;
    int idx = lane32;
#pragma unroll
    for (int bit = 16; bit > 0; bit >>= 1) {
        const float om = __shfl_xor(mag, bit);
        const float ov = __shfl_xor(val, bit);
        const int oi = __shfl_xor(idx, bit);
        const bool take = om > mag || (om == mag && oi < idx);
        mag = take ? om : mag;
        val = take ? ov : val;
        idx = take ? oi : idx;
    }
    return mag > 0.0f ? val : 0.0f; // nothing beat the fold's initial +0
}

__device__ __forceinline__ void q4_encode_store(float x, uint8_t *dst_block, int lane32)
{
    const float vmax = half_wave_vmax(x, lane32);
    const float d = -vmax / 8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float t = roundf(x * id) + 8.0f;
    const float c = fminf(15.0f, fmaxf(0.0f, t));
    const int q = (t != t) ? 0 : (int)c; // NaN encodes as 0, like Rust's `as u8`
    const int hi = __shfl_xor(q, 16);
    if (lane32 == 0)
        *reinterpret_cast<__half *>(dst_block) = __float2half_rn(d);
    if (lane32 < 16)
        dst_block[2 + lane32] = (uint8_t)(q | (hi << 4));
}

__global__ void __launch_bounds__(256) kv_encode_q4_kernel(
    const float *__restrict__ k, const float *__restrict__ v, uint8_t *__restrict__ kc,
    uint8_t *__restrict__ vc, int n_kv, int head_dim, int stride, const int32_t *__restrict__ pos,
    int pos_stride, size_t slot_bytes, int start, int src0)
{
    const int h = blockIdx.x;
    const int u = blockIdx.y;
    const int t = threadIdx.x;
    if (t >= head_dim)
        return;
    const int chunk = t >> 5;
    const int lane32 = t & 31;
    const int nchunk = head_dim >> 5;
    const int p = pos ? pos[(size_t)u * pos_stride] : start + u;
    const size_t src = ((size_t)(src0 + u) * n_kv + h) * head_dim + t;
    const size_t off = (size_t)u * slot_bytes +
                       (((size_t)h * stride + p) * nchunk + chunk) * kQ4BlockBytes;
    q4_encode_store(k[src], kc + off, lane32);
    q4_encode_store(v[src], vc + off, lane32);
}

int launch_kv_encode(hipStream_t st, int q4, const float *k, const float *v, uint8_t *kc, uint8_t *vc,
                     int n_kv, int head_dim, int stride, const int32_t *pos, int pos_stride,
                     size_t slot_bytes, int units, int start, int src0, int /*rows*/)
{
    if (units == 0)
        return 0;
    const int block = head_dim < 64 ? 64 : head_dim;
    // grid.y is limited to 65535: walk long chunks in slices.
    for (int u0 = 0; u0 < units; u0 += 32768) {
        const int n = units - u0 < 32768 ? units - u0 : 32768;
        HIPML_LAUNCH(q4 ? kv_encode_q4_kernel : kv_encode_q8_kernel, dim3(n_kv, n, 1),
                           dim3(block, 1, 1), 0, st, k, v, kc + (size_t)u0 * slot_bytes,
                           vc + (size_t)u0 * slot_bytes, n_kv, head_dim, stride,
                           pos ? pos + (size_t)u0 * pos_stride : nullptr, pos_stride, slot_bytes,
                           start + u0, src0 + u0);
        int rc = launched(q4 ? "kv_encode_q4" : "kv_encode_q8");
        if (rc)
            return rc;
    }
    return 0;
}

// ---- RoPE ----------------------------------------------------------------------
//
// NeoX pair k is (k, k + n_rot/2); the angle of pair k at position p is
// p * theta^(-2k/n_rot).  cos/sin come from the host-built f32 table.  A position outside the
// table is an error: the entry points refuse it where the host knows the positions, and where they
// live in device memory the rotated values come out as NaN.  Only when the caller has opted in
// (hipml_rope_allow_device_angles) such a position is served by f64 pow/sincos on the device, within
// one f32 ulp of the table but not bit-identical to it.  The kernels take the table's row count with
// a sign: tab_rows >= 0 allows the device angles, -(rows) - 1 does not.

__device__ __forceinline__ int rope_rows(int tab_rows) { return tab_rows >= 0 ? tab_rows : -(tab_rows + 1); }

__device__ __forceinline__ void rope_cs(const float *__restrict__ tab, int tab_rows, int half,
                                        int k, int p, int n_rot, float theta, float &cs, float &sn)
{
    if (tab != nullptr && p >= 0 && p < rope_rows(tab_rows)) {
        const float2 e = reinterpret_cast<const float2 *>(tab)[(size_t)p * half + k];
        cs = e.x;
        sn = e.y;
    } else if (tab_rows < 0) {
        cs = sn = __builtin_nanf("");
    } else {
        const double freq = pow((double)theta, -2.0 * (double)k / (double)n_rot);
        double s, c;
        sincos((double)p * freq, &s, &c);
        cs = (float)c;
        sn = (float)s;
    }
}

// grid (n_heads, rows); 64 threads.  Row r takes its four position ids from
// pos[r*pos_stride .. +3] (sections pick one per pair), or all four equal to
// pos[r*pos_stride] when `text` is set.
__global__ void __launch_bounds__(64) mrope_kernel(
    const float *x, float *y, int n_heads, int head_dim, int n_rot, int s0, int s1, int s2, int s3,
    const int32_t *__restrict__ pos, int pos_stride, int text, float theta,
    const float *__restrict__ tab, int tab_rows)
{
    const int h = blockIdx.x;
    const int r = blockIdx.y;
    const int half = n_rot >> 1;
    const int sect = s0 + s1 + s2 + s3;
    const int32_t *pr = pos + (size_t)r * pos_stride;
    const size_t base = ((size_t)r * n_heads + h) * (size_t)head_dim;
    for (int k = threadIdx.x; k < half; k += blockDim.x) {
        int p = pr[0];
        if (!text && sect > 0) {
            const int s = k % sect;
            if (s < s0)
                p = pr[0];
            else if (s < s0 + s1)
                p = pr[1];
            else if (s < s0 + s1 + s2)
                p = pr[2];
            else
                p = pr[3];
        }
        float cs, sn;
        rope_cs(tab, tab_rows, half, k, p, n_rot, theta, cs, sn);
        const float x1 = x[base + k];
        const float x2 = x[base + half + k];
        y[base + k] = x1 * cs - x2 * sn;
        y[base + half + k] = x1 * sn + x2 * cs;
    }
    // channels >= n_rot pass through
    if (y != x) {
        for (int d = n_rot + threadIdx.x; d < head_dim; d += blockDim.x)
            y[base + d] = x[base + d];
    }
}

// 256 threads = 8 head rows x 32 lanes; head row r of the chunk = (token r / (n_head + n_kv),
// q head or k head); token t rotates at pos0 + t.
__global__ void __launch_bounds__(256) rope_chunk_kernel(
    float *__restrict__ q, float *__restrict__ kx, int n_head, int n_kv, int head_dim, int n_rot,
    float theta, int pos0, int tokens, const float *__restrict__ tab, int tab_rows)
{
    const int per = n_head + n_kv;
    const long long r = (long long)blockIdx.x * 8 + (threadIdx.x >> 5);
    if (r >= (long long)tokens * per)
        return;
    const int t = (int)(r / per);
    const int h = (int)(r - (long long)t * per);
    const int half = n_rot >> 1;
    const int p = pos0 + t;
    float *row = h < n_head ? q + ((size_t)t * n_head + h) * head_dim
                            : kx + ((size_t)t * n_kv + (h - n_head)) * head_dim;
    for (int k = threadIdx.x & 31; k < half; k += 32) {
        float cs, sn;
        rope_cs(tab, tab_rows, half, k, p, n_rot, theta, cs, sn);
        const float x1 = row[k];
        const float x2 = row[half + k];
        row[k] = x1 * cs - x2 * sn;
        row[half + k] = x1 * sn + x2 * cs;
    }
}

static const float *table_for(const RopeTable &tab, float theta, int n_rot, int *rows)
{
    if (tab.dev != nullptr && tab.theta == theta && tab.n_rot == n_rot) {
        *rows = tab.device_angles ? tab.max_pos : -tab.max_pos - 1;
        return tab.dev;
    }
    *rows = 0;
    return nullptr;
}

int launch_mrope(hipStream_t st, const float *x, float *y, int n_heads, int head_dim, int n_rot,
                 int s0, int s1, int s2, int s3, const int32_t *pos, int pos_stride, int rows,
                 float theta, const RopeTable &tab)
{
    int tab_rows = 0;
    const float *t = table_for(tab, theta, n_rot, &tab_rows);
    const int text = pos_stride != 0 ? 1 : 0; // batched rows carry (pos, seq) pairs: text only
    for (int r0 = 0; r0 < rows; r0 += 32768) {
        const int n = rows - r0 < 32768 ? rows - r0 : 32768;
        const size_t off = (size_t)r0 * n_heads * head_dim;
        HIPML_LAUNCH(mrope_kernel, dim3(n_heads, n, 1), dim3(64, 1, 1), 0, st, x + off,
                           y + off, n_heads, head_dim, n_rot, s0, s1, s2, s3,
                           pos + (size_t)r0 * pos_stride, pos_stride, text, theta, t, tab_rows);
        int rc = launched("mrope_f32");
        if (rc)
            return rc;
    }
    return 0;
}

int launch_rope_chunk(hipStream_t st, float *q, float *k, int n_head, int n_kv, int head_dim,
                      int n_rot, float theta, int pos0, int tokens, const RopeTable &tab)
{
    int tab_rows = 0;
    const float *t = table_for(tab, theta, n_rot, &tab_rows);
    const int slab = 1 << 20; // tokens per launch: keeps the row count inside the grid limit
    for (int t0 = 0; t0 < tokens; t0 += slab) {
        const int n = tokens - t0 < slab ? tokens - t0 : slab;
        const long long rows = (long long)n * (n_head + n_kv);
        HIPML_LAUNCH(rope_chunk_kernel, dim3((unsigned)((rows + 7) / 8), 1, 1), dim3(256, 1, 1), 0,
                           st, q + (size_t)t0 * n_head * head_dim, k + (size_t)t0 * n_kv * head_dim,
                           n_head, n_kv, head_dim, n_rot, theta, pos0 + t0, n, t, tab_rows);
        int rc = launched("rope_chunk_f32");
        if (rc)
            return rc;
    }
    return 0;
}

// A block of 32 values held four per lane by 8 neighbouring lanes (value 4 l8 + j in component j):
// the same quantizers as above (the maximum is exact whatever the order it is taken in; the q4_0
// winner is the first of the largest, by index), with 16-bit stores of the packed bytes.
typedef float float4e __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void q8_encode_store4(const float4e x, uint8_t *dst_block, int l8)
{
    float m = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
#pragma unroll
    for (int bit = 4; bit > 0; bit >>= 1)
        m = fmaxf(m, __shfl_xor(m, bit));
    const float d = m / 127.0f;
    const float id = d > 0.0f ? 1.0f / d : 0.0f;
    uint32_t pk = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float t = roundf(x[j] * id);
        const float c = fminf(127.0f, fmaxf(-127.0f, t));
        const int q = (t != t) ? 0 : (int)c;
        pk |= (uint32_t)(uint8_t)(int8_t)q << (8 * j);
    }
    if (l8 == 0)
        *reinterpret_cast<__half *>(dst_block) = __float2half_rn(d);
    uint16_t *p16 = reinterpret_cast<uint16_t *>(dst_block + 2 + 4 * l8);
    p16[0] = (uint16_t)pk;
    p16[1] = (uint16_t)(pk >> 16);
}

__device__ __forceinline__ void q4_encode_store4(const float4e x, uint8_t *dst_block, int l8)
{
    // the value of largest magnitude, the first one on a tie; NaN never wins
    float mag = -2.0f, val = 0.0f;
    int idx = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float mj = fabsf(x[j]);
        if (!(mj == mj))
            mj = -1.0f;
        if (mj > mag) {
            mag = mj;
            val = x[j];
            idx = 4 * l8 + j;
        }
    }
#pragma unroll
    for (int bit = 4; bit > 0; bit >>= 1) {
        const float om = __shfl_xor(mag, bit);
        const float ov = __shfl_xor(val, bit);
        const int oi = __shfl_xor(idx, bit);
        const bool take = om > mag || (om == mag && oi < idx);
        mag = take ? om : mag;
        val = take ? ov : val;
        idx = take ? oi : idx;
    }
    const float vmax = mag > 0.0f ? val : 0.0f;
    const float d = -vmax / 8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t pk = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float t = roundf(x[j] * id) + 8.0f;
        const float c = fminf(15.0f, fmaxf(0.0f, t));
        const int q = (t != t) ? 0 : (int)c;
        const int hi = __shfl_xor(q, 4); // value 16 further on: four lanes up, same component
        pk |= (uint32_t)(q | (hi << 4)) << (8 * j);
    }
    if (l8 == 0)
        *reinterpret_cast<__half *>(dst_block) = __float2half_rn(d);
    if (l8 < 4) {
        uint16_t *p16 = reinterpret_cast<uint16_t *>(dst_block + 2 + 4 * l8);
        p16[0] = (uint16_t)pk;
        p16[1] = (uint16_t)(pk >> 16);
    }
}

// RoPE of a chunk and the append of its K/V rows in one launch, four values per lane so that the whole
// chunk is one round of workgroups (with a value per lane the launch was two and a half rounds, each a
// memory round trip long).  The first `q_blocks` workgroups rotate 32 query head rows each: 8 lanes
// per row, lane l8 holds x1 = row[4 l8 ..] and x2 = row[32 + 4 l8 ..] of the 32 pairs.  The others
// take four (token, kv head) units each, one wave per unit: lane l holds values 4 l .. 4 l + 3 of the
// K row and of the V row; the pair partners of the rotated channels (lanes 0-7 and 8-15) meet through
// a lane exchange; the rotated row is written back and both rows are quantized, a block of 32 values
// being 8 neighbouring lanes.  The expressions of rope_chunk_kernel and of the append kernels, so the
// same bits as the two separate launches.  head_dim 256, n_rot 64 (checked by the caller).
constexpr int kRecRowsPerBlock = 32; // query rows per workgroup
constexpr int kRecUnitsPerBlock = 4; // (token, kv head) units per workgroup
template <bool Q4>
__global__ void __launch_bounds__(256) rope_encode_chunk_kernel(
    float *__restrict__ q, float *__restrict__ kx, const float *__restrict__ vx, uint8_t *__restrict__ kc,
    uint8_t *__restrict__ vc, int n_head, int n_kv, int n_rot, float theta, int pos0, int tokens,
    int stride, int q_blocks, const float *__restrict__ tab, int tab_rows)
{
    const int half = n_rot >> 1; // 32
    // cos/sin of pairs 4 g .. 4 g + 3 at position p
    auto cos_sin = [&](int g, int p, float (&cs)[4], float (&sn)[4]) {
        if (tab != nullptr && p >= 0 && p < rope_rows(tab_rows)) {
            const float4e *e = reinterpret_cast<const float4e *>(tab + ((size_t)p * half + 4 * g) * 2);
            const float4e c0 = e[0], c1 = e[1];
            cs[0] = c0[0], sn[0] = c0[1], cs[1] = c0[2], sn[1] = c0[3];
            cs[2] = c1[0], sn[2] = c1[1], cs[3] = c1[2], sn[3] = c1[3];
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                rope_cs(tab, tab_rows, half, 4 * g + j, p, n_rot, theta, cs[j], sn[j]);
        }
    };
    if ((int)blockIdx.x < q_blocks) {
        const long long r = (long long)blockIdx.x * kRecRowsPerBlock + (threadIdx.x >> 3);
        if (r >= (long long)tokens * n_head)
            return;
        const int l8 = threadIdx.x & 7;
        const int t = (int)(r / n_head);
        float *row = q + (size_t)r * kHeadDim;
        const float4e x1 = *reinterpret_cast<const float4e *>(row + 4 * l8);
        const float4e x2 = *reinterpret_cast<const float4e *>(row + half + 4 * l8);
        float cs[4], sn[4];
        cos_sin(l8, pos0 + t, cs, sn);
        float4e y1, y2;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            y1[j] = x1[j] * cs[j] - x2[j] * sn[j];
            y2[j] = x1[j] * sn[j] + x2[j] * cs[j];
        }
        *reinterpret_cast<float4e *>(row + 4 * l8) = y1;
        *reinterpret_cast<float4e *>(row + half + 4 * l8) = y2;
        return;
    }
    const int u = ((int)blockIdx.x - q_blocks) * kRecUnitsPerBlock + (threadIdx.x >> 6); // (token, kv head)
    if (u >= tokens * n_kv)
        return; // a whole wave: nothing below crosses waves
    const int tok = u / n_kv, h = u - tok * n_kv;
    const int lane = threadIdx.x & 63, l8 = lane & 7;
    float *krow = kx + (size_t)u * kHeadDim;
    float4e xk = *reinterpret_cast<const float4e *>(krow + 4 * lane);
    const float4e xv = *reinterpret_cast<const float4e *>(vx + (size_t)u * kHeadDim + 4 * lane);
    float cs[4] = {1, 1, 1, 1}, sn[4] = {0, 0, 0, 0};
    if (lane < 16)
        cos_sin(l8, pos0 + tok, cs, sn);
    float4e other;
#pragma unroll
    for (int j = 0; j < 4; j++)
        other[j] = __shfl_xor(xk[j], 8); // lanes 0-7 hold x1 of the pairs, lanes 8-15 their x2
    if (lane < 16) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            xk[j] = lane < 8 ? xk[j] * cs[j] - other[j] * sn[j] : other[j] * sn[j] + xk[j] * cs[j];
        *reinterpret_cast<float4e *>(krow + 4 * lane) = xk;
    }
    const size_t blk = ((size_t)h * stride + (pos0 + tok)) * (kHeadDim / 32) + (lane >> 3);
    if (Q4) {
        q4_encode_store4(xk, kc + blk * kQ4BlockBytes, l8);
        q4_encode_store4(xv, vc + blk * kQ4BlockBytes, l8);
    } else {
        q8_encode_store4(xk, kc + blk * kQ8BlockBytes, l8);
        q8_encode_store4(xv, vc + blk * kQ8BlockBytes, l8);
    }
}

int launch_rope_encode_chunk(hipStream_t st, int q4, float *q, float *k, const float *v, uint8_t *kc,
                             uint8_t *vc, int n_head, int n_kv, int n_rot, float theta, int pos0,
                             int tokens, int stride, const RopeTable &tab)
{
    int tab_rows = 0;
    const float *t = table_for(tab, theta, n_rot, &tab_rows);
    const int slab = 1 << 18; // tokens per launch: keeps the grid inside 2^31 workgroups
    for (int t0 = 0; t0 < tokens; t0 += slab) {
        const int n = tokens - t0 < slab ? tokens - t0 : slab;
        // (q == nullptr: the query rows are rotated elsewhere, e.g. where the attention kernel loads them)
        const int q_blocks = q == nullptr ? 0 : (int)(((long long)n * n_head + kRecRowsPerBlock - 1) / kRecRowsPerBlock);
        const dim3 grid((unsigned)(q_blocks + (n * n_kv + kRecUnitsPerBlock - 1) / kRecUnitsPerBlock), 1, 1);
        float *qq = q == nullptr ? nullptr : q + (size_t)t0 * n_head * kHeadDim;
        float *kk = k + (size_t)t0 * n_kv * kHeadDim;
        const float *vv = v + (size_t)t0 * n_kv * kHeadDim;
        if (q4)
            HIPML_LAUNCH(rope_encode_chunk_kernel<true>, grid, dim3(256, 1, 1), 0, st, qq, kk, vv, kc, vc,
                               n_head, n_kv, n_rot, theta, pos0 + t0, n, stride, q_blocks, t, tab_rows);
        else
            HIPML_LAUNCH(rope_encode_chunk_kernel<false>, grid, dim3(256, 1, 1), 0, st, qq, kk, vv, kc, vc,
                               n_head, n_kv, n_rot, theta, pos0 + t0, n, stride, q_blocks, t, tab_rows);
        int rc = launched("rope_encode_chunk");
        if (rc)
            return rc;
    }
    return 0;
}

// ---- attention front end ------------------------------------------------------------
//
// q|gate split, per-head RMS norm of q and k, M-RoPE of both, one wave per (row, head):
// the reference's attn_front_f32 (crates/hipml-kernels/kernels/attn_front_f32.hip:34-135, one
// token) and qg_split_chunk_f32 + norm_rope_chunk_f32 (attn_chunk_f32.hip:22-98, a chunk of rows).
// The arithmetic is theirs, operation for operation, at head_dim 256: the sum of squares is
// one square per element folded by the halving tree red[t] += red[t + off], off = 128 .. 1 (a
// lane holds elements l, l+64, l+128, l+192, so two levels are in-lane adds and six are lane
// exchanges; IEEE addition commutes, so every lane ends with red[0]); mean = sum / 256;
// scale = 1 / sqrtf(mean + eps) with the correctly rounded divide and square root; the value is
// (x * scale) * w; the rotation reads cos/sin as the other RoPE kernels here do.
// grid: ceil((n_heads + n_kv) * rows / 4) workgroups of 4 waves.  `pos` (device int32[4]) gives
// the four M-RoPE position ids of a single row; when it is null, row t rotates at pos0 + t.
// Per-row positions of a batch of sequences, and what the append half of a fused launch needs.
struct FrontAppend {
    const int32_t *rowpos; // non-null: row r belongs to sequence r and sits at text position
                           // rowpos[2 r] (device int32 [rows][2] = position, live length)
    size_t slot_bytes;     // with rowpos: sequence r's cache starts r * slot_bytes into kc / vc
    const float *v;        // [rows][n_kv][256]
    uint8_t *kc, *vc;      // caches
    const int32_t *step;   // row 0 goes to position step[0]; null: row r goes to start + r (or rowpos)
    int start, stride;
};

// ENC: 0 = front end only, 1 = also quantize the finished K row and the V row to q8_0 and append
// them, 2 = the same to q4_0 -- the K wave keeps its row in registers (element lane + 64 j in slot
// j, so a half-wave holds one block of 32, as the append kernels' 32-lane groups do) and n_kv more
// waves per row take the V rows.  Same expressions on the same values: the bits of the two launches.
template <int ENC>
__global__ void __launch_bounds__(256) front_kernel(
    const float *__restrict__ qg, float *__restrict__ q, float *__restrict__ gate, float *k,
    const float *__restrict__ qw, const float *__restrict__ kw, int n_heads, int n_kv, int n_rot,
    int s0, int s1, int s2, int s3, const int32_t *__restrict__ pos, int pos0, int rows, float theta,
    float eps, const float *__restrict__ tab, int tab_rows, const FrontAppend ap)
{
    __shared__ float buf[4][kHeadDim];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int per_row = n_heads + n_kv;
    const int idx = blockIdx.x * 4 + wave;
    const int nfront = per_row * rows;
    if (idx >= nfront + (ENC ? n_kv * rows : 0))
        return; // no workgroup-wide barrier below: waves are independent
    const int lane32 = lane & 31;
    if (ENC && idx >= nfront) {
        // a V row: quantize and append
        const int u = idx - nfront;
        const int row = u / n_kv, h = u - row * n_kv;
        const int p = ap.step ? ap.step[0] : ap.rowpos ? ap.rowpos[2 * row] : ap.start + row;
        uint8_t *vc = ap.vc + (ap.rowpos ? (size_t)row * ap.slot_bytes : 0);
        const float *src = ap.v + (size_t)u * kHeadDim;
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            x[j] = src[lane + 64 * j];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const size_t blk = ((size_t)h * ap.stride + p) * (kHeadDim / 32) + 2 * j + (lane >> 5);
            if (ENC == 2)
                q4_encode_store(x[j], vc + blk * kQ4BlockBytes, lane32);
            else
                q8_encode_store(x[j], vc + blk * kQ8BlockBytes, lane32);
        }
        return;
    }
    const int row = idx / per_row;
    const int hb = idx - row * per_row;
    const bool is_q = hb < n_heads;
    const int h = is_q ? hb : hb - n_heads;
    const float *src = is_q ? qg + ((size_t)row * n_heads + h) * (2 * kHeadDim)
                            : k + ((size_t)row * n_kv + h) * kHeadDim;
    float *dst = is_q ? q + ((size_t)row * n_heads + h) * kHeadDim
                      : k + ((size_t)row * n_kv + h) * kHeadDim;
    const float *w = is_q ? qw : kw;

    // everything this wave will need from memory is asked for here: the row, the gate half, the norm
    // weights and the rotation's cos/sin (the position does not depend on the data)
    float x[4], wv[4], g[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
        x[j] = src[lane + 64 * j];
#pragma unroll
    for (int j = 0; j < 4; j++)
        wv[j] = w[lane + 64 * j];
    if (is_q) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            g[j] = src[kHeadDim + lane + 64 * j];
    }
    const int half = n_rot >> 1;
    const int sect = s0 + s1 + s2 + s3;
    float cs[4], sn[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int e = lane + 64 * j;
        cs[j] = 1.0f;
        sn[j] = 0.0f;
        if (e < n_rot) {
            const int c = e < half ? e : e - half;
            int p = pos ? pos[0] : ap.rowpos ? ap.rowpos[2 * row] : pos0 + row;
            if (pos && sect > 0) {
                const int sc = c % sect;
                if (sc < s0)
                    p = pos[0];
                else if (sc < s0 + s1)
                    p = pos[1];
                else if (sc < s0 + s1 + s2)
                    p = pos[2];
                else
                    p = pos[3];
            }
            rope_cs(tab, tab_rows, half, c, p, n_rot, theta, cs[j], sn[j]);
        }
    }
    if (is_q) {
        float *gd = gate + ((size_t)row * n_heads + h) * kHeadDim;
#pragma unroll
        for (int j = 0; j < 4; j++)
            gd[lane + 64 * j] = g[j];
    }
    const float a0 = x[0] * x[0] + x[2] * x[2]; // off = 128
    const float a1 = x[1] * x[1] + x[3] * x[3];
    float sum = a0 + a1;                        // off = 64
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        sum += __shfl_xor(sum, off);
    const float mean_sq = sum / (float)kHeadDim;
    const float scale = 1.0f / sqrtf(mean_sq + eps);
#pragma unroll
    for (int j = 0; j < 4; j++)
        buf[wave][lane + 64 * j] = x[j] * scale * wv[j];
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    // element e = lane + 64 j: rotated with its partner when e < n_rot (the first half of the pairs
    // takes x1 c - x2 s, the second x1 s + x2 c), passed through otherwise
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int e = lane + 64 * j;
        float out = buf[wave][e];
        if (e < n_rot) {
            const bool first = e < half;
            const int c = first ? e : e - half;
            const float x1 = buf[wave][c];
            const float x2 = buf[wave][c + half];
            out = first ? x1 * cs[j] - x2 * sn[j] : x1 * sn[j] + x2 * cs[j];
        }
        dst[e] = out;
        x[j] = out;
    }
    if (ENC && !is_q) {
        const int p = ap.step ? ap.step[0] : ap.rowpos ? ap.rowpos[2 * row] : ap.start + row;
        uint8_t *kc = ap.kc + (ap.rowpos ? (size_t)row * ap.slot_bytes : 0);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const size_t blk = ((size_t)h * ap.stride + p) * (kHeadDim / 32) + 2 * j + (lane >> 5);
            if (ENC == 2)
                q4_encode_store(x[j], kc + blk * kQ4BlockBytes, lane32);
            else
                q8_encode_store(x[j], kc + blk * kQ8BlockBytes, lane32);
        }
    }
}

// enc: -1 = front end only (v, kc, vc unused), 0 = q8_0, 1 = q4_0 append of the K and V rows.
int launch_front(hipStream_t st, const float *qg, float *q, float *gate, float *k, const float *qw,
                 const float *kw, int n_heads, int n_kv, int n_rot, int s0, int s1, int s2, int s3,
                 const int32_t *pos, int pos0, int rows, float theta, float eps, const RopeTable &tab,
                 int enc, const float *v, uint8_t *kc, uint8_t *vc, const int32_t *step, int start,
                 int stride, const int32_t *rowpos, size_t slot_bytes)
{
    int tab_rows = 0;
    const float *t = table_for(tab, theta, n_rot, &tab_rows);
    const int per_row = n_heads + n_kv + (enc >= 0 ? n_kv : 0);
    const int max_rows = 1 << 22; // keeps (rows * per_row) far inside int
    for (int r0 = 0; r0 < rows; r0 += max_rows) {
        const int n = rows - r0 < max_rows ? rows - r0 : max_rows;
        const unsigned grid = (unsigned)(((long long)per_row * n + 3) / 4);
        const FrontAppend ap = {rowpos ? rowpos + (size_t)r0 * 2 : nullptr, slot_bytes,
                                v ? v + (size_t)r0 * n_kv * kHeadDim : nullptr,
                                kc ? kc + (rowpos ? (size_t)r0 * slot_bytes : 0) : nullptr,
                                vc ? vc + (rowpos ? (size_t)r0 * slot_bytes : 0) : nullptr, step, start + r0,
                                stride};
        auto kern = enc < 0 ? front_kernel<0> : enc == 0 ? front_kernel<1> : front_kernel<2>;
        HIPML_LAUNCH(kern, dim3(grid, 1, 1), dim3(256, 1, 1), 0, st,
                           qg + (size_t)r0 * n_heads * 2 * kHeadDim, q + (size_t)r0 * n_heads * kHeadDim,
                           gate + (size_t)r0 * n_heads * kHeadDim, k + (size_t)r0 * n_kv * kHeadDim, qw, kw,
                           n_heads, n_kv, n_rot, s0, s1, s2, s3, pos, pos0 + r0, n, theta, eps, t, tab_rows, ap);
        int rc = launched(enc < 0 ? "attn_front_f32" : "attn_front_encode_f32");
        if (rc)
            return rc;
    }
    return 0;
}

// ---- sigmoid output gate ----------------------------------------------------------
//
// y = x * (1 / (1 + exp(-g))) (crates/hipml-core/src/ops.rs:354-360).  Four
// values per thread through 128-bit accesses when the pointers allow it.

__global__ void __launch_bounds__(256) q_gate_kernel4(const float4 *x, const float4 *__restrict__ g,
                                                     float4 *y, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4)
        return;
    const float4 a = x[i];
    const float4 b = g[i];
    float4 r;
    r.x = gated(a.x, b.x);
    r.y = gated(a.y, b.y);
    r.z = gated(a.z, b.z);
    r.w = gated(a.w, b.w);
    y[i] = r;
}

__global__ void __launch_bounds__(256) q_gate_kernel1(const float *x, const float *__restrict__ g,
                                                     float *y, size_t first, size_t n)
{
    const size_t i = first + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n)
        return;
    y[i] = gated(x[i], g[i]);
}

int launch_q_gate(hipStream_t st, const float *x, const float *gate, float *y, size_t n)
{
    if (n == 0)
        return 0;
    const bool aligned = (((uintptr_t)x | (uintptr_t)gate | (uintptr_t)y) & 15) == 0;
    size_t n4 = aligned ? n / 4 : 0;
    if (n4 > 0) {
        const size_t blocks = (n4 + 255) / 256;
        HIPML_LAUNCH(q_gate_kernel4, dim3((unsigned)blocks, 1, 1), dim3(256, 1, 1), 0, st,
                           reinterpret_cast<const float4 *>(x),
                           reinterpret_cast<const float4 *>(gate), reinterpret_cast<float4 *>(y),
                           n4);
        int rc = launched("q_gate_f32");
        if (rc)
            return rc;
    }
    const size_t done = n4 * 4;
    if (done < n) {
        const size_t blocks = (n - done + 255) / 256;
        HIPML_LAUNCH(q_gate_kernel1, dim3((unsigned)blocks, 1, 1), dim3(256, 1, 1), 0, st, x,
                           gate, y, done, n);
        return launched("q_gate_f32");
    }
    return 0;
}

// ---- prefix snapshot / restore of cache rows ------------------------------------------
//
// Rows [0, rows) of every KV head, K and V, between two caches that differ only in their rows per
// head (crates/hipml-model/src/gpu/prefix.rs:214-239 packs a prefix as [head][pos][row] with one
// device copy per head and array; this is one launch, legal under capture).  16 bytes per thread
// and turn: a row is 272 or 144 bytes, so every head's span starts and ends on a 16-byte boundary.

__global__ void __launch_bounds__(256) kv_rows_copy_kernel(const uint4 *__restrict__ k_src,
                                                          const uint4 *__restrict__ v_src,
                                                          uint4 *__restrict__ k_dst, uint4 *__restrict__ v_dst,
                                                          size_t src_head16, size_t dst_head16, size_t span16)
{
    const uint4 *src = (blockIdx.z ? v_src : k_src) + blockIdx.y * src_head16;
    uint4 *dst = (blockIdx.z ? v_dst : k_dst) + blockIdx.y * dst_head16;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < span16; i += (size_t)gridDim.x * 256)
        dst[i] = src[i];
}

int launch_kv_rows_copy(hipStream_t st, int q4, const uint8_t *k_src, const uint8_t *v_src, uint8_t *k_dst,
                        uint8_t *v_dst, int n_kv, int src_stride, int dst_stride, int rows)
{
    const size_t row16 = (size_t)(q4 ? kRowBytesQ4 : kRowBytes) / 16;
    const size_t span16 = (size_t)rows * row16;
    if (span16 == 0)
        return 0;
    size_t blocks = (span16 + 255) / 256;
    if (blocks > 512)
        blocks = 512; // 2,048 workgroups over K, V and four heads fill the chip; the rest is the loop
    HIPML_LAUNCH(kv_rows_copy_kernel, dim3((unsigned)blocks, (unsigned)n_kv, 2), dim3(256, 1, 1), 0, st,
                       reinterpret_cast<const uint4 *>(k_src), reinterpret_cast<const uint4 *>(v_src),
                       reinterpret_cast<uint4 *>(k_dst), reinterpret_cast<uint4 *>(v_dst),
                       (size_t)src_stride * row16, (size_t)dst_stride * row16, span16);
    return launched("kv_rows_copy");
}

} // namespace hipml
