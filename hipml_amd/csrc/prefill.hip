// Causal GQA chunk prefill over a q8_0 KV cache for gfx950 (wave64, MFMA).
//
// One workgroup = one KV head x one tile of 32 query tokens (x one key slice when
// split).  Wave w of the workgroup owns query head kvh*group + w, so a wave's
// MFMA column n is query token t0 + n.  All waves share the K/V tile, which is
// dequantized once per workgroup into f16 in LDS.
//
// All MFMAs are v_mfma_f32_32x32x16_f16:
//   S^T[key 32][tok 32] += K[key][d 16] . Q^T[d 16][tok]       (16 steps over d)
//   O^T[d 32][tok 32]   += V^T[d][key 16] . P^T[key 16][tok]   (2 key halves x 8 d tiles)
// V^T comes from the row-major f16 V tile through the LDS transpose read
// (ds_read_b64_tr_b16); P^T is the S^T accumulator layout converted in place, so
// probabilities never move between lanes and every per-token scalar (max, sum,
// rescale) lives in lane%32.
//
// Numerics follow the reference's chunk kernel: Q, dequantized K/V (f16 scale x
// int8, one rounding) and P are f16 operands; scores, softmax and accumulation
// are fp32; softmax runs in log2 units.

#include "common.h"

namespace hipml {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));

constexpr int kQTile = 32;   // query tokens per workgroup
constexpr int kKTile = 32;   // keys per LDS tile
constexpr int kRowF16 = 528; // bytes per dequantized row in LDS: 512 + 16 pad
constexpr float kLog2e = 1.4426950408889634f;

struct ChunkArgs {
    const float *q;
    const uint8_t *kc;
    const uint8_t *vc;
    float *out;
    float *part_acc;
    float *part_ml;
    int n_head, n_kv, group;
    int pos0, tokens, stride, splits, qslots;
    float scale_log2;
};

struct __attribute__((packed, aligned(2))) Raw16 {
    uint4v v;
};

// 16 int8 -> 16 f16 (value * d), d an f16 scale: the bytes become 1024 + (b+128)
// in f16 by bit tricks, the bias is subtracted exactly, then one packed multiply
// rounds d*b once -- the same value as (f16)((float)d * (float)b).
__device__ __forceinline__ void dequant16(uint4v raw, _Float16 d, uint4v &lo, uint4v &hi)
{
    const half2v bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    const half2v dd = {d, d};
    uint32_t o[8];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t x = raw[w] ^ 0x80808080u;
        const uint32_t a = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u); // [0x64,b1,0x64,b0]
        const uint32_t b = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u); // [0x64,b3,0x64,b2]
        o[2 * w] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(half2v, a) - bias) * dd);
        o[2 * w + 1] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(half2v, b) - bias) * dd);
    }
    lo = (uint4v){o[0], o[1], o[2], o[3]};
    hi = (uint4v){o[4], o[5], o[6], o[7]};
}

template <bool SPLIT>
__global__ void __launch_bounds__(512) chunk_q8_kernel(const ChunkArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t Ks[kKTile * kRowF16];
    __shared__ __attribute__((aligned(16))) uint8_t Vs[kKTile * kRowF16];

    const int wave = threadIdx.x >> 6; // query head within the group
    const int lane = threadIdx.x & 63;
    const int ln = lane & 31;  // MFMA column: token within the tile
    const int lh = lane >> 5;  // k half-group
    const int kvh = blockIdx.x;
    const int t0 = blockIdx.y * kQTile;
    const int split = SPLIT ? blockIdx.z : 0;
    const int head = kvh * a.group + wave;

    // visible key range of this workgroup
    const int last_tok = (t0 + kQTile < a.tokens ? t0 + kQTile : a.tokens) - 1;
    const int seq_block = a.pos0 + last_tok + 1;
    int klo = 0, khi = seq_block;
    if (SPLIT) {
        klo = (int)((long long)seq_block * split / a.splits);
        khi = (int)((long long)seq_block * (split + 1) / a.splits);
    }
    const int tok = t0 + ln;
    const int my_last_key = a.pos0 + tok; // inclusive causal bound of this lane's token
    const bool tok_valid = tok < a.tokens;

    // ---- Q^T operand: 16 k-steps of 8 f16 (d = ks*16 + lh*8 + j) ---------------------------
    half8 qf[16];
    {
        const int tq = tok_valid ? tok : a.tokens - 1;
        const float *qp = a.q + ((size_t)tq * a.n_head + head) * kHeadDim + lh * 8;
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            const float4v f0 = *reinterpret_cast<const float4v *>(qp + ks * 16);
            const float4v f1 = *reinterpret_cast<const float4v *>(qp + ks * 16 + 4);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                qf[ks][j] = (_Float16)f0[j];
                qf[ks][4 + j] = (_Float16)f1[j];
            }
        }
    }

    float16v O[8];
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            O[t][i] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    const uint8_t *kbase = a.kc + (size_t)kvh * a.stride * kRowBytes;
    const uint8_t *vbase = a.vc + (size_t)kvh * a.stride * kRowBytes;

    // staging role: thread b < 256 owns block (key b/8, chunk b%8) of the tile
    const int sb = threadIdx.x;
    const bool stager = sb < 256;
    uint4v rk0, rk1, rv0, rv1;
    uint16_t rks = 0, rvs = 0;
    auto issue = [&](int k0) {
        if (stager) {
            int key = k0 + (sb >> 3);
            key = key < khi ? key : khi - 1;
            const size_t off = (size_t)key * kRowBytes + (size_t)(sb & 7) * kQ8BlockBytes;
            rks = *reinterpret_cast<const uint16_t *>(kbase + off);
            rk0 = reinterpret_cast<const Raw16 *>(kbase + off + 2)->v;
            rk1 = reinterpret_cast<const Raw16 *>(kbase + off + 18)->v;
            rvs = *reinterpret_cast<const uint16_t *>(vbase + off);
            rv0 = reinterpret_cast<const Raw16 *>(vbase + off + 2)->v;
            rv1 = reinterpret_cast<const Raw16 *>(vbase + off + 18)->v;
        }
    };
    auto stage = [&]() {
        if (stager) {
            const int r = sb >> 3, c = sb & 7;
            uint4v a0, a1, a2, a3;
            dequant16(rk0, __builtin_bit_cast(_Float16, rks), a0, a1);
            dequant16(rk1, __builtin_bit_cast(_Float16, rks), a2, a3);
            uint4v *dk = reinterpret_cast<uint4v *>(Ks + r * kRowF16 + c * 64);
            dk[0] = a0;
            dk[1] = a1;
            dk[2] = a2;
            dk[3] = a3;
            dequant16(rv0, __builtin_bit_cast(_Float16, rvs), a0, a1);
            dequant16(rv1, __builtin_bit_cast(_Float16, rvs), a2, a3);
            uint4v *dv = reinterpret_cast<uint4v *>(Vs + r * kRowF16 + c * 64);
            dv[0] = a0;
            dv[1] = a1;
            dv[2] = a2;
            dv[3] = a3;
        }
    };

    // V transpose-read geometry: 16-lane group G = lane/16 covers d rows (G&1)*16.. of the
    // 32-row tile and k half-group lh = G>>1; lane L of the group supplies key (L/4), d run (L%4)*4.
    const int gl = lane & 15;
    const int vtr_off = (gl >> 2) * kRowF16 + (((lane >> 4) & 1) * 16 + (gl & 3) * 4) * 2;

    if (klo < khi)
        issue(klo);
    for (int k0 = klo; k0 < khi; k0 += kKTile) {
        __syncthreads(); // previous tile fully consumed
        stage();
        if (k0 + kKTile < khi)
            issue(k0 + kKTile);
        __syncthreads();

        // ---- S^T = K . Q^T ------------------------------------------------------------------
        float16v S;
#pragma unroll
        for (int i = 0; i < 16; i++)
            S[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            const half8 A =
                *reinterpret_cast<const half8 *>(Ks + ln * kRowF16 + (ks * 16 + lh * 8) * 2);
            S = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, qf[ks], S, 0, 0, 0);
        }

        // ---- online softmax; lane holds keys (i/4)*8 + lh*4 + i%4 of column ln ---------------
        const bool need_mask = (k0 + kKTile - 1 > a.pos0 + t0) || (k0 + kKTile > khi);
        float mt = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float s = S[i] * a.scale_log2;
            if (need_mask) {
                const int kg = k0 + (i >> 2) * 8 + lh * 4 + (i & 3);
                s = (kg <= my_last_key && kg < khi) ? s : -INFINITY;
            }
            S[i] = s;
            mt = fmaxf(mt, s);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32));
        const float m_new = fmaxf(m_run, mt);
        const bool dead = m_new == -INFINITY;
        const float corr = dead ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
        float ls = 0.0f;
        half8 P[2];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float e = dead ? 0.0f : __builtin_amdgcn_exp2f(S[i] - m_new);
            const _Float16 eh = (_Float16)e;
            ls += (float)eh; // the sum uses the rounded weights the PV product uses
            P[i >> 3][i & 7] = eh;
        }
        l_run = l_run * corr + ls;
        if (__any(m_new > m_run)) {
#pragma unroll
            for (int t = 0; t < 8; t++)
                O[t] *= corr;
        }
        m_run = m_new;

        // ---- O^T += V^T . P^T ------------------------------------------------------------------
#pragma unroll
        for (int u = 0; u < 2; u++) {
#pragma unroll
            for (int dt = 0; dt < 8; dt++) {
                // keys of read q: (2u+q)*8 + lh*4 + {0..3}
                const uint8_t *vp = Vs + vtr_off + dt * 64;
                const short4v r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3))) *)(vp + ((2 * u) * 8 + lh * 4) * kRowF16));
                const short4v r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3))) *)(vp + ((2 * u + 1) * 8 + lh * 4) * kRowF16));
                half8 A;
                const half4 h0 = __builtin_bit_cast(half4, r0);
                const half4 h1 = __builtin_bit_cast(half4, r1);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    A[j] = h0[j];
                    A[4 + j] = h1[j];
                }
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, P[u], O[dt], 0, 0, 0);
            }
        }
    }

    // ---- epilogue --------------------------------------------------------------------------
    l_run += __shfl_xor(l_run, 32);
    if (!tok_valid)
        return;
    if (SPLIT) {
        const size_t row = ((size_t)split * a.qslots + tok) * a.n_head + head;
        float *pa = a.part_acc + row * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 8; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4v x = {O[dt][g * 4], O[dt][g * 4 + 1], O[dt][g * 4 + 2], O[dt][g * 4 + 3]};
                *reinterpret_cast<float4v *>(pa + dt * 32 + g * 8 + lh * 4) = x;
            }
        if (lh == 0) {
            a.part_ml[row * 2] = m_run;
            a.part_ml[row * 2 + 1] = l_run;
        }
    } else {
        const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
        float *po = a.out + ((size_t)tok * a.n_head + head) * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 8; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4v x = {O[dt][g * 4] * inv, O[dt][g * 4 + 1] * inv, O[dt][g * 4 + 2] * inv,
                                   O[dt][g * 4 + 3] * inv};
                *reinterpret_cast<float4v *>(po + dt * 32 + g * 8 + lh * 4) = x;
            }
    }
}

// Fold the key slices: grid (tokens, n_head), 256 threads = head_dim.
__global__ void __launch_bounds__(256) chunk_combine_kernel(
    const float *__restrict__ part_acc, const float *__restrict__ part_ml, float *__restrict__ out,
    int n_head, int qslots, int splits)
{
    const int tok = blockIdx.x;
    const int head = blockIdx.y;
    const int d = threadIdx.x;
    float m = -INFINITY;
    for (int s = 0; s < splits; s++) {
        const size_t row = ((size_t)s * qslots + tok) * n_head + head;
        if (part_ml[row * 2 + 1] > 0.0f)
            m = fmaxf(m, part_ml[row * 2]);
    }
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < splits; s++) {
        const size_t row = ((size_t)s * qslots + tok) * n_head + head;
        const float l = part_ml[row * 2 + 1];
        if (l > 0.0f) {
            const float w = __builtin_amdgcn_exp2f(part_ml[row * 2] - m);
            num = fmaf(part_acc[row * kHeadDim + d], w, num);
            den = fmaf(l, w, den);
        }
    }
    out[((size_t)tok * n_head + head) * kHeadDim + d] = den > 0.0f ? num / den : 0.0f;
}

int launch_chunk_q8(hipStream_t st, const float *q, const uint8_t *kc, const uint8_t *vc,
                    float *out, int n_head, int n_kv, int pos0, int tokens, int stride,
                    float *part_acc, float *part_ml, int splits)
{
    ChunkArgs a;
    a.q = q;
    a.kc = kc;
    a.vc = vc;
    a.out = out;
    a.part_acc = part_acc;
    a.part_ml = part_ml;
    a.n_head = n_head;
    a.n_kv = n_kv;
    a.group = n_head / n_kv;
    a.pos0 = pos0;
    a.tokens = tokens;
    a.stride = stride;
    a.splits = splits;
    a.qslots = (tokens + 31) / 32 * 32;
    a.scale_log2 = kLog2e / 16.0f; // 1/sqrt(256), as the reference's chunk launcher fixes it
    const unsigned qtiles = (unsigned)((tokens + kQTile - 1) / kQTile);
    const dim3 block((unsigned)(a.group * 64), 1, 1);
    if (splits < 2) {
        hipLaunchKernelGGL(chunk_q8_kernel<false>, dim3((unsigned)n_kv, qtiles, 1), block, 0, st, a);
        return launched("attn_chunk_q8");
    }
    hipLaunchKernelGGL(chunk_q8_kernel<true>, dim3((unsigned)n_kv, qtiles, (unsigned)splits), block,
                       0, st, a);
    int rc = launched("attn_chunk_q8_split");
    if (rc)
        return rc;
    hipLaunchKernelGGL(chunk_combine_kernel, dim3((unsigned)tokens, (unsigned)n_head, 1),
                       dim3(256, 1, 1), 0, st, part_acc, part_ml, out, n_head, a.qslots, splits);
    return launched("attn_chunk_combine");
}

} // namespace hipml
