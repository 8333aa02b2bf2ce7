// Split-K decode attention over a q8_0 KV cache for gfx950 (wave64, MFMA).
//
// One workgroup (4 waves) owns one (kv head, key split, slot).  Each wave walks
// its own 32-key tiles of the split with a private online softmax; the four
// waves merge in LDS and write one unnormalised partial per (row, head, split).
// A second kernel merges the splits.
//
// Orientation (all MFMAs are v_mfma_f32_16x16x32_f16):
//   S^T[key][n]  = K[key][:] . Q^T[:][n]      A = K bytes as f16, B = Q (hi + lo f16)
//   O^T[d][n]   += V^T[d][key] . P'[key][n]   A = V bytes as f16 (LDS transpose read),
//                                              B = P' = p * scale_of_block(key, d/32), hi + lo f16
// n runs over (query row, head of the GQA group): up to 4 rows x 8 heads, in
// tiles of 16 columns.  The C layout of S^T (row = 4*(lane/16)+i, col = lane%16)
// is exactly the B layout the PV product needs, so probabilities never leave
// their lane, and every per-column scalar (max, sum, rescale) lives in lane%16.
//
// Exactness tricks:
//   - int8 -> f16 without arithmetic: byte b^0x80 = b+128 placed in the low byte
//     of an f16 is the subnormal (b+128)*2^-24; MFMA multiplies subnormals
//     exactly.  For K the +128 is cancelled by seeding the accumulator with
//     -128*2^-24*sum(q_block); for V by one packed f16 subtract of 2^-17.
//   - one q8 block (32 values) is one MFMA contraction, so the f16 block scale
//     multiplies an exact integer dot product in fp32 (as the CPU definition's
//     d * q does, crates/hipml-core/src/ops.rs:486-515 of the reference).
//   - Q is split into hi + lo f16 halves: two MFMAs, ~22 bits of Q.

#include "common.h"

namespace hipml {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

constexpr int kTileKeys = 32;         // keys per wave tile
constexpr int kLdsRow = 288;          // 256 payload bytes + 32 pad (bank spread)
constexpr int kWaveLds = 2 * kTileKeys * kLdsRow + 2 * kTileKeys * 16; // 19456
constexpr int kWaves = 4;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kTwo24 = 16777216.0f;

struct DecodeArgs {
    const float *q;
    const uint8_t *k;
    const uint8_t *v;
    float *part_acc;
    float *part_ml;
    const int32_t *pos;
    int n_kv, group, stride, splits;
    float scale_log2; // scale * log2(e) * 2^24
    size_t kv_slot_bytes, acc_slot, ml_slot, q_slot;
    uint16_t row0[kMaxSlots];
    uint8_t cols[kMaxSlots];
};

struct __attribute__((packed, aligned(2))) Raw16 {
    uint4v v;
};

__device__ __forceinline__ half8 bytes_to_subnormal_f16(int2v w)
{
    // byte u -> f16 bits 0x00uu = u * 2^-24
    const uint32_t x0 = (uint32_t)w[0] ^ 0x80808080u;
    const uint32_t x1 = (uint32_t)w[1] ^ 0x80808080u;
    uint4v r;
    r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c010c00u);
    r[1] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
    r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
    r[3] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
    return __builtin_bit_cast(half8, r);
}

__device__ __forceinline__ half8 sub_bias(half8 a)
{
    // (b+128)*2^-24 - 128*2^-24, exact in subnormal f16 arithmetic
    const _Float16 bias = __builtin_bit_cast(_Float16, (uint16_t)0x0080);
    return a - bias;
}

__device__ __forceinline__ float xor_max(float x, int mask)
{
    return fmaxf(x, __shfl_xor(x, mask));
}

template <int NT>
__global__ void __launch_bounds__(256) decode_q8_kernel(const DecodeArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds_all[kWaves * kWaveLds];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int lm = lane & 15; // MFMA row/col within the 16-tile
    const int lg = lane >> 4; // k-group
    const int kvh = blockIdx.x / a.splits;
    const int split = blockIdx.x - kvh * a.splits;
    const int slot = blockIdx.y;
    const int row0 = a.row0[slot];
    const int ncols = a.cols[slot];
    const int group = a.group;
    const int nvalid = ncols * group;

    // live lengths of this slot's rows
    int seqc[kMaxCols];
    int seq_max = 0;
#pragma unroll
    for (int c = 0; c < kMaxCols; c++) {
        int s = c < ncols ? a.pos[(size_t)(row0 + c) * 2 + 1] : 0;
        s = s < 0 ? 0 : (s > a.stride ? a.stride : s);
        seqc[c] = s;
        seq_max = s > seq_max ? s : seq_max;
    }
    const int per = (seq_max + a.splits - 1) / a.splits;
    const int lo = split * per;
    const int hi = lo + per < seq_max ? lo + per : seq_max;
    const int ntile = hi > lo ? (hi - lo + kTileKeys - 1) / kTileKeys : 0;

    uint8_t *lds = lds_all + wave * kWaveLds;
    uint8_t *Kp = lds;
    uint8_t *Vp = lds + kTileKeys * kLdsRow;
    uint8_t *sK = lds + 2 * kTileKeys * kLdsRow;
    uint8_t *sV = sK + kTileKeys * 16;

    const uint8_t *kbase = a.k + (size_t)slot * a.kv_slot_bytes + (size_t)kvh * a.stride * kRowBytes;
    const uint8_t *vbase = a.v + (size_t)slot * a.kv_slot_bytes + (size_t)kvh * a.stride * kRowBytes;

    // ---- Q operand: column n = nt*16 + lm -> (row n/group, head n%group) -------------
    half8 qhi[NT][8], qlo[NT][8];
    float cinit[NT][8];
    int seq_n[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const int n = nt * 16 + lm;
        const bool valid = n < nvalid;
        const int col = valid ? n / group : 0;
        const int head = valid ? n - col * group : 0;
        seq_n[nt] = valid ? seqc[col] : 0;
        const float *qp = a.q + (size_t)(row0 + col) * a.q_slot +
                          (size_t)(kvh * group + head) * kHeadDim + lg * 8;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            float4v f0 = {0, 0, 0, 0}, f1 = {0, 0, 0, 0};
            if (valid) {
                f0 = *reinterpret_cast<const float4v *>(qp + c * 32);
                f1 = *reinterpret_cast<const float4v *>(qp + c * 32 + 4);
            }
            float sum = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float x = j < 4 ? f0[j] : f1[j - 4];
                const _Float16 h = (_Float16)x;
                const _Float16 l = (_Float16)(x - (float)h);
                qhi[nt][c][j] = h;
                qlo[nt][c][j] = l;
                sum += (float)h + (float)l;
            }
            // the block's 32 values are spread over the four k-groups
            sum += __shfl_xor(sum, 16);
            sum += __shfl_xor(sum, 32);
            cinit[nt][c] = -128.0f / kTwo24 * sum;
        }
    }

    // ---- running state --------------------------------------------------------------
    float m_run[NT], l_run[NT];
    float4v O[NT][16];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        m_run[nt] = -INFINITY;
        l_run[nt] = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; t++)
            O[nt][t] = (float4v){0, 0, 0, 0};
    }

    // ---- staging: lane owns blocks b = lane + 64*j of the tile (key b/8, chunk b%8) ----
    uint4v kp0[4], kp1[4], vp0[4], vp1[4];
    uint16_t ks[4], vs[4];
    auto issue_loads = [&](int tile) {
        const int key0 = lo + tile * kTileKeys;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int b = lane + 64 * j;
            int key = key0 + (b >> 3);
            key = key < hi ? key : hi - 1; // never touch rows past the live range
            const size_t off = (size_t)key * kRowBytes + (size_t)(b & 7) * kQ8BlockBytes;
            ks[j] = *reinterpret_cast<const uint16_t *>(kbase + off);
            kp0[j] = reinterpret_cast<const Raw16 *>(kbase + off + 2)->v;
            kp1[j] = reinterpret_cast<const Raw16 *>(kbase + off + 18)->v;
            vs[j] = *reinterpret_cast<const uint16_t *>(vbase + off);
            vp0[j] = reinterpret_cast<const Raw16 *>(vbase + off + 2)->v;
            vp1[j] = reinterpret_cast<const Raw16 *>(vbase + off + 18)->v;
        }
    };
    auto store_lds = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int b = lane + 64 * j;
            const int r = b >> 3, c = b & 7;
            *reinterpret_cast<uint4v *>(Kp + r * kLdsRow + c * 32) = kp0[j];
            *reinterpret_cast<uint4v *>(Kp + r * kLdsRow + c * 32 + 16) = kp1[j];
            *reinterpret_cast<uint4v *>(Vp + r * kLdsRow + c * 32) = vp0[j];
            *reinterpret_cast<uint4v *>(Vp + r * kLdsRow + c * 32 + 16) = vp1[j];
            *reinterpret_cast<uint16_t *>(sK + r * 16 + c * 2) = ks[j];
            *reinterpret_cast<uint16_t *>(sV + r * 16 + c * 2) = vs[j];
        }
    };

    // V transpose-read address: lane (2r+e) of its 16-lane group supplies key slot r
    // (slot r<4: key lg*4+r, slot r>=4: key 16+lg*4+(r-4)), bytes [8e, 8e+8) of a 16-d run.
    const int tr_r = lm >> 1;
    const int tr_key = (tr_r >> 2) * 16 + lg * 4 + (tr_r & 3);
    const uint8_t *vtr = Vp + tr_key * kLdsRow + (lm & 1) * 8;

    int tile = wave;
    if (tile < ntile)
        issue_loads(tile);
    for (; tile < ntile; tile += kWaves) {
        store_lds();
        if (tile + kWaves < ntile)
            issue_loads(tile + kWaves);
        const int key0 = lo + tile * kTileKeys;

        // ---- scores --------------------------------------------------------------------
        half8 sk[2][4];
#pragma unroll
        for (int ms = 0; ms < 2; ms++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                sk[ms][i] = *reinterpret_cast<const half8 *>(sK + (ms * 16 + lg * 4 + i) * 16);

        float S[NT][2][4];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    S[nt][ms][i] = 0.0f;

#pragma unroll
        for (int ms = 0; ms < 2; ms++) {
#pragma unroll
            for (int c = 0; c < 8; c++) {
                const int2v raw = *reinterpret_cast<const int2v *>(
                    Kp + (ms * 16 + lm) * kLdsRow + c * 32 + lg * 8);
                const half8 A = bytes_to_subnormal_f16(raw);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    const float ci = cinit[nt][c];
                    float4v part = {ci, ci, ci, ci};
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, qhi[nt][c], part, 0, 0, 0);
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, qlo[nt][c], part, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        S[nt][ms][i] = fmaf((float)sk[ms][i][c], part[i], S[nt][ms][i]);
                }
            }
        }

        // ---- online softmax (log2 units), per column n = lane%16 -----------------------
        float p[NT][2][4];
        bool grew = false;
        float corr[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            const int lim = hi < seq_n[nt] ? hi : seq_n[nt];
            float mt = -INFINITY;
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int key = key0 + ms * 16 + lg * 4 + i;
                    const float s = key < lim ? S[nt][ms][i] * a.scale_log2 : -INFINITY;
                    S[nt][ms][i] = s;
                    mt = fmaxf(mt, s);
                }
            mt = xor_max(mt, 16);
            mt = xor_max(mt, 32);
            const float m_new = fmaxf(m_run[nt], mt);
            corr[nt] = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run[nt] - m_new);
            grew = grew || (m_new > m_run[nt]);
            float ls = 0.0f;
#pragma unroll
            for (int ms = 0; ms < 2; ms++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e = m_new == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(S[nt][ms][i] - m_new);
                    p[nt][ms][i] = e;
                    ls += e;
                }
            l_run[nt] = l_run[nt] * corr[nt] + ls;
            m_run[nt] = m_new;
        }
        if (__any(grew)) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int t = 0; t < 16; t++)
                    O[nt][t] *= corr[nt];
        }

        // ---- O^T += V^T . P' ---------------------------------------------------------------
        half8 sv[2][4];
#pragma unroll
        for (int ms = 0; ms < 2; ms++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // rows past `hi` are duplicates of the last live row: finite scale, p = 0
                sv[ms][i] = *reinterpret_cast<const half8 *>(sV + (ms * 16 + lg * 4 + i) * 16);
            }
#pragma unroll
        for (int c = 0; c < 8; c++) {
            // P' = p * block scale, carried as hi + lo f16 so the product keeps ~22 bits
            half8 Ph[NT], Pl[NT];
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int ms = 0; ms < 2; ms++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float x = p[nt][ms][i] * (float)sv[ms][i][c];
                        const _Float16 h = (_Float16)x;
                        Ph[nt][ms * 4 + i] = h;
                        Pl[nt][ms * 4 + i] = (_Float16)(x - (float)h);
                    }
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const int2v raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                    (int2v __attribute__((address_space(3))) *)(vtr + c * 32 + hf * 16));
                const half8 A = sub_bias(bytes_to_subnormal_f16(raw));
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    float4v o = O[nt][c * 2 + hf];
                    o = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Ph[nt], o, 0, 0, 0);
                    o = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Pl[nt], o, 0, 0, 0);
                    O[nt][c * 2 + hf] = o;
                }
            }
        }
    }

    // ---- merge the four waves and write the split's partial -------------------------------
    // O^T C layout: lane holds d = t*16 + lg*4 + i for column n = lane%16.
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        l_run[nt] += __shfl_xor(l_run[nt], 16);
        l_run[nt] += __shfl_xor(l_run[nt], 32);
    }
    float *wl = reinterpret_cast<float *>(lds); // per wave: [16][256] acc, then [16] m, [16] l
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        __syncthreads(); // everyone is done with the tile buffers / previous round
#pragma unroll
        for (int t = 0; t < 16; t++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                wl[lm * kHeadDim + t * 16 + lg * 4 + i] = O[nt][t][i];
        if (lg == 0) {
            wl[16 * kHeadDim + lm] = m_run[nt];
            wl[16 * kHeadDim + 16 + lm] = l_run[nt];
        }
        __syncthreads();
        // thread -> (column n, 16 consecutive d): 16 columns x 16 d-runs = 256 threads
        const int n = threadIdx.x >> 4;
        const int d0 = (threadIdx.x & 15) * 16;
        const int ng = nt * 16 + n;
        if (ng < nvalid) {
            float mw[kWaves], lw[kWaves];
            float ms = -INFINITY;
#pragma unroll
            for (int w = 0; w < kWaves; w++) {
                const float *o = reinterpret_cast<const float *>(lds_all + w * kWaveLds);
                mw[w] = o[16 * kHeadDim + n];
                lw[w] = o[16 * kHeadDim + 16 + n];
                ms = fmaxf(ms, mw[w]);
            }
            float lsum = 0.0f;
            float wgt[kWaves];
#pragma unroll
            for (int w = 0; w < kWaves; w++) {
                wgt[w] = mw[w] == -INFINITY ? 0.0f : exp2f(mw[w] - ms);
                lsum += lw[w] * wgt[w];
            }
            const int col = ng / group;
            const int head = kvh * group + (ng - col * group);
            const size_t slice = (size_t)head * a.splits + split;
            float *pa = a.part_acc + (size_t)(row0 + col) * a.acc_slot + slice * kHeadDim + d0;
#pragma unroll
            for (int dd = 0; dd < 16; dd += 4) {
                float4v acc = {0, 0, 0, 0};
#pragma unroll
                for (int w = 0; w < kWaves; w++) {
                    const float *o = reinterpret_cast<const float *>(lds_all + w * kWaveLds);
                    const float4v x = *reinterpret_cast<const float4v *>(o + n * kHeadDim + d0 + dd);
                    acc += x * (wgt[w] * kTwo24);
                }
                *reinterpret_cast<float4v *>(pa + dd) = acc;
            }
            if ((threadIdx.x & 15) == 0) {
                float *pm = a.part_ml + (size_t)(row0 + col) * a.ml_slot + slice * 2;
                pm[0] = ms;
                pm[1] = lsum;
            }
        }
    }
}

// out[row][head][d] = sum_s acc_s[d] * 2^(m_s - m) / sum_s l_s * 2^(m_s - m); 0 when no
// split saw a key.  grid (n_heads, rows), 256 threads = head_dim.
__global__ void __launch_bounds__(256) decode_reduce_kernel(
    const float *__restrict__ part_acc, const float *__restrict__ part_ml, float *__restrict__ out,
    int splits, size_t acc_slot, size_t ml_slot, size_t q_slot)
{
    const int head = blockIdx.x;
    const int row = blockIdx.y;
    const int d = threadIdx.x;
    const float *ml = part_ml + (size_t)row * ml_slot + (size_t)head * splits * 2;
    const float *acc = part_acc + (size_t)row * acc_slot + (size_t)head * splits * kHeadDim + d;
    float m = -INFINITY;
    for (int s = 0; s < splits; s++)
        if (ml[s * 2 + 1] > 0.0f)
            m = fmaxf(m, ml[s * 2]);
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < splits; s++) {
        const float l = ml[s * 2 + 1];
        if (l > 0.0f) {
            const float w = exp2f(ml[s * 2] - m);
            num = fmaf(acc[(size_t)s * kHeadDim], w, num);
            den = fmaf(l, w, den);
        }
    }
    out[(size_t)row * q_slot + (size_t)head * kHeadDim + d] = den > 0.0f ? num / den : 0.0f;
}

int launch_decode_q8(hipStream_t st, const DecodeLaunch &L)
{
    DecodeArgs a;
    a.q = L.q;
    a.k = L.k;
    a.v = L.v;
    a.part_acc = L.part_acc;
    a.part_ml = L.part_ml;
    a.pos = L.pos;
    a.n_kv = L.n_kv;
    a.group = L.n_heads / L.n_kv;
    a.stride = L.stride;
    a.splits = L.splits;
    a.scale_log2 = L.scale * kLog2e * kTwo24;
    a.kv_slot_bytes = L.kv_slot_bytes;
    a.acc_slot = L.acc_slot;
    a.ml_slot = L.ml_slot;
    a.q_slot = L.q_slot;
    for (int s = 0; s < kMaxSlots; s++) {
        a.row0[s] = s < L.slots ? L.row0[s] : 0;
        a.cols[s] = s < L.slots ? L.cols[s] : 0;
    }
    const dim3 grid((unsigned)(L.n_kv * L.splits), (unsigned)L.slots, 1);
    if (L.max_cols * a.group <= 16)
        hipLaunchKernelGGL(decode_q8_kernel<1>, grid, dim3(256, 1, 1), 0, st, a);
    else
        hipLaunchKernelGGL(decode_q8_kernel<2>, grid, dim3(256, 1, 1), 0, st, a);
    int rc = launched("attn_decode_kv_q8");
    if (rc)
        return rc;
    hipLaunchKernelGGL(decode_reduce_kernel, dim3((unsigned)L.n_heads, (unsigned)L.total_rows, 1),
                       dim3(256, 1, 1), 0, st, L.part_acc, L.part_ml, L.out, L.splits, L.acc_slot,
                       L.ml_slot, L.q_slot);
    return launched("attn_decode_kv_reduce");
}

} // namespace hipml
