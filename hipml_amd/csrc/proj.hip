// Projections over Q8_0 weight matrices for gfx950 (wave64, MFMA): the step after the attention
// core (the output projection W_o) and, with other shapes, the one before it (W_q, W_k, W_v).
//
// W is [m][k/32] blocks of 34 bytes (f16 scale d, 32 int8), row-major; y[r][row] = sum_k W[row][k] x[r][k]
// (crates/hipml-core/src/quant.rs:653-675, crates/hipml-core/src/ops.rs:102-104,136-176).
//
// gemv_q8_rows_kernel: one or two activation rows, bound by streaming W once from HBM.
//   All MFMAs are v_mfma_f32_16x16x32_f16 with A = x (activation rows), B = W (16 weight rows),
//   one q8 block = one contraction, so the f16 block scale multiplies an exact integer dot product
//   in fp32: acc += d * (x . q), as the CPU definition's d*q products summed in fp32.
//   Fetch: a step is a pair of blocks of one weight row, 68 bytes at a dword boundary.  Lane 4*r + g
//   requests, with dword-aligned loads only, the 12 bytes that hold quarter g of the even block
//   (2 bytes in, realigned with alignbit) and the 8 of the odd block's quarter; the scales ride
//   along in lanes g = 0 and g = 3.  The four lanes of a quad read contiguous bytes.  (The MFMA's own
//   lane order, row = lane % 16, with 2-byte aligned 64-bit loads made every lane several requests
//   of its own: 9.5 M cache accesses per call and 1.0 TB/s.)  One ds_bpermute per register then
//   moves the data to the MFMA lane (row lm, quarter lg).  The C
//   tile puts weight row lm back in lane lm (rows of C are activation rows), where its scale is.
//   int8 -> f16 exactly: byte b^0x80 = b+128 under a high byte 0x64 is the f16 1024 + (b+128);
//   one packed f16 subtract of 1152 leaves b.  x enters as hi + lo f16 halves (two MFMAs, ~22 bits),
//   converted once per workgroup into LDS in operand order (whole rows: a pass is a few rows at most).
//   The waves of a workgroup split k; a wave requests the activations first, then two chunks of
//   its weight blocks (all of them for k = 6144) before it waits for anything, and the partial sums
//   meet in LDS in a fixed order (no atomics: the result does not depend on timing).
// gemv_q8_tile_kernel (further down): the same stream for 3 to 128 rows, activations as full A tiles.

#include "common.h"

namespace hipml {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t uint3a4 __attribute__((ext_vector_type(3), aligned(4)));

constexpr int kQ8Block = 34;


// 8 int8 (two dwords) -> 8 f16 holding the same integers, exactly.
__device__ __forceinline__ half8 int8x8_to_f16(uint32_t w0, uint32_t w1)
{
    const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
    const uint32_t hi = 0x64646464u;
    uint4v r;
    r[0] = __builtin_amdgcn_perm(hi, x0, 0x04010400u);
    r[1] = __builtin_amdgcn_perm(hi, x0, 0x04030402u);
    r[2] = __builtin_amdgcn_perm(hi, x1, 0x04010400u);
    r[3] = __builtin_amdgcn_perm(hi, x1, 0x04030402u);
    half8 h = __builtin_bit_cast(half8, r);
    const half8 off = {1152, 1152, 1152, 1152, 1152, 1152, 1152, 1152};
    return h - off;
}

// 8 f32 -> hi and lo f16 halves with hi + lo = x to ~22 bits.
__device__ __forceinline__ void split_hi_lo(const float4v &a, const float4v &b, half8 &hi, half8 &lo)
{
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float x0 = j < 2 ? a[2 * j] : b[2 * j - 4];
        const float x1 = j < 2 ? a[2 * j + 1] : b[2 * j - 3];
        const half2v h = __builtin_bit_cast(half2v, __builtin_amdgcn_cvt_pkrtz(x0, x1));
        // x - h (exact: h holds the leading bits of x) in one mixed-precision instruction per value, which reads
        // the f16 half in place; the compiler turns the same expression into a conversion and a subtraction
        const uint32_t hb = __builtin_bit_cast(uint32_t, h);
        float r0, r1;
        asm("v_fma_mix_f32 %0, -%1, 1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r0) : "v"(hb), "v"(x0));
        asm("v_fma_mix_f32 %0, -%1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r1) : "v"(hb), "v"(x1));
        const half2v l = __builtin_bit_cast(half2v, __builtin_amdgcn_cvt_pkrtz(r0, r1));
        hi[2 * j] = h[0];
        hi[2 * j + 1] = h[1];
        lo[2 * j] = l[0];
        lo[2 * j + 1] = l[1];
    }
}

// One chunk of a wave's steps, as fetched.  A step is a pair of blocks of one weight row (68 bytes,
// dword aligned): the fetch lane of k quarter g holds bytes 8g..8g+11 of the pair (the even block's
// quarter sits 2 bytes in; g = 0 also catches the even scale, g = 3 the odd one) and the odd block's
// quarter, which is aligned.
template <int TILES, int CH>
struct GemvChunk {
    uint3a4 e[CH][TILES];
    uint2a4 o[CH][TILES];
};

constexpr int kGemvMaxRows = 2;        // activation rows per pass (their operands live in LDS)
constexpr int kGemvLdsBudget = 128 << 10;

// Activation rows per pass for a given k: as many (up to kGemvMaxRows) as keep the hi/lo operands of
// the whole rows, 4 bytes per element, inside the LDS budget; 0 = k too large.
__host__ __device__ inline int gemv_rows_per_pass(int k)
{
    const int fit = kGemvLdsBudget / (4 * k);
    return fit > kGemvMaxRows ? kGemvMaxRows : fit;
}
static_assert(kGemvLdsBudget / 4 / 8 / 512 <= 8, "a pass is staged in one round of at most 8 groups per thread");

// LDS: x operands [k/32 blocks][2*rp A rows: hi of rows 0..rp-1, then lo][4 quarters][8 x f16], then
// the partial sums [WAVES][TILES][32 lanes] float4.  The hi and the lo halves are different rows of
// ONE A operand: A rows 0..3 carry hi, rows 4..7 lo, so a block is one MFMA and the two partial
// products come out in lanes 0..15 (hi) and 16..31 (lo) of the C tile.
template <int WAVES, int TILES, int CH, int XG>
__global__ void __launch_bounds__(64 * WAVES, TILES == 1 ? 2 : 1) gemv_q8_rows_kernel(const uint8_t *__restrict__ w,
                                                                const float *__restrict__ x,
                                                                float *__restrict__ y, int m, int k,
                                                                int rows, int rp)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int lm = lane & 15, lg = lane >> 4; // MFMA operand lane: weight row lm, k quarter lg
    const int fr = lane >> 2, fg = lane & 3;  // fetch lane: weight row fr, k quarter fg
    const int pull = (lm * 4 + lg) * 4;       // byte address of the fetch lane that holds this lane's operand
    const int nb = k >> 5;
    const size_t row_bytes = (size_t)nb * kQ8Block;
    const int m0 = blockIdx.x * (16 * TILES);
    const int r0 = blockIdx.y * rp;
    const int nrows = rows - r0 < rp ? rows - r0 : rp;
    const int nu = nb >> 1; // steps: pairs of blocks
    const int u_lo = (int)((long)wave * nu / WAVES), u_hi = (int)((long)(wave + 1) * nu / WAVES);
    float4v *red = reinterpret_cast<float4v *>(lds + (size_t)nb * rp * 128);
    const int per_row = k >> 3; // 8-element groups of one activation row

    // ---- 1. this thread's share of the activations, requested first (they are waited for first) --
    // group e = 8 consecutive k of one row; (row, e) pairs are dealt round-robin to the threads
    const int groups = nrows * (k >> 3);
    // XG groups in flight per thread and round; a thread with fewer left wraps around to groups that
    // are not its own (loaded, not stored) rather than all such threads asking for one address
    float4v xa[XG], xb[XG];
    auto x_issue = [&](int g0) {
#pragma unroll
        for (int i = 0; i < XG; i++) {
            int g = g0 + i * 64 * WAVES;
            g = g < groups ? g : g % groups;
            const float *p = x + (size_t)r0 * k + (size_t)g * 8; // rows are contiguous: group g of the pass

            xa[i] = *reinterpret_cast<const float4v *>(p);
            xb[i] = *reinterpret_cast<const float4v *>(p + 4);
        }
    };
    auto x_store = [&](int g0) {
#pragma unroll
        for (int i = 0; i < XG; i++) {
            const int g = g0 + i * 64 * WAVES;
            if (g < groups) {
                const int r = rp == 1 ? 0 : g / per_row, e = g - r * per_row;
                half8 hi, lo;
                split_hi_lo(xa[i], xb[i], hi, lo);
                uint8_t *blk = lds + (size_t)(e >> 2) * rp * 128 + (e & 3) * 16;
                *reinterpret_cast<half8 *>(blk + r * 64) = hi;
                *reinterpret_cast<half8 *>(blk + (rp + r) * 64) = lo;
            }
        }
    };
    x_issue(threadIdx.x);
    // every wave's activation requests enter the CU's memory pipeline before any wave's weight
    // requests: the pipeline serves them in order, and the first barrier below waits for the last
    // wave's activations
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. the first two chunks of this wave's weight blocks ------------------------------------
    // rows past the end are clamped: they load (and compute) a duplicate that is never stored
    const uint8_t *wp[TILES];
#pragma unroll
    for (int t = 0; t < TILES; t++) {
        const int row = m0 + t * 16 + fr < m ? m0 + t * 16 + fr : m - 1;
        wp[t] = w + (size_t)row * row_bytes;
    }
    typedef GemvChunk<TILES, CH> Chunk;
    auto fetch = [&](Chunk &c, int u0) {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            int uc = u0 + i < u_hi ? u0 + i : u_hi - 1;
            uc = uc < 0 ? 0 : uc;
#pragma unroll
            for (int t = 0; t < TILES; t++) {
                const uint8_t *unit = wp[t] + (size_t)uc * (2 * kQ8Block);
                c.e[i][t] = *reinterpret_cast<const uint3a4 *>(unit + fg * 8);
                c.o[i][t] = *reinterpret_cast<const uint2a4 *>(unit + 36 + fg * 8);
            }
        }
    };
    Chunk A, B;
    fetch(A, u_lo);
    fetch(B, u_lo + CH);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 3. activations to LDS as MFMA operands -----------------------------------------------
    x_store(threadIdx.x); // XG covers every group: the launcher sizes the pass for that
    __syncthreads();

    // ---- 4. the block steps --------------------------------------------------------------------
    float4v acc[TILES];
#pragma unroll
    for (int t = 0; t < TILES; t++)
        acc[t] = (float4v){0, 0, 0, 0};
    // A row lm: hi of activation row lm for lm < 4, lo of row lm - 4 for 4 <= lm < 8; the rest, and
    // rows past the live ones, repeat a valid slot (their products are never read)
    const int ar = (lm & 3) < nrows ? (lm & 3) : nrows - 1;
    const uint8_t *xop = lds + ((size_t)(((lm >> 2) & 1) * rp + ar) * 4 + lg) * 16;
    // One step = operands staged (realign, gather scales, move to the MFMA lanes, read x), then the
    // arithmetic; a step's staging is issued before the previous step's arithmetic so the LDS
    // round trips are covered, and the scheduler may not move anything across a step: a step waits
    // for its own two loads only.
    struct Staged {
        uint32_t q[TILES][4];
        uint32_t ds[TILES];
        half8 x0, x1;
    };
    auto stage = [&](Staged &s, const Chunk &c, int i, int u) {
        const int uc = u < u_hi ? u : u_hi - 1;
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            const uint3a4 e = c.e[i][t];
            // in the fetch lane: the even quarter realigned; both scales gathered in the quad's lane 0
            const int e2_of_g3 = __builtin_amdgcn_update_dpp(0, (int)e[2], 0xFF, 0xf, 0xf, true);
            const int sc = (int)((e[0] & 0xffffu) | ((uint32_t)e2_of_g3 & 0xffff0000u));
            s.q[t][0] = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)__builtin_amdgcn_alignbit(e[1], e[0], 16));
            s.q[t][1] = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)__builtin_amdgcn_alignbit(e[2], e[1], 16));
            s.q[t][2] = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)c.o[i][t][0]);
            s.q[t][3] = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)c.o[i][t][1]);
            s.ds[t] = (uint32_t)__builtin_amdgcn_ds_bpermute(lm * 16, sc);
        }
        s.x0 = *reinterpret_cast<const half8 *>(xop + (size_t)uc * rp * 256);
        s.x1 = *reinterpret_cast<const half8 *>(xop + (size_t)uc * rp * 256 + rp * 128);
    };
    auto math = [&](const Staged &s, int u) {
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            const float d0 = u < u_hi ? (float)__builtin_bit_cast(_Float16, (uint16_t)(s.ds[t] & 0xffffu)) : 0.0f;
            const float d1 = u < u_hi ? (float)__builtin_bit_cast(_Float16, (uint16_t)(s.ds[t] >> 16)) : 0.0f;
            const half8 w0 = int8x8_to_f16(s.q[t][0], s.q[t][1]), w1 = int8x8_to_f16(s.q[t][2], s.q[t][3]);
            float4v p0 = {0, 0, 0, 0}, p1 = {0, 0, 0, 0};
            p0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(s.x0, w0, p0, 0, 0, 0);
            p1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(s.x1, w1, p1, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[t][j] = fmaf(d1, p1[j], fmaf(d0, p0[j], acc[t][j]));
        }
    };
    auto compute = [&](const Chunk &c, int u0) {
        Staged s0, s1;
        stage(s0, c, 0, u0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < CH; i += 2) {
            if (i + 1 < CH)
                stage(s1, c, i + 1, u0 + i + 1);
            __builtin_amdgcn_sched_barrier(0);
            math(s0, u0 + i);
            __builtin_amdgcn_sched_barrier(0);
            if (i + 1 < CH) {
                if (i + 2 < CH)
                    stage(s0, c, i + 2, u0 + i + 2);
                __builtin_amdgcn_sched_barrier(0);
                math(s1, u0 + i + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // The first two chunks (all of a wave's steps up to k = 64 * 2 * CH * WAVES) are straight-line
    // code, so each step waits for exactly its own loads while the rest are still in flight.
    // Longer rows continue in a loop that fetches and consumes two chunks per turn; nothing is
    // carried in registers from one turn to the next (carried chunks made the compiler copy them at
    // the loop head, behind a wait for every outstanding load).
    if (u_hi > u_lo) {
        compute(A, u_lo);
        compute(B, u_lo + CH);
        for (int u = u_lo + 2 * CH; u < u_hi; u += 2 * CH) {
            fetch(A, u);
            fetch(B, u + CH);
            compute(A, u);
            compute(B, u + CH);
        }
    }

    // ---- 5. the k slices meet in a fixed order: lanes 0..15 hold the hi products of activation
    // rows 0..3, lanes 16..31 the lo products ---------------------------------------------------
    if (lg < 2) {
#pragma unroll
        for (int t = 0; t < TILES; t++)
            red[(wave * TILES + t) * 32 + lane] = acc[t];
    }
    __syncthreads();
    if (threadIdx.x < 16 * TILES) {
        const int t = threadIdx.x >> 4, l = threadIdx.x & 15;
        float4v hi = red[t * 32 + l], lo = red[t * 32 + 16 + l];
#pragma unroll
        for (int u = 1; u < WAVES; u++) {
            hi += red[(u * TILES + t) * 32 + l];
            lo += red[(u * TILES + t) * 32 + 16 + l];
        }
        const float4v s = hi + lo;
        const int row = m0 + t * 16 + l;
        if (row < m) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (j < nrows)
                    y[(size_t)(r0 + j) * m + row] = s[j];
        }
    }
}

// ---- gemv_q8_dma_kernel: one to eight activation rows, the weight rows moved into LDS as they lie in memory ----
//
// The row kernel above asks for its weights in 12- and 8-byte pieces per lane, which the memory pipeline serves
// at 10.0 us for the 33.4 MB of a 5120 x 6144 matrix; the same bytes as whole pieces of rows through
// global_load_lds_dwordx4 need no registers while they travel and arrive sooner.  A workgroup takes `rows_wg`
// consecutive weight rows (m / 256 where that is 16..32: one workgroup per CU and every CU the same bytes; one or
// two MFMA tiles of 16 rows); its waves deal the rows' chunks of 256 values (8 blocks, 272 bytes: the smallest
// piece of a row that starts and ends at a 16-byte boundary) round-robin, and a wave keeps two chunks in flight
// into a ring of two buffers.  Nothing is shared between the waves until their sums meet, so the loop has no
// barrier.
// The activations take the same road as raw f32 and become MFMA operands in place (the 128 bytes of a block's 32
// floats of one row become 64 bytes of f16 hi halves and 64 of lo halves, x = hi + lo to ~22 bits): with one row,
// all of a wave's chunks before the loop, while the first weights travel; with more rows, a chunk's values ride
// behind its weights in the ring and are converted when the chunk has arrived.
// One v_mfma_f32_16x16x32_f16 per block and tile with A = activations (A rows 0..7 the hi halves of rows 0..7, A
// rows 8..15 the lo halves), B = 16 weight rows.  Lane (lm, lg) reads its 8 bytes of weight row lm, quarter lg of
// the block, from the raw rows with dword-aligned reads (even blocks sit 2 bytes past a boundary and are
// realigned; LDS reads at 2-byte alignment measured four times slower).  The weight bytes enter the MFMA as the
// f16 subnormals (b + 128) x 2^-24, one v_perm_b32 per pair: exact, and the offset 128 comes out again as
// 128 x 2^-24 x (sum of the block's activation halves), a number the wave forms once per block and chunk.  The
// block's scale multiplies the corrected fp32 dot product, as the CPU definition's d * q products summed in
// fp32; 2^24 multiplies the final sum.
// A (row, weight row) result is the sum, in a fixed order, of eight chains (chunk c belongs to chain c % 8, a
// chain adds its blocks in order), hi and lo halves apart until the end: the same operations in the same order
// whatever RP, the wave count and rows_wg are and whichever rows travel with it, so a verify group's rows have the
// bits of their plain decodes (crates/hipml-kernels/src/attn_gpu.rs:930-932).
constexpr int kDmaChunkBytes = 8 * kQ8Block; // 272: one row's share of a chunk
constexpr int kDmaChains = 8;
constexpr float kTwo24f = 16777216.0f;

__device__ __forceinline__ uint32_t proj_lds_address(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// 64 lanes x 16 bytes from base + voff (per lane) to LDS address lds_at + 16 * lane; ONCE: read once (weights)
template <bool ONCE>
__device__ __forceinline__ void proj_dma16(uint32_t lds_at, const uint8_t *base, uint32_t voff)
{
    if (ONCE)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                     :
                     : "s"(lds_at), "v"(voff), "s"(base)
                     : "memory");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_at), "v"(voff), "s"(base)
                     : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vm()
{
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// 8 int8 (two dwords) -> 8 f16 subnormals (b + 128) x 2^-24, exactly
__device__ __forceinline__ half8 int8x8_to_f16_sub(uint32_t w0, uint32_t w1)
{
    const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
    uint4v r;
    r[0] = __builtin_amdgcn_perm(0u, x0, 0x0c010c00u);
    r[1] = __builtin_amdgcn_perm(0u, x0, 0x0c030c02u);
    r[2] = __builtin_amdgcn_perm(0u, x1, 0x0c010c00u);
    r[3] = __builtin_amdgcn_perm(0u, x1, 0x0c030c02u);
    return __builtin_bit_cast(half8, r);
}

// The variants: RP activation rows per pass on WAVES waves; NI requests of 64 x 16 bytes per chunk of weights
// (rows_wg x 17 pieces), which also says how many 16-row tiles cover rows_wg.
constexpr bool gemv_dma_front(int rp) { return rp == 1; }
constexpr int gemv_dma_tiles(int ni) { return ni > 5 ? 2 : 1; }
constexpr int kDmaDepth = 2; // chunks in flight per wave (three measured no faster)
// a ring entry: the chunk's weights as they arrive (rows_wg x 272 bytes) and, behind them, its activations
inline int gemv_dma_entry(int rp, int rows_wg) { return rows_wg * kDmaChunkBytes + (gemv_dma_front(rp) ? 0 : rp * 1024); }
inline int gemv_dma_lds(int rp, int ni, int waves, int rows_wg, int k)
{
    const int per_wave = ((k >> 8) + waves - 1) / waves; // chunks of a wave
    // rings (at least the 1 KB per chain and tile in which the chains' sums meet at the end); front: the waves'
    // activations, 1 KB per chunk; the waves' offset tables [8 blocks][2 rp] floats per chunk (front: every chunk,
    // else the ring's two)
    int ring = kDmaDepth * gemv_dma_entry(rp, rows_wg);
    const int sums = kDmaChains / waves * gemv_dma_tiles(ni) * 64 * 16;
    ring = ring > sums ? ring : sums;
    return waves * ring + (gemv_dma_front(rp) ? waves * per_wave * (1024 + 64) : waves * 2 * 64 * rp);
}

template <int RP, int NI, int WAVES>
__global__ void __launch_bounds__(64 * WAVES, 1) gemv_q8_dma_kernel(const uint8_t *__restrict__ w,
                                                                                 const float *__restrict__ x,
                                                                                 float *__restrict__ y, int m, int k,
                                                                                 int rows, int rows_wg)
{
    static_assert(RP == 1 || RP == 2 || RP == 4 || RP == 8, "activation rows per pass");
    static_assert(WAVES == 4 || WAVES == 8, "the eight chains are dealt to four or eight waves");
    constexpr int kWaves = WAVES;
    constexpr int kNCh = kDmaChains / kWaves; // chains of a wave
    constexpr int kNT = gemv_dma_tiles(NI);
    constexpr bool kFront = gemv_dma_front(RP);
    constexpr int kDepth = kDmaDepth;
    constexpr int kReq = NI + (kFront ? 0 : RP); // requests per chunk
    constexpr int kNJ = RP < 4 ? RP : 4;         // accumulator rows a lane needs
    constexpr int kUnits = 32 * RP;              // (block, row, quarter) units of 8 activations per chunk
    constexpr int kPasses = (kUnits + 63) / 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int lm = lane & 15, lg = lane >> 4;
    const int nb = k >> 5;
    const int nchunk = nb >> 3;
    const uint32_t row_bytes = (uint32_t)nb * kQ8Block;
    const int m0 = blockIdx.x * rows_wg;
    const int r0 = blockIdx.y * RP;
    const int nrows = rows - r0 < RP ? rows - r0 : RP;
    const int pieces = rows_wg * 17;
    if ((pieces + 63) / 64 != NI)
        return; // (the launcher's contract: the waits below count NI requests per chunk of weights)
    const int mine = wave < nchunk ? (nchunk - wave + kWaves - 1) / kWaves : 0; // chunks wave, wave + kWaves, ...
    const int per_wave = (nchunk + kWaves - 1) / kWaves;

    const int entry = pieces * 16 + (kFront ? 0 : RP * 1024);
    constexpr int kSums = kNCh * kNT * 64 * 16; // where this wave's chains leave their sums: the head of its ring
    const int ring_bytes = kDepth * entry > kSums ? kDepth * entry : kSums;
    uint8_t *ring = lds + wave * ring_bytes;
    uint8_t *xfront = lds + kWaves * ring_bytes + wave * per_wave * 1024; // (front only)
    uint8_t *after_x = lds + kWaves * ring_bytes + (kFront ? kWaves * per_wave * 1024 : 0);
    float *offs = reinterpret_cast<float *>(after_x + wave * (kFront ? per_wave * 64 : 2 * 64 * RP));
    const uint32_t ring_at = proj_lds_address(ring);

    // ---- requests ---------------------------------------------------------------------------------------------
    // weights: piece p = 64 j + lane of the chunk: row p / 17 of the workgroup, 16 bytes p % 17 of its 272; rows
    // past the end of the matrix repeat the last one (never stored)
    uint32_t woff[NI];
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const int p = j * 64 + lane;
        const int pr = p / 17, pq = p - pr * 17;
        const int row = m0 + pr < m ? m0 + pr : m - 1;
        woff[j] = (uint32_t)row * row_bytes + (uint32_t)pq * 16u;
    }
    const uint8_t *xb = reinterpret_cast<const uint8_t *>(x + (size_t)r0 * k);
    auto issue = [&](int i) {
        const uint32_t at = ring_at + (uint32_t)((i % kDepth) * entry);
        const uint32_t c = (uint32_t)(wave + i * kWaves);
        // activations behind the weights: one request per row, its 256 floats of the chunk as they lie in memory;
        // rows past the live ones repeat the last
        if (!kFront) {
#pragma unroll
            for (int r = 0; r < RP; r++) {
                const uint32_t rr = (uint32_t)(r < nrows ? r : nrows - 1);
                proj_dma16<false>(at + pieces * 16 + r * 1024, xb, rr * (uint32_t)k * 4u + c * 1024u + lane * 16u);
            }
        }
        // (NI = ceil(pieces / 64): every request has a live lane, so each chunk counts NI requests)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            if (j * 64 + lane < pieces)
                proj_dma16<true>(at + j * 1024, w, woff[j] + c * kDmaChunkBytes);
        }
    };
    if (kFront) {
        for (int i = 0; i < mine; i++)
            proj_dma16<false>(proj_lds_address(xfront) + i * 1024, xb, (uint32_t)(wave + i * kWaves) * 1024u + lane * 16u);
    }
#pragma unroll
    for (int i = 0; i < kDepth; i++)
        if (i < mine)
            issue(i);
    // all but the newest `newer` chunks (at most kDepth - 1) have arrived: requests return in order
    auto wait_chunks = [&](int newer) {
        if (newer >= 2 && kDepth > 2)
            wait_vm<(kDepth > 2 ? 2 : 0) * kReq>();
        else if (newer >= 1)
            wait_vm<kReq>();
        else
            wait_vm<0>();
    };

    // ---- activations -> operands, in place: unit ((block b, row r), quarter q): 8 floats -> 8 hi and 8 lo halves in
    // the operand order of the block, and the block's offset terms.  Every unit of an area is read before any is
    // written (one wave, LDS in program order).
    auto unit_write = [&](uint8_t *area, float *off, int b, int r, int q, bool on, const float4v &a4, const float4v &b4) {
        half8 hi, lo;
        split_hi_lo(a4, b4, hi, lo);
        float sh = 0.0f, sl = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            sh += (float)hi[e];
            sl += (float)lo[e];
        }
        // over the unit's four quarters (the lanes of a quad)
        sh += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sh), 0xB1, 0xf, 0xf, true));
        sl += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sl), 0xB1, 0xf, 0xf, true));
        sh += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sh), 0x4E, 0xf, 0xf, true));
        sl += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sl), 0x4E, 0xf, 0xf, true));
        if (on) {
            uint8_t *blk = area + b * (RP * 128) + q * 16;
            *reinterpret_cast<half8 *>(blk + r * 64) = hi;
            *reinterpret_cast<half8 *>(blk + (RP + r) * 64) = lo;
            if (q == 0) {
                off[b * 2 * RP + r] = sh * (128.0f / kTwo24f);
                off[b * 2 * RP + RP + r] = sl * (128.0f / kTwo24f);
            }
        }
    };
    if (kFront) {
        // two chunks per pass: lanes 0..31 the units of chunk 2 ps, lanes 32..63 those of chunk 2 ps + 1
        constexpr int kFrontPasses = 2;
        // only weights are still travelling
        if (mine >= 2)
            wait_vm<2 * NI>();
        else
            wait_vm<NI>();
        for (int i0 = 0; i0 < mine; i0 += 2 * kFrontPasses) {
            float4v a4[kFrontPasses], b4[kFrontPasses];
#pragma unroll
            for (int ps = 0; ps < kFrontPasses; ps++) {
                const int i = i0 + 2 * ps + (lane >> 5);
                const uint8_t *src = xfront + (i < mine ? i : 0) * 1024 + (lane & 31) * 32;
                a4[ps] = *reinterpret_cast<const float4v *>(src);
                b4[ps] = *reinterpret_cast<const float4v *>(src + 16);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int ps = 0; ps < kFrontPasses; ps++) {
                const int i = i0 + 2 * ps + (lane >> 5);
                unit_write(xfront + i * 1024, offs + i * 16, (lane & 31) >> 2, 0, lane & 3, i < mine, a4[ps], b4[ps]);
            }
        }
    }

    float4v acc[kNCh][kNT];
#pragma unroll
    for (int s = 0; s < kNCh; s++)
#pragma unroll
        for (int t = 0; t < kNT; t++)
            acc[s][t] = (float4v){0, 0, 0, 0};
    // A row lm: half lm / 8 (hi, lo) of activation row lm % 8; rows past the live ones repeat a valid slot
    // (their products are never read)
    const int arow = (lm & 7) < nrows ? (lm & 7) : nrows - 1;
    const int xslot = (((lm >> 3) * RP + arow) * 4 + lg) * 16;
    // the lane's accumulators are C rows 4 lg + j: half lg / 2, activation rows 4 (lg % 2) + j
    const int obase = (lg >> 1) * RP + ((lg & 1) * 4 < RP ? (lg & 1) * 4 : 0);
    int wrow[kNT]; // (rows of the second tile past rows_wg repeat the last: never stored)
#pragma unroll
    for (int t = 0; t < kNT; t++)
        wrow[t] = (t * 16 + lm < rows_wg ? t * 16 + lm : rows_wg - 1) * kDmaChunkBytes;

    auto chunk = [&](int i, float4v (&sum)[kNT]) {
        wait_chunks(mine - 1 - i < kDepth - 1 ? mine - 1 - i : kDepth - 1);
        uint8_t *buf = ring + (i % kDepth) * entry;
        uint8_t *xa = kFront ? xfront + i * 1024 : buf + pieces * 16;
        float *off = offs + (kFront ? i : (i & 1)) * (16 * RP);
        if (!kFront) {
            float4v a4[kPasses], b4[kPasses];
#pragma unroll
            for (int ps = 0; ps < kPasses; ps++) {
                const int u = ps * 64 + lane;
                const int br = u >> 2, q = u & 3;
                const int b = br / RP, r = br - b * RP;
                const uint8_t *src = xa + (u < kUnits ? r * 1024 + b * 128 + q * 32 : 0);
                a4[ps] = *reinterpret_cast<const float4v *>(src);
                b4[ps] = *reinterpret_cast<const float4v *>(src + 16);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int ps = 0; ps < kPasses; ps++) {
                const int u = ps * 64 + lane;
                const int br = u >> 2, q = u & 3;
                const int b = br / RP, r = br - b * RP;
                unit_write(xa, off, b, r, q, u < kUnits, a4[ps], b4[ps]);
            }
        }
        // ---- the chunk's 8 blocks, in two halves: the reads of the second travel while the first is multiplied
        half8 xop[8];
        float ofs[8][kNJ];
        uint32_t qa[8][kNT], qb[8][kNT], qc[4][kNT];
        _Float16 dh[8][kNT];
        auto read_block = [&](int b) {
            xop[b] = *reinterpret_cast<const half8 *>(xa + b * (RP * 128) + xslot);
#pragma unroll
            for (int j = 0; j < kNJ; j++)
                ofs[b][j] = off[b * 2 * RP + obase + j];
#pragma unroll
            for (int t = 0; t < kNT; t++) {
                const uint8_t *blk = buf + wrow[t] + b * kQ8Block;
                // the lane's 8 bytes sit 2 bytes past a dword boundary in even blocks (three dwords, realigned
                // below) and at one in odd blocks
                if ((b & 1) == 0) {
                    const uint3a4 e = *reinterpret_cast<const uint3a4 *>(blk + lg * 8);
                    qa[b][t] = e[0];
                    qb[b][t] = e[1];
                    qc[b >> 1][t] = e[2];
                } else {
                    const uint2a4 o = *reinterpret_cast<const uint2a4 *>(blk + 2 + lg * 8);
                    qa[b][t] = o[0];
                    qb[b][t] = o[1];
                }
                dh[b][t] = *reinterpret_cast<const _Float16 *>(blk);
            }
        };
        auto math_block = [&](int b) {
#pragma unroll
            for (int t = 0; t < kNT; t++) {
                uint32_t q0 = qa[b][t], q1 = qb[b][t];
                if ((b & 1) == 0) {
                    q0 = __builtin_amdgcn_alignbit(qb[b][t], qa[b][t], 16);
                    q1 = __builtin_amdgcn_alignbit(qc[b >> 1][t], qb[b][t], 16);
                }
                const float d = (float)dh[b][t];
                const half8 wv = int8x8_to_f16_sub(q0, q1);
                float4v p = {0, 0, 0, 0};
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(xop[b], wv, p, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < kNJ; j++)
                    sum[t][j] = fmaf(d, p[j] - ofs[b][j], sum[t][j]);
            }
        };
#pragma unroll
        for (int b = 0; b < 4; b++)
            read_block(b);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 4; b < 8; b++)
            read_block(b);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < 4; b++)
            math_block(b);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 4; b < 8; b++)
            math_block(b);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the wave's reads of this entry are done
        if (i + kDepth < mine)
            issue(i + kDepth);
    };
    // chunk wave + i kWaves belongs to chain wave + (i % kNCh) kWaves
    for (int i0 = 0; i0 < mine; i0 += kNCh) {
#pragma unroll
        for (int s = 0; s < kNCh; s++)
            if (i0 + s < mine)
                chunk(i0 + s, acc[s]);
    }

    // ---- the chains' sums meet in their order; lanes lg = 0, 1 hold the hi products of activation rows 4 lg + j,
    // lanes lg = 2, 3 the lo products ----------------------------------------------------------------------------
    // (a wave leaves its chains' sums at the head of its own ring, which it has finished reading)
    auto sums_of = [&](int chain, int t) {
        return reinterpret_cast<float4v *>(lds + (chain % kWaves) * ring_bytes) + ((chain / kWaves) * kNT + t) * 64;
    };
#pragma unroll
    for (int s = 0; s < kNCh; s++)
#pragma unroll
        for (int t = 0; t < kNT; t++)
            sums_of(wave + s * kWaves, t)[lane] = acc[s][t];
    __syncthreads();
    if (threadIdx.x < 32 * kNT) {
        const int t = threadIdx.x >> 5, l = threadIdx.x & 31; // (weight row 16 t + l % 16, activation rows 4 (l / 16) + j)
        float4v hi = sums_of(0, t)[l], lo = sums_of(0, t)[32 + l];
#pragma unroll
        for (int c = 1; c < kDmaChains; c++) {
            hi += sums_of(c, t)[l];
            lo += sums_of(c, t)[32 + l];
        }
        const float4v s = (hi + lo) * kTwo24f;
        const int wr = t * 16 + (l & 15);
        if (wr < rows_wg && m0 + wr < m) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int r = (l >> 4) * 4 + j;
                if (r < nrows)
                    y[(size_t)(r0 + r) * m + m0 + wr] = s[j];
            }
        }
    }
}

// ---- gemv_q8_dma_tile_kernel: 10 to 128 activation rows over the same stream of raw weight rows, 64 a pass ------
//
// More rows than the kernel above holds operands for.  The workgroups are the same (rows_wg consecutive weight
// rows, one workgroup per CU, eight waves), but the waves walk the chunks together: for a chunk of 256 values the
// workgroup fetches its weight rows and the same 256 values of every activation row as raw f32 (1 KB per row, all
// through global_load_lds_dwordx4, the requests dealt to the waves), and wave w multiplies block w of the chunk.  So
// a workgroup reads every activation once, from LDS.
// Lane (row lm, quarter lg) of an A tile reads its 8 floats and splits them into hi and lo halves in registers;
// a block and tile is two chained MFMAs (hi, then lo into the same fp32 sums) per weight tile, the weights exactly as
// f16 integers (1024 + u trick), the block scale applied to the fp32 dot product.  The activation rows lie 1,040
// bytes apart in LDS, so the 16 rows of a tile start in 16 different banks.
// Two rings: kDW chunks of weights and kDX chunks of activations are in flight, two barriers per chunk.  Vector
// memory returns in order, so a wave that waits for its activation requests of a chunk also waits for every weight
// request it made before them: the activations of chunk c + kDX are asked for before the weights of chunk c + kDW,
// and the wait counts the activation requests behind it only.
// A (row, weight row) result is the sum in wave order of eight chains (block b of every chunk belongs to chain b):
// the same whatever the number of rows, and other bits than those of the kernel for up to 8 rows.
constexpr int kTileRowPitch = 1040;
// (chunks of activations / of weights in flight, measured at 5120 x 6144 over 16 / 24 / 32 / 64 rows: 2 / 3: 17.5 / 23.4 /
// 23.5 / 39.8 us; 2 / 4: 17.9 / 29.0 / 29.1 / 41.4; 3 / 6: 18.3 / 25.5 / 25.6 / -; the tile kernel below: 19.6 / 25.8 / 29.7 /
// 54.5.  The figures for 24 and 32 rows move between 23.4 and 29.6 us from run to run of the same build, those for 16 and 64
// do not.  Two chunks a turn of the loop, half the barriers: 20.5 / 26.7 / 26.9 against 17.5 / 29.6 / 29.7 in one run; every
// workgroup starting at another chunk, so that they do not all ask for the same activation bytes at once: 20.8 / 24.3 / 24.5 /
// 39.2 against 17.4 / 23.4 / 23.5 / 39.7 in one run.  Not fetching the 8 rows of a last tile that has no more than 8 live
// ones (HALF): 17 and 24 rows 21.9 us where 32 rows take 23.5, 33 and 40 rows 34.7 / 34.8 where 48 take 35.1.  Sixteen waves,
// two per block of a chunk with one weight tile each: 18.4 / 24.9 / 45.9 us at 16 / 24 / 64 rows against 17.0 / 22.7 / 34.0.)
constexpr int gemv_tile_dx(int) { return 2; }
constexpr int gemv_tile_dw(int) { return 3; }
inline int gemv_dma_tile_lds(int xt, int ni, int rows_wg)
{
    const int ring = gemv_tile_dw(xt) * rows_wg * 17 * 16 + gemv_tile_dx(xt) * 16 * xt * kTileRowPitch;
    const int sums = 8 * xt * gemv_dma_tiles(ni) * 64 * 16;
    return ring > sums ? ring : sums;
}

template <int XT, int NI, bool HALF>
__global__ void __launch_bounds__(512, 1) gemv_q8_dma_tile_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x,
                                                                   float *__restrict__ y, int m, int k, int rows,
                                                                   int rows_wg)
{
    constexpr int kNT = gemv_dma_tiles(NI);
    constexpr int kXRows = 16 * XT;
    constexpr int kDX = gemv_tile_dx(XT), kDW = gemv_tile_dw(XT);
    static_assert(kDW > kDX, "a chunk's weights are asked for before its activations");
    // activation requests of a wave per chunk: one per row, 16 XT rows, or 8 fewer (HALF: the last tile has at most
    // 8 live rows; the other 8 are never fetched, hold whatever the ring held, and their sums are never stored)
    constexpr int kNX = 2 * XT - (HALF ? 1 : 0);
    constexpr int kWMost = (NI + 7) / 8;     // weight requests of a wave per chunk, or one less
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int lm = lane & 15, lg = lane >> 4;
    const int nb = k >> 5;
    const int nchunk = nb >> 3;
    const uint32_t row_bytes = (uint32_t)nb * kQ8Block;
    const int m0 = blockIdx.x * rows_wg;
    const int r0 = blockIdx.y * kXRows;
    const int nrows = rows - r0 < kXRows ? rows - r0 : kXRows;
    const int pieces = rows_wg * 17;
    if ((pieces + 63) / 64 != NI)
        return; // (the launcher's contract: a chunk of weights is NI requests)
    const int wbytes = pieces * 16;
    constexpr int kXBytes = kXRows * kTileRowPitch;
    uint8_t *wring = lds, *xring = lds + kDW * wbytes;
    const uint32_t wring_at = proj_lds_address(wring), xring_at = proj_lds_address(xring);

    // weights of chunk c: request q = wave + 8 j < NI brings 64 pieces (piece p: row p / 17 of the workgroup, 16
    // bytes p % 17 of its 272; rows past the end of the matrix repeat the last)
    uint32_t woff[kWMost];
#pragma unroll
    for (int j = 0; j < kWMost; j++) {
        const int p = (wave + 8 * j) * 64 + lane;
        const int pr = p / 17, pq = p - pr * 17;
        const int row = m0 + pr < m ? m0 + pr : m - 1;
        woff[j] = (uint32_t)row * row_bytes + (uint32_t)pq * 16u;
    }
    int wreq = 0; // weight requests of this wave per chunk
#pragma unroll
    for (int j = 0; j < kWMost; j++)
        wreq += wave + 8 * j < NI ? 1 : 0;
    auto issue_w = [&](int c) {
        const uint32_t at = wring_at + (uint32_t)((c % kDW) * wbytes);
#pragma unroll
        for (int j = 0; j < kWMost; j++) {
            const int q = wave + 8 * j;
            if (q < NI && q * 64 + lane < pieces)
                proj_dma16<true>(at + q * 1024, w, woff[j] + (uint32_t)c * kDmaChunkBytes);
        }
    };
    // activations of chunk c: rows wave + 8 j of the pass (rows past the live ones repeat the last), 256 floats each
    const uint8_t *xb = reinterpret_cast<const uint8_t *>(x + (size_t)r0 * k);
    uint32_t xoff[kNX];
#pragma unroll
    for (int j = 0; j < kNX; j++) {
        const int r = wave + 8 * j;
        xoff[j] = (uint32_t)(r < nrows ? r : nrows - 1) * (uint32_t)k * 4u + lane * 16u;
    }
    auto issue_x = [&](int c) {
        const uint32_t at = xring_at + (uint32_t)((c % kDX) * kXBytes);
#pragma unroll
        for (int j = 0; j < kNX; j++)
            proj_dma16<false>(at + (wave + 8 * j) * kTileRowPitch, xb, xoff[j] + (uint32_t)c * 1024u);
    };
#pragma unroll
    for (int c = 0; c < kDW; c++)
        if (c < nchunk)
            issue_w(c);
#pragma unroll
    for (int c = 0; c < kDX; c++)
        if (c < nchunk)
            issue_x(c);

    float4v acc[XT][kNT];
#pragma unroll
    for (int xt = 0; xt < XT; xt++)
#pragma unroll
        for (int t = 0; t < kNT; t++)
            acc[xt][t] = (float4v){0, 0, 0, 0};
    int wrow[kNT]; // (rows of the second tile past rows_wg repeat the last: never stored)
#pragma unroll
    for (int t = 0; t < kNT; t++)
        wrow[t] = (t * 16 + lm < rows_wg ? t * 16 + lm : rows_wg - 1) * kDmaChunkBytes;
    const int b = wave; // this wave's block of every chunk

    for (int c = 0; c < nchunk; c++) {
        // This wave's requests for chunk c have arrived once only those made after them are outstanding.  In the
        // steady state these are, in order, the weights of chunk c + 1, then per chunk finished since (kDX of them)
        // the activations and the weights asked for behind it: kDX - 1 sets of activations and kDX of weights in
        // all.  Counting the activation sets alone waits for requests made a chunk ago as well; measured at 16 / 24 /
        // 48 / 64 rows: 17.5 / 21.9 / 35.1 / 39.7 us so, 17.5 / 23.2 / 31.2 / 35.7 with the full count, hence the full
        // count from three activation tiles on.  At the ends, where some of those chunks do not exist, only the
        // activation sets that do are counted, which errs on the side of waiting.
        {
            static_assert(kDX == 2 && kDW == 3 && kWMost <= 2, "the counts below");
            const int behind = nchunk - 1 - c < kDX - 1 ? nchunk - 1 - c : kDX - 1;
            if (XT >= 3 && c >= kDX && c + kDW - 1 < nchunk) {
                if (wreq == 0)
                    wait_vm<kNX>();
                else if (wreq == 1)
                    wait_vm<kNX + kDX>();
                else
                    wait_vm<kNX + 2 * kDX>();
            } else if (behind >= 1) {
                wait_vm<kNX>();
            } else {
                wait_vm<0>();
            }
        }
        __syncthreads(); // ... and every wave's
        const uint8_t *wbuf = wring + (c % kDW) * wbytes;
        const uint8_t *xa = xring + (c % kDX) * kXBytes + b * 128 + lg * 32;
        half8 wv[kNT];
        float d[kNT];
#pragma unroll
        for (int t = 0; t < kNT; t++) {
            const uint8_t *blk = wbuf + wrow[t] + b * kQ8Block;
            uint32_t q0, q1;
            if ((b & 1) == 0) { // (uniform) even blocks sit 2 bytes past a dword boundary
                const uint3a4 e = *reinterpret_cast<const uint3a4 *>(blk + lg * 8);
                q0 = __builtin_amdgcn_alignbit(e[1], e[0], 16);
                q1 = __builtin_amdgcn_alignbit(e[2], e[1], 16);
            } else {
                const uint2a4 o = *reinterpret_cast<const uint2a4 *>(blk + 2 + lg * 8);
                q0 = o[0];
                q1 = o[1];
            }
            d[t] = (float)*reinterpret_cast<const _Float16 *>(blk);
            wv[t] = int8x8_to_f16(q0, q1);
        }
#pragma unroll
        for (int xt = 0; xt < XT; xt++) {
            const uint8_t *src = xa + (xt * 16 + lm) * kTileRowPitch;
            const float4v a4 = *reinterpret_cast<const float4v *>(src);
            const float4v b4 = *reinterpret_cast<const float4v *>(src + 16);
            half8 hi, lo;
            split_hi_lo(a4, b4, hi, lo);
#pragma unroll
            for (int t = 0; t < kNT; t++) {
                float4v p = {0, 0, 0, 0};
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi, wv[t], p, 0, 0, 0);
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo, wv[t], p, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[xt][t][j] = fmaf(d[t], p[j], acc[xt][t][j]);
            }
        }
        __syncthreads(); // every wave is done with the chunk's entries: later chunks may land in them
        if (c + kDX < nchunk)
            issue_x(c + kDX);
        if (c + kDW < nchunk)
            issue_w(c + kDW);
    }

    // ---- the waves' sums meet in wave order (the rings are free: the loop ended on a barrier) --------------------
    float4v *red = reinterpret_cast<float4v *>(lds);
#pragma unroll
    for (int xt = 0; xt < XT; xt++)
#pragma unroll
        for (int t = 0; t < kNT; t++)
            red[((wave * XT + xt) * kNT + t) * 64 + lane] = acc[xt][t];
    __syncthreads();
    for (int e = threadIdx.x; e < XT * kNT * 64; e += 512) {
        const int l = e & 63, xt_t = e >> 6;
        const int xt = xt_t / kNT, t = xt_t - xt * kNT;
        float4v s = red[e];
#pragma unroll
        for (int u = 1; u < 8; u++)
            s += red[u * (XT * kNT * 64) + e];
        const int wr = t * 16 + (l & 15);
        if (wr < rows_wg && m0 + wr < m) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int r = xt * 16 + (l >> 4) * 4 + j;
                if (r < nrows)
                    y[(size_t)(r0 + r) * m + m0 + wr] = s[j];
            }
        }
    }
}

// ---- gemv_q8_tile_kernel: 3 to 128 activation rows (batched decode, verify groups) --------------
//
// The same streaming of W as above, with the activations as full 16-row A tiles: A row = activation
// row, hi and lo halves as two chained MFMAs, XT tiles (16 or 32 rows) per pass.  The rows' operands
// no longer fit LDS, and need not: the waves of a workgroup split k, so no two of them want the same
// activations; lane (lm, lg) loads the 8 f32 of row lm, k quarter lg of each block straight from
// global memory (L2: the rows are a few hundred KB that every workgroup reads) and splits them in
// registers.  A step (a pair of blocks: 16 XT registers of activations, 5 TILES of weights) is one
// record; four records rotate, each refilled as soon as it has been consumed, activations before
// weights in request order (the loads complete in order: a step then waits for nothing younger than
// itself).  What the time is made of at 5120 x 6144 and 16 rows: 13.1 us with the activation loads
// taken out (the arithmetic is hidden behind the weight stream), 16.1 with all of them hitting L1,
// 19.8 as it is: every workgroup reads every row (393 KB through its CU's L1 for 208 KB of weights).
// Four weight tiles per workgroup halve that and leave 80 workgroups, too few to keep HBM busy (27.5 us).
template <int TILES, int XT>
struct TileRec {
    float4v x[XT][2][2]; // [tile][block of the pair][half of the 8 values]
    uint3a4 e[TILES];
    uint2a4 o[TILES];
};

template <int WAVES, int TILES, int XT, int STEPS>
__global__ void __launch_bounds__(64 * WAVES, 1) gemv_q8_tile_kernel(const uint8_t *__restrict__ w,
                                                                   const float *__restrict__ x,
                                                                   float *__restrict__ y, int m, int k, int rows)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int lm = lane & 15, lg = lane >> 4; // MFMA operand lane: A row / weight row lm, k quarter lg
    const int fr = lane >> 2, fg = lane & 3;  // fetch lane: weight row fr, k quarter fg
    const int pull = (lm * 4 + lg) * 4;
    const int nb = k >> 5;
    const size_t row_bytes = (size_t)nb * kQ8Block;
    const int m0 = blockIdx.x * (16 * TILES);
    const int r0 = blockIdx.y * (16 * XT);
    const int nu = nb >> 1; // steps: pairs of blocks
    // The steps are dealt to the waves round-robin: the activation rows are a multiple of the L2's
    // channel interleave apart, so the 16 rows of one load meet in one channel, and only the k
    // offsets of requests in flight spread the traffic; eight neighbouring steps are 2 KB of a row.
    // (With a contiguous slice of k per wave the activation loads cost 10 us on top of 13.)
    float4v *red = reinterpret_cast<float4v *>(lds);

    // rows past the end are clamped: loaded and multiplied, never stored
    const float *xp[XT];
#pragma unroll
    for (int t = 0; t < XT; t++) {
        const int r = r0 + t * 16 + lm < rows ? r0 + t * 16 + lm : rows - 1;
        xp[t] = x + (size_t)r * k + lg * 8;
    }
    const uint8_t *wp[TILES];
#pragma unroll
    for (int t = 0; t < TILES; t++) {
        const int row = m0 + t * 16 + fr < m ? m0 + t * 16 + fr : m - 1;
        wp[t] = w + (size_t)row * row_bytes;
    }
    typedef TileRec<TILES, XT> Rec;
    auto fetch = [&](Rec &c, int u) {
        const int uc = u < nu ? u : nu - 1;
#pragma unroll
        for (int t = 0; t < XT; t++)
#pragma unroll
            for (int b = 0; b < 2; b++) {
                const float *p = xp[t] + (size_t)uc * 64 + b * 32;
                c.x[t][b][0] = *reinterpret_cast<const float4v *>(p);
                c.x[t][b][1] = *reinterpret_cast<const float4v *>(p + 4);
            }
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            const uint8_t *unit = wp[t] + (size_t)uc * (2 * kQ8Block);
            c.e[t] = *reinterpret_cast<const uint3a4 *>(unit + fg * 8);
            c.o[t] = *reinterpret_cast<const uint2a4 *>(unit + 36 + fg * 8);
        }
    };
    float4v acc[TILES][XT];
#pragma unroll
    for (int t = 0; t < TILES; t++)
#pragma unroll
        for (int a = 0; a < XT; a++)
            acc[t][a] = (float4v){0, 0, 0, 0};
    auto consume = [&](const Rec &c, int u) {
        const bool live = u < nu;
        half8 hi[XT][2], lo[XT][2];
#pragma unroll
        for (int a = 0; a < XT; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
                split_hi_lo(c.x[a][b][0], c.x[a][b][1], hi[a][b], lo[a][b]);
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            const uint3a4 e = c.e[t];
            const int e2_of_g3 = __builtin_amdgcn_update_dpp(0, (int)e[2], 0xFF, 0xf, 0xf, true);
            const int sc = (int)((e[0] & 0xffffu) | ((uint32_t)e2_of_g3 & 0xffff0000u));
            const uint32_t q0 = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)__builtin_amdgcn_alignbit(e[1], e[0], 16));
            const uint32_t q1 = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)__builtin_amdgcn_alignbit(e[2], e[1], 16));
            const uint32_t q2 = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)c.o[t][0]);
            const uint32_t q3 = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)c.o[t][1]);
            const uint32_t ds = (uint32_t)__builtin_amdgcn_ds_bpermute(lm * 16, sc);
            const float d0 = live ? (float)__builtin_bit_cast(_Float16, (uint16_t)(ds & 0xffffu)) : 0.0f;
            const float d1 = live ? (float)__builtin_bit_cast(_Float16, (uint16_t)(ds >> 16)) : 0.0f;
            const half8 w0 = int8x8_to_f16(q0, q1), w1 = int8x8_to_f16(q2, q3);
#pragma unroll
            for (int a = 0; a < XT; a++) {
                float4v p0 = {0, 0, 0, 0}, p1 = {0, 0, 0, 0};
                p0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi[a][0], w0, p0, 0, 0, 0);
                p1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi[a][1], w1, p1, 0, 0, 0);
                p0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo[a][0], w0, p0, 0, 0, 0);
                p1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo[a][1], w1, p1, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[t][a][j] = fmaf(d1, p1[j], fmaf(d0, p0[j], acc[t][a][j]));
            }
        }
    };
    // STEPS > 0: every wave has exactly STEPS steps (the launcher checks) and the code is straight
    // line, so each step waits for exactly its own loads.  Otherwise a loop of four steps per turn
    // (the records keep their registers; the compiler waits for every outstanding load at the head
    // of a turn); a fetch past the wave's last step repeats it and a step past it multiplies by a
    // zero scale.  The scheduler may not move a step's arithmetic past the refill behind it, or the
    // other way round: either makes the wave wait for loads it has only just asked for.
    Rec c[4];
    const int u_lo = wave;
    fetch(c[0], u_lo);
    fetch(c[1], u_lo + WAVES);
    fetch(c[2], u_lo + 2 * WAVES);
    fetch(c[3], u_lo + 3 * WAVES);
    if (STEPS > 0) {
#pragma unroll
        for (int i = 0; i < STEPS; i++) {
            __builtin_amdgcn_sched_barrier(0);
            consume(c[i & 3], u_lo + i * WAVES);
            __builtin_amdgcn_sched_barrier(0);
            if (i + 4 < STEPS)
                fetch(c[i & 3], u_lo + (i + 4) * WAVES);
        }
    } else {
        for (int u = u_lo; u < nu; u += 4 * WAVES) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                __builtin_amdgcn_sched_barrier(0);
                consume(c[i], u + i * WAVES);
                __builtin_amdgcn_sched_barrier(0);
                fetch(c[i], u + (i + 4) * WAVES);
            }
        }
    }

    // the k slices meet in a fixed order: C row 4 lg + j = activation row, column lm = weight row
#pragma unroll
    for (int t = 0; t < TILES; t++)
#pragma unroll
        for (int a = 0; a < XT; a++)
            red[((wave * TILES + t) * XT + a) * 64 + lane] = acc[t][a];
    __syncthreads();
    for (int i = threadIdx.x; i < TILES * XT * 64; i += 64 * WAVES) {
        float4v s = red[i];
#pragma unroll
        for (int u = 1; u < WAVES; u++)
            s += red[u * TILES * XT * 64 + i];
        const int l = i & 63, a = (i >> 6) % XT, t = (i >> 6) / XT;
        const int row = m0 + t * 16 + (l & 15);
        const int r = r0 + a * 16 + 4 * (l >> 4);
        if (row < m) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (r + j < rows)
                    y[(size_t)(r + j) * m + row] = s[j];
        }
    }
}

template <int WAVES, int TILES, int XT, int STEPS>
static int launch_gemv_tile_steps(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows)
{
    const size_t lds = (size_t)WAVES * TILES * XT * 64 * sizeof(float4v);
    auto kern = gemv_q8_tile_kernel<WAVES, TILES, XT, STEPS>;
    const dim3 grid((unsigned)((m + 16 * TILES - 1) / (16 * TILES)), (unsigned)((rows + 16 * XT - 1) / (16 * XT)), 1);
    HIPML_LAUNCH(kern, grid, dim3(64 * WAVES, 1, 1), lds, st, w, x, y, m, k, rows);
    return launched("gemv_q8_0_rows");
}

template <int WAVES, int TILES, int XT>
static int launch_gemv_tile(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows)
{
    // straight-line variants for the model's two inner sizes: 6144 (W_o) and 5120 (W_q, W_k, W_v)
    if (k == 64 * WAVES * 12)
        return launch_gemv_tile_steps<WAVES, TILES, XT, 12>(st, w, x, y, m, k, rows);
    if (k == 64 * WAVES * 10)
        return launch_gemv_tile_steps<WAVES, TILES, XT, 10>(st, w, x, y, m, k, rows);
    return launch_gemv_tile_steps<WAVES, TILES, XT, 0>(st, w, x, y, m, k, rows);
}

template <int WAVES, int TILES, int CH, int XG>
static int launch_gemv_xg(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k,
                          int rows, int rp)
{
    const size_t lds = (size_t)(k >> 5) * rp * 128 + (size_t)WAVES * TILES * 32 * sizeof(float4v);
    auto kern = gemv_q8_rows_kernel<WAVES, TILES, CH, XG>;
    const dim3 grid((unsigned)((m + 16 * TILES - 1) / (16 * TILES)), (unsigned)((rows + rp - 1) / rp), 1);
    HIPML_LAUNCH(kern, grid, dim3(64 * WAVES, 1, 1), lds, st, w, x, y, m, k, rows, rp);
    return launched("gemv_q8_0_rows");
}

template <int WAVES, int TILES, int CH>
static int launch_gemv_variant(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k,
                               int rows, int rp)
{
    // 8-element groups of the activations per thread
    const int need = (rp * (k >> 3) + 64 * WAVES - 1) / (64 * WAVES);
    if (need <= 2)
        return launch_gemv_xg<WAVES, TILES, CH, 2>(st, w, x, y, m, k, rows, rp);
    if (need <= 4)
        return launch_gemv_xg<WAVES, TILES, CH, 4>(st, w, x, y, m, k, rows, rp);
    // rp * k <= 32,768 (the LDS budget), so 8 groups per thread always cover a pass
    return launch_gemv_xg<WAVES, TILES, CH, 8>(st, w, x, y, m, k, rows, rp);
}

// the most waves (8, else 4) whose rings and tables fit a CU's LDS; 0: none
static int gemv_dma_waves(int rp, int ni, int rows_wg, int k)
{
    for (int waves = 8; waves >= 4; waves -= 4)
        if (gemv_dma_lds(rp, ni, waves, rows_wg, k) <= (160 << 10))
            return waves;
    return 0;
}

template <int RP, int NI>
static int launch_gemv_dma(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows, int rows_wg)
{
    const dim3 grid((unsigned)((m + rows_wg - 1) / rows_wg), (unsigned)((rows + RP - 1) / RP), 1);
    const int waves = gemv_dma_waves(RP, NI, rows_wg, k);
    const size_t lds = (size_t)gemv_dma_lds(RP, NI, waves, rows_wg, k);
    if (waves == 8)
        HIPML_LAUNCH((gemv_q8_dma_kernel<RP, NI, 8>), grid, dim3(512, 1, 1), lds, st, w, x, y, m, k, rows, rows_wg);
    else
        HIPML_LAUNCH((gemv_q8_dma_kernel<RP, NI, 4>), grid, dim3(256, 1, 1), lds, st, w, x, y, m, k, rows, rows_wg);
    return launched("gemv_q8_0_rows");
}

template <int NI>
static int launch_gemv_dma_rows(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows, int rows_wg)
{
    if (rows == 1)
        return launch_gemv_dma<1, NI>(st, w, x, y, m, k, rows, rows_wg);
    if (rows == 2)
        return launch_gemv_dma<2, NI>(st, w, x, y, m, k, rows, rows_wg);
    if (rows <= 4)
        return launch_gemv_dma<4, NI>(st, w, x, y, m, k, rows, rows_wg);
    return launch_gemv_dma<8, NI>(st, w, x, y, m, k, rows, rows_wg);
}

// Up to eight rows over the raw-row kernel: rows of whole 256-value chunks at 16-byte boundaries, addressed with
// 32-bit offsets, and LDS room for every row count (so that all of them take this kernel, or none).  Returns -1
// where the shape does not qualify (the kernels above serve it).
static int try_gemv_dma(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows)
{
    if (rows > 8 || k % 256 != 0 || (reinterpret_cast<uintptr_t>(w) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(x) & 15) != 0 || (size_t)m * (k >> 5) * kQ8Block >= ((size_t)1 << 32) ||
        (size_t)rows * k * sizeof(float) >= ((size_t)1 << 32))
        return -1;
    // the fewest weight rows per workgroup that make one round of the chip's 256 CUs
    static const int kRowsWg[4] = {16, 20, 24, 32}, kNi[4] = {5, 6, 7, 9};
    int v = 3;
    for (int i = 0; i < 4; i++)
        if ((m + kRowsWg[i] - 1) / kRowsWg[i] <= 256) {
            v = i;
            break;
        }
    for (int rp = 1; rp <= 8; rp *= 2)
        if (gemv_dma_waves(rp, kNi[v], kRowsWg[v], k) == 0)
            return -1;
    switch (v) {
    case 0: return launch_gemv_dma_rows<5>(st, w, x, y, m, k, rows, 16);
    case 1: return launch_gemv_dma_rows<6>(st, w, x, y, m, k, rows, 20);
    case 2: return launch_gemv_dma_rows<7>(st, w, x, y, m, k, rows, 24);
    default: return launch_gemv_dma_rows<9>(st, w, x, y, m, k, rows, 32);
    }
}

static int gemv_tile_xt(int rows)
{
    const int pass = rows > 64 ? (rows + 1) / 2 : rows;
    return (pass + 15) / 16;
}

template <int XT, int NI>
static int launch_gemv_dma_tile(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows,
                                int rows_wg)
{
    const dim3 grid((unsigned)((m + rows_wg - 1) / rows_wg), (unsigned)((rows + 16 * XT - 1) / (16 * XT)), 1);
    const size_t lds = (size_t)gemv_dma_tile_lds(XT, NI, rows_wg);
    if (grid.y == 1 && rows <= 16 * XT - 8)
        HIPML_LAUNCH((gemv_q8_dma_tile_kernel<XT, NI, true>), grid, dim3(512, 1, 1), lds, st, w, x, y, m, k, rows, rows_wg);
    else
        HIPML_LAUNCH((gemv_q8_dma_tile_kernel<XT, NI, false>), grid, dim3(512, 1, 1), lds, st, w, x, y, m, k, rows, rows_wg);
    return launched("gemv_q8_0_rows");
}

template <int NI>
static int launch_gemv_dma_tiles(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows,
                                 int rows_wg)
{
    // the activation tiles of a pass: as many as the rows need, up to four; more than 64 rows: two passes (the
    // grid's second dimension) that share the rows evenly
    const int xt = gemv_tile_xt(rows);
    switch (xt) {
    case 1: return launch_gemv_dma_tile<1, NI>(st, w, x, y, m, k, rows, rows_wg);
    case 2: return launch_gemv_dma_tile<2, NI>(st, w, x, y, m, k, rows, rows_wg);
    case 3: return launch_gemv_dma_tile<3, NI>(st, w, x, y, m, k, rows, rows_wg);
    default: return launch_gemv_dma_tile<4, NI>(st, w, x, y, m, k, rows, rows_wg);
    }
}

// 9 rows and more over the raw-row tile kernel, under the conditions of try_gemv_dma.  Returns -1 where the shape
// does not qualify.
static int try_gemv_dma_tile(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows)
{
    if (k % 256 != 0 || (reinterpret_cast<uintptr_t>(w) & 15) != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0 ||
        (size_t)m * (k >> 5) * kQ8Block >= ((size_t)1 << 32) || (size_t)rows * k * sizeof(float) >= ((size_t)1 << 32))
        return -1;
    static const int kRowsWg[4] = {16, 20, 24, 32};
    int v = 3;
    for (int i = 0; i < 4; i++)
        if ((m + kRowsWg[i] - 1) / kRowsWg[i] <= 256) {
            v = i;
            break;
        }
    static const int kNi[4] = {5, 6, 7, 9};
    const int xt = gemv_tile_xt(rows);
    if (gemv_dma_tile_lds(xt, kNi[v], kRowsWg[v]) > (160 << 10))
        return -1;
    switch (v) {
    case 0: return launch_gemv_dma_tiles<5>(st, w, x, y, m, k, rows, 16);
    case 1: return launch_gemv_dma_tiles<6>(st, w, x, y, m, k, rows, 20);
    case 2: return launch_gemv_dma_tiles<7>(st, w, x, y, m, k, rows, 24);
    default: return launch_gemv_dma_tiles<9>(st, w, x, y, m, k, rows, 32);
    }
}

int launch_gemv_q8_rows(hipStream_t st, const uint8_t *w, const float *x, float *y, int m, int k, int rows)
{
    // (10 rows and more: the raw-row tile kernel, in two passes beyond 64; 9 rows measured slower there than in the
    // tile kernel below: 17.2 against 16.0 us at 5120 x 6144)
    const int dma = rows <= 8 ? try_gemv_dma(st, w, x, y, m, k, rows)
                              : (rows >= 10 && rows <= 128 ? try_gemv_dma_tile(st, w, x, y, m, k, rows) : -1);
    if (dma >= 0)
        return dma;
    // three rows or more: full A tiles of 16 or 32 rows (measured at 5120 x 6144, 4 rows: 14.6 us
    // against 16.7 us for the row kernel with two weight tiles per workgroup; 1 row: 13.6 against 12.1)
    if (rows > kGemvMaxRows)
        return rows > 16 ? launch_gemv_tile<8, 2, 2>(st, w, x, y, m, k, rows)
                         : launch_gemv_tile<8, 2, 1>(st, w, x, y, m, k, rows);
    int rp = gemv_rows_per_pass(k);
    if (rp < 1)
        return fail(HIPML_ATTN_E_RANGE, "k %d: one activation row does not fit the LDS operand buffer", k);
    rp = rows < rp ? rows : rp;
    // One 16-row weight tile per workgroup keeps the kernel inside 128 registers, so two workgroups
    // share a CU and the 320 workgroups of a 5120-row matrix start together (workgroups start in
    // windows of as many as fit the chip; a second window opens when the first has drained).
    return launch_gemv_variant<8, 1, 6>(st, w, x, y, m, k, rows, rp);
}


// ---- gemm_q8_f16_kernel: many activation rows (a prefill chunk) ---------------------------------
//
// y[t][row] for a 128 (tokens) x 128 (weight rows) tile per workgroup, MFMA-bound:
// v_mfma_f32_32x32x16_f16 with A = x (f32 -> f16, round to nearest), B = W dequantized to f16 (d*q, one
// rounding: the precision class of the reference's f16-operand prefill kernels and of this library's
// chunk attention), fp32 accumulation.  Four consumer waves, each a 64 x 64 piece (2 x 2 MFMA tiles),
// and eight producer waves that fetch and stage.  A k step is 64 values = one 68-byte pair of blocks per
// weight row; both operand tiles are staged as [128 rows][64 f16] with a 144-byte row pitch (128-bit
// reads and writes of 16 consecutive rows then touch every bank once), double buffered, one barrier
// per step.  A fetch record is refilled as soon as it has been staged.  (One set of four waves doing
// both, interleaved by hand MFMA by MFMA, took 1,600 cycles per step with a single workgroup on the
// CU: every wait left its SIMD idle.)
// Weight fetch uses the lane order of the row kernel above (quad = the four quarters of a pair of
// blocks, dword-aligned loads).
// X16: the activations arrive as f16 (written by gate_f16_kernel below).  With f32 activations a
// step moves 32 KB of them through the CU's 64-byte-per-cycle vector memory path -- more cycles
// than the step's MFMAs take (measured: 700 of a step's 2,200 cycles are spent issuing loads) -- and
// every one of the m/128 workgroups of a token tile repeats that; f16 halves it and drops the
// conversion.


typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

constexpr int kGemmT = 128, kGemmM = 128;
constexpr int kGemmUnits = 1;                     // 64-value units (pairs of blocks) per step
constexpr int kGemmK = 64 * kGemmUnits;           // values per step
constexpr int kGemmPitch = kGemmK * 2 + 16;       // 144: an odd number of 16-byte groups
constexpr int kGemmTile = 128 * kGemmPitch;       // one operand tile
constexpr int kGemmBuf = 2 * kGemmTile;           // x tile + w tile
constexpr int kGemmLds = 2 * kGemmBuf;            // double buffered: 73,728 bytes
constexpr int kGemmWaves = 8;                     // producer waves
constexpr int kGemmCWaves = 4;                    // consumer waves

// What one producer thread fetches for one step: per unit WN weight (row, quarter) pairs, and XN
// 16-byte pieces of the activation tile.
template <int WN, int XN>
struct GemmFetch {
    uint3a4 e[kGemmUnits][WN];   // even-block quarter (+ scales in quad lanes 0 and 3)
    uint2a4 o[kGemmUnits][WN];   // odd-block quarter
    float4v x[XN];               // f32: 4 activations; f16: 8
};

// 8 exact integer f16 times the block scale (f16): the product has at most 19 significant bits and
// is rounded once, as f16(d * q) is.
__device__ __forceinline__ half8 dequant8(uint32_t w0, uint32_t w1, _Float16 d)
{
    const half8 q = int8x8_to_f16(w0, w1);
    const half8 dv = {d, d, d, d, d, d, d, d};
    return q * dv;
}

// kGemmCWaves consumer waves first, then NW producer waves: 4 + 8.  Consumers own 64 x 64 pieces
// (2 x 2 MFMA tiles: every operand read feeds two MFMAs, 64 KB of LDS reads per step instead of the
// 96 KB of eight 32 x 64 pieces), producers one weight (row, quarter) pair and two activation pieces
// per thread and step.  LDS serves a wave at about 34 B/clk for 128-bit reads and 16-20 B/clk for
// 128-bit writes whatever the others do, up to well over 128 B/clk in all (measured), so eight
// producer waves stage a tile in less time than four.  Measured at 5120 x 6144, 672 tokens, gate
// pass included: 4 + 4 waves 77.3, 8 + 8 waves 76.5, 4 + 8 waves 71.6 us.
template <bool X16, int NW>
__global__ void __launch_bounds__(64 * (NW + kGemmCWaves)) gemm_q8_f16_kernel(const uint8_t *__restrict__ w,
                                                              const void *__restrict__ xv,
                                                              float *__restrict__ y, int m, int k, int tokens)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int NT = 64 * NW; // producer threads
    constexpr int NC = kGemmCWaves;
    constexpr int KU = kGemmUnits;
    const bool producer = threadIdx.x >= 64 * NC;
    const int tid = producer ? threadIdx.x - 64 * NC : threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63; // within the role
    const int m0 = blockIdx.x * kGemmM, t0 = blockIdx.y * kGemmT;
    const int nunits = k >> 6;
    const int nsteps = (nunits + KU - 1) / KU;   // the last step may hold fewer units: zero weights
    const size_t row_bytes = (size_t)(k >> 5) * kQ8Block;
    constexpr int WN = 512 / NT;                 // weight (row, quarter) pairs per producer thread and unit
    constexpr int WROWS = NT / 4;                // rows covered by one such pair of the workgroup
    constexpr int XELT = X16 ? 2 : 4;            // bytes per activation
    constexpr int XV = 16 / XELT;                // activations per 16-byte piece
    constexpr int XPR = kGemmK / XV;             // pieces per tile row
    constexpr int XN = 128 * XPR / NT;           // pieces per producer thread
    constexpr int XROWS = NT / XPR;              // rows covered by one piece of the workgroup

    // fetch roles
    const int fr = tid >> 2, fg = tid & 3; // weight rows fr + WROWS h, k quarter fg of each block
    const uint8_t *wp[WN];
#pragma unroll
    for (int h = 0; h < WN; h++) {
        const int row = m0 + fr + WROWS * h < m ? m0 + fr + WROWS * h : m - 1;
        wp[h] = w + (size_t)row * row_bytes + fg * 8;
    }
    // activations: 16 bytes per load, XPR consecutive lanes cover a tile row
    const int xr = tid / XPR, xc = tid % XPR;
    const uint8_t *xp[XN];
#pragma unroll
    for (int i = 0; i < XN; i++) {
        const int t = t0 + xr + XROWS * i < tokens ? t0 + xr + XROWS * i : tokens - 1;
        xp[i] = static_cast<const uint8_t *>(xv) + ((size_t)t * k) * XELT;
    }
    typedef GemmFetch<WN, XN> Fetch;
    auto fetch = [&](Fetch &f, int s) {
        const int sc = s < nsteps ? s : nsteps - 1;
#pragma unroll
        for (int u = 0; u < KU; u++) {
            const int g = sc * KU + u < nunits ? sc * KU + u : nunits - 1;
#pragma unroll
            for (int h = 0; h < WN; h++) {
                const uint8_t *unit = wp[h] + (size_t)g * (2 * kQ8Block);
                f.e[u][h] = *reinterpret_cast<const uint3a4 *>(unit);
                f.o[u][h] = *reinterpret_cast<const uint2a4 *>(unit + 36);
            }
        }
        // a piece past the end of the row (second unit of a short last step) repeats the row's last
        // piece: it meets zero weights
        int kx = sc * kGemmK + xc * XV;
        if (KU > 1)
            kx = kx + XV <= k ? kx : k - XV;
#pragma unroll
        for (int i = 0; i < XN; i++)
            f.x[i] = *reinterpret_cast<const float4v *>(xp[i] + (size_t)kx * XELT);
    };
    auto stage = [&](const Fetch &f, uint8_t *buf, int s) {
        uint8_t *xt = buf, *wt = buf + kGemmTile;
#pragma unroll
        for (int i = 0; i < XN; i++) {
            if (X16) {
                *reinterpret_cast<float4v *>(xt + (xr + XROWS * i) * kGemmPitch + xc * 16) = f.x[i];
            } else {
                // round to nearest even (v_cvt_pk_f16_f32): truncation would bias every product the same way
                const half4v v = __builtin_convertvector(f.x[i], half4v);
                *reinterpret_cast<half4v *>(xt + (xr + XROWS * i) * kGemmPitch + xc * 8) = v;
            }
        }
#pragma unroll
        for (int u = 0; u < KU; u++) {
            const bool live = KU == 1 || s * KU + u < nunits;
#pragma unroll
            for (int h = 0; h < WN; h++) {
                const uint3a4 e = f.e[u][h];
                const uint32_t s0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e[0], 0x00, 0xf, 0xf, true);
                const uint32_t s1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e[2], 0xFF, 0xf, 0xf, true);
                const _Float16 d0 = __builtin_bit_cast(_Float16, (uint16_t)(live ? s0 & 0xffffu : 0u));
                const _Float16 d1 = __builtin_bit_cast(_Float16, (uint16_t)(live ? s1 >> 16 : 0u));
                const half8 v0 = dequant8(__builtin_amdgcn_alignbit(e[1], e[0], 16),
                                          __builtin_amdgcn_alignbit(e[2], e[1], 16), d0);
                const half8 v1 = dequant8(f.o[u][h][0], f.o[u][h][1], d1);
                uint8_t *dst = wt + (fr + WROWS * h) * kGemmPitch + u * 128 + fg * 16;
                *reinterpret_cast<half8 *>(dst) = v0;        // k = fg*8 .. of the even block
                *reinterpret_cast<half8 *>(dst + 64) = v1;   // k = 32 + fg*8 .. (the odd block)
            }
        }
    };

    // MFMA roles: consumer wave (wt, wm) owns AT 32-token tiles from token wt * 32 AT and weight rows
    // wm*64..: 64 x 64 per wave with four consumers, 32 x 64 with eight
    constexpr int AT = 8 / NC;
    const int wt_ = wave >> 1, wm_ = wave & 1;
    const int ln = lane & 31, lh = lane >> 5;
    float16v acc[AT][2];
#pragma unroll
    for (int a = 0; a < AT; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++)
                acc[a][b][i] = 0.0f;
    // All operands of a step are named first and the scheduling groups below pin the order: the reads
    // of the first 16 values of k, then one MFMA and one read in turn, so that a read's LDS latency
    // is covered by MFMAs (left to itself the compiler read, waited, multiplied: 840 cycles per step
    // for 512 of MFMA).
    auto multiply = [&](const uint8_t *buf) {
        const uint8_t *xa = buf + (wt_ * 32 * AT + ln) * kGemmPitch + lh * 16;
        const uint8_t *wb = buf + kGemmTile + (wm_ * 64 + ln) * kGemmPitch + lh * 16;
        half8 A[4 * KU][AT], B[4 * KU][2];
#pragma unroll
        for (int kk = 0; kk < 4 * KU; kk++) {
#pragma unroll
            for (int a = 0; a < AT; a++)
                A[kk][a] = *reinterpret_cast<const half8 *>(xa + a * 32 * kGemmPitch + kk * 32);
#pragma unroll
            for (int b = 0; b < 2; b++)
                B[kk][b] = *reinterpret_cast<const half8 *>(wb + b * 32 * kGemmPitch + kk * 32);
        }
#pragma unroll
        for (int kk = 0; kk < 4 * KU; kk++)
#pragma unroll
            for (int a = 0; a < AT; a++)
#pragma unroll
                for (int b = 0; b < 2; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[kk][a], B[kk][b], acc[a][b], 0, 0, 0);
        constexpr int per = AT + 2;             // reads per 16 values of k
        constexpr int reads = 4 * KU * per, mfmas = 4 * KU * AT * 2;
        __builtin_amdgcn_sched_group_barrier(0x100, per, 0);
#pragma unroll
        for (int i = 0; i < reads - per; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, mfmas - (reads - per), 0);
    };

    // The second half of the waves produce (fetch, dequantize, write the next step's tiles), the first
    // half consume (operand reads and MFMAs of the current step); one barrier per step hands a buffer
    // over.  A SIMD holds waves of both kinds, and a VALU wave and an MFMA wave of one SIMD issue side
    // by side.  (Two units per step, half as many barriers, measured slower: 76.5 against 72.8 us at
    // 672 tokens.)
    if (producer) {
        // Four fetch records in rotation: a record is refilled as soon as it has been staged and is
        // staged again four steps later, so its loads have three steps to arrive (with two records the
        // producers spent 860 cycles of a 1,400-cycle step waiting for them).  Four steps per turn keep
        // the records in the same registers; a fetch past the last step repeats it.
        Fetch r0, r1, r2, r3;
        fetch(r0, 0);
        fetch(r1, 1);
        fetch(r2, 2);
        fetch(r3, 3);
        stage(r0, lds, 0);
        fetch(r0, 4);
        __syncthreads();
        int s = 0;
        for (; s + 4 <= nsteps; s += 4) {
            stage(r1, lds + kGemmBuf, s + 1); // step s + 1, while step s is multiplied
            fetch(r1, s + 5);
            __syncthreads();
            stage(r2, lds, s + 2);
            fetch(r2, s + 6);
            __syncthreads();
            stage(r3, lds + kGemmBuf, s + 3);
            fetch(r3, s + 7);
            __syncthreads();
            stage(r0, lds, s + 4);            // step s + 4
            fetch(r0, s + 8);
            __syncthreads();
        }
        // the last one to three steps: their records are already on the way
        const int rest = nsteps - s;
        if (rest >= 1) {
            if (rest >= 2)
                stage(r1, lds + kGemmBuf, s + 1);
            __syncthreads();
        }
        if (rest >= 2) {
            if (rest >= 3)
                stage(r2, lds, s + 2);
            __syncthreads();
        }
        if (rest >= 3)
            __syncthreads();
        return;
    }
    __syncthreads();
    for (int s = 0; s + 2 <= nsteps; s += 2) {
        multiply(lds);
        __syncthreads();
        multiply(lds + kGemmBuf);
        __syncthreads();
    }
    if (nsteps & 1) {
        multiply(lds);
        __syncthreads();
    }

    // C tile: lane holds column ln (weight row), rows (i/4)*8 + lh*4 + i%4 (tokens)
#pragma unroll
    for (int a = 0; a < AT; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int row = m0 + wm_ * 64 + b * 32 + ln;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int t = t0 + wt_ * 32 * AT + a * 32 + (i >> 2) * 8 + lh * 4 + (i & 3);
                if (t < tokens && row < m)
                    y[(size_t)t * m + row] = acc[a][b][i];
            }
        }
}

// x16[i] = f16(x[i] * sigmoid(gate[i])) (gate may be null: plain conversion), 8 values per thread.
// The gate is the expression every gating kernel of this library uses, the rounding the one the
// f32-activation GEMM applies when it stages x: the two routes give the same bits.
__global__ void __launch_bounds__(256) gate_f16_kernel(const float4v *__restrict__ x,
                                                      const float4v *__restrict__ gate,
                                                      half8 *__restrict__ x16, size_t n8)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8)
        return;
    float4v a = x[2 * i], b = x[2 * i + 1];
    if (gate != nullptr) {
        const float4v ga = gate[2 * i], gb = gate[2 * i + 1];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            a[j] = gated(a[j], ga[j]);
            b[j] = gated(b[j], gb[j]);
        }
    }
    const half4v ha = __builtin_convertvector(a, half4v), hb = __builtin_convertvector(b, half4v);
    half8 h;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        h[j] = ha[j];
        h[4 + j] = hb[j];
    }
    x16[i] = h;
}

template <int WAVES, int TILES, int CH>
static hipError_t raise_gemv_lds()
{
    hipError_t e = hipSuccess;
    auto raise = [&](const void *f) {
        if (e == hipSuccess)
            e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 160 << 10);
    };
    raise(reinterpret_cast<const void *>(&gemv_q8_rows_kernel<WAVES, TILES, CH, 2>));
    raise(reinterpret_cast<const void *>(&gemv_q8_rows_kernel<WAVES, TILES, CH, 4>));
    raise(reinterpret_cast<const void *>(&gemv_q8_rows_kernel<WAVES, TILES, CH, 8>));
    return e;
}

int proj_init()
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q8_f16_kernel<false, kGemmWaves>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q8_f16_kernel<true, kGemmWaves>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLds);
    if (e == hipSuccess)
        e = raise_gemv_lds<8, 1, 6>();
    auto raise = [&](const void *f) {
        if (e == hipSuccess)
            e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 160 << 10);
    };
#define HIPML_RAISE_DMA(ni) \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<1, ni, 8>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<2, ni, 8>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<4, ni, 8>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<8, ni, 8>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<1, ni, 4>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<2, ni, 4>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<4, ni, 4>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_kernel<8, ni, 4>));
    HIPML_RAISE_DMA(5) HIPML_RAISE_DMA(6) HIPML_RAISE_DMA(7) HIPML_RAISE_DMA(9)
#undef HIPML_RAISE_DMA
#define HIPML_RAISE_TILE(ni) \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<1, ni, false>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<2, ni, false>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<3, ni, false>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<4, ni, false>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<1, ni, true>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<2, ni, true>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<3, ni, true>)); \
    raise(reinterpret_cast<const void *>(&gemv_q8_dma_tile_kernel<4, ni, true>));
    HIPML_RAISE_TILE(5) HIPML_RAISE_TILE(6) HIPML_RAISE_TILE(7) HIPML_RAISE_TILE(9)
#undef HIPML_RAISE_TILE
    if (e != hipSuccess)
        return fail((int)e, "hipFuncSetAttribute(projection LDS) failed: %d (%s)", (int)e, hipGetErrorString(e));
    return 0;
}

// x16 != nullptr: gate (optional) and convert into x16 first, then the GEMM over f16 activations;
// x == nullptr: x16 already holds them.
int launch_gemm_q8_f16(hipStream_t st, const uint8_t *w, const float *x, const float *gate, float *y, int m,
                       int k, int tokens, void *x16)
{
    const dim3 grid((unsigned)((m + kGemmM - 1) / kGemmM), (unsigned)((tokens + kGemmT - 1) / kGemmT), 1);
    if (x16 == nullptr) {
        HIPML_LAUNCH((gemm_q8_f16_kernel<false, kGemmWaves>), grid, dim3(64 * (kGemmWaves + kGemmCWaves), 1, 1), kGemmLds,
                           st, w, x, y, m, k, tokens);
        return launched("gemm_q8_0_f16");
    }
    if (x != nullptr) {
        const size_t n8 = (size_t)tokens * k / 8;
        HIPML_LAUNCH(gate_f16_kernel, dim3((unsigned)((n8 + 255) / 256), 1, 1), dim3(256, 1, 1), 0, st,
                           reinterpret_cast<const float4v *>(x), reinterpret_cast<const float4v *>(gate),
                           static_cast<half8 *>(x16), n8);
        int rc = launched("gate_f16");
        if (rc)
            return rc;
    }
    HIPML_LAUNCH((gemm_q8_f16_kernel<true, kGemmWaves>), grid, dim3(64 * (kGemmWaves + kGemmCWaves), 1, 1), kGemmLds, st, w,
                       x16, y, m, k, tokens);
    return launched("gemm_q8_0_f16");
}

} // namespace hipml
