// Causal GQA chunk prefill over a q8_0 KV cache for gfx950 (wave64, MFMA).
//
// Work unit ("task") = 32 query tokens x 1 query head.  The tasks of one KV head are
// numbered token-tile major (task = token_tile * group + head_in_group); a workgroup of 8
// waves takes 8 consecutive tasks (x one key slice when split), one per wave, two waves per
// SIMD.  All 8 tasks share the K/V stream: a tile of 64 keys is fetched as 68-byte units
// (two whole q8_0 blocks of one key per thread, dword-aligned 128-bit loads), dequantized
// once per workgroup to f16 and written to one of two LDS buffers.  The two waves of a SIMD
// run one slot apart, so one does VALU work (dequantization, softmax) while the other issues
// MFMAs; LDS operand reads are pinned two MFMAs ahead with scheduling groups.
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
//
// The same kernel also runs over an f16 copy of the cache (template parameter F16): then nothing is
// dequantized or staged by the waves, whole tiles come in through global_load_lds, and the V tile is
// stored transposed so that the PV operands are plain 128-bit reads.  kv_f16_tiles_kernel makes that copy.
//
// Deep in a prefix the sliced chunk over such tiles is served by chunk_f16_t64_kernel instead: 64 tokens per
// wave, one wave per SIMD, O in the accumulation registers (see there); the cache entry points reach it for
// long chunks by making the tiles in their scratch first (chunk_tiles_plan).

#include "common.h"

#include <type_traits>

namespace hipml {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef short short4v __attribute__((ext_vector_type(4)));

constexpr int kQTile = 32;    // query tokens per task
constexpr int kTasks = 8;     // tasks (= waves) per workgroup
constexpr int kPfThreads = 64 * kTasks;
constexpr int kKTile = 64;    // keys per LDS tile
// f16 rows in LDS: 512 bytes + pad.  528 keeps the K operand's 128-bit reads (lane = row) and
// the staging writes conflict free; 544 does the same for the V transpose reads (8 rows x 64
// bytes per instruction) at the price of 2-way conflicts on V's staging writes.
constexpr int kKRow = 528;
constexpr int kVRow = 544;
constexpr int kVOff = kKTile * kKRow;                  // V tile follows the K tile
constexpr int kBufBytes = kKTile * (kKRow + kVRow);    // 68,608
constexpr int kQLdsSteps = 3;                          // d-steps of the Q operand parked in LDS
constexpr int kQLdsOff = 2 * kBufBytes;                // after the two tile buffers (137,216)
constexpr int kPfLds = kQLdsOff + kTasks * kQLdsSteps * 1024; // 161,792 of 163,840
// The f16 copy of a cache (hipml_kv_f16_rows): per KV head and 64-key tile, the K rows as they lie in
// LDS (pitch kKRow) and the V rows transposed, [256 d][64 keys in operand order] with a pitch of 144
// bytes (128-bit reads of 32 consecutive rows fall into distinct banks).  A tile is then one
// contiguous piece of memory that global_load_lds copies to LDS as it is.
constexpr int kVtRow = 144;
constexpr int kKTileBytes = kKTile * kKRow;              // 33,792
constexpr int kVtTileBytes = kHeadDim * kVtRow;          // 36,864
constexpr int kBufBytesF = kKTileBytes + kVtTileBytes;   // 70,656
constexpr int kTilesLds = kKTile * kVRow;                // 34,816: one staged tile of kv_f16_tiles_kernel (the V pitch is the larger)
constexpr int kPfLdsF = 2 * kBufBytesF;                  // 141,312: no Q steps parked, the staging registers are free
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kPfLazy = 8.0f; // growth of a maximum (log2 units) that moves the reference exponent of chunk_q8_kernel

struct ChunkArgs {
    const float *q;
    const uint8_t *kc;
    const uint8_t *vc;
    const uint8_t *k16; // f16 copy of the cache (F16 kernels): K tiles, [n_kv][tile_stride][kKTileBytes]
    const uint8_t *vt;  //                                      V^T tiles, [n_kv][tile_stride][kVtTileBytes]
    int tile_stride;    // tiles per KV head in the copy
    float *out;
    _Float16 *out16;   // chunk_wg_kernel only: if set, the finished rows go here as f16 instead of to `out`
    const float *rope_tab; // chunk_wg_kernel<., true> only: cos/sin table [position][32][2]; q holds unrotated rows
    const float *gate; // optional [tokens][n_head][256]: out = attention * sigmoid(gate)
    float *part_acc;
    float *part_ml;
    int n_head, n_kv, group;
    int pos0, tokens, stride, splits, qslots;
    int ntask;  // tasks per KV head = ceil(tokens/32) * group
    int nblock; // task blocks per KV head = ceil(ntask/8)
    // Key slices per task block.  A block whose last token sees few keys (the early blocks of a
    // chunk near position 0) is cut into fewer slices than `splits`: slices(block) =
    // min(splits, ceil(tiles(block) / slice_tiles)); a block with one slice writes its final
    // output itself.  nslice = sum over blocks; uniform = every block has `splits` slices.
    int slice_tiles, nslice, uniform;
    float scale_log2;
};

// Half of a 68-byte unit [s0 | 32 x i8 | s1 | 32 x i8] of a key row, as the nine dwords that cover
// one block: dwords 0..8 for the first block (scale in the low half of dword 0), dwords 8..16 for
// the second (scale in the high half of dword 8, payload dword-aligned behind it).
struct Half {
    uint4v p, q;
    uint32_t r; // dword 8 of the unit, in both halves
};

__device__ __forceinline__ void load_half0(Half &h, const uint8_t *u)
{
    h.p = *reinterpret_cast<const uint4a4 *>(u);
    h.q = *reinterpret_cast<const uint4a4 *>(u + 16);
    h.r = *reinterpret_cast<const uint32_t *>(u + 32);
}

__device__ __forceinline__ void load_half1(Half &h, const uint8_t *u)
{
    h.r = *reinterpret_cast<const uint32_t *>(u + 32);
    h.p = *reinterpret_cast<const uint4a4 *>(u + 36);
    h.q = *reinterpret_cast<const uint4a4 *>(u + 52);
}

// q4_0: a unit is 36 bytes [s0 | 16 bytes | s1 | 16 bytes] at a dword boundary; one block is the
// five dwords 0..4 (scale in the low half of dword 0) or 4..8 (scale in the high half of dword 4,
// payload dword-aligned behind it).  Byte j of a block carries element j in its low nibble and
// element j + 16 in its high nibble (crates/hipml-core/src/kv.rs:201-218).
struct Half4 {
    uint4v p;
    uint32_t r; // dword 4 of the unit, in both halves
};

__device__ __forceinline__ void load_half0(Half4 &h, const uint8_t *u)
{
    h.p = *reinterpret_cast<const uint4a4 *>(u);
    h.r = *reinterpret_cast<const uint32_t *>(u + 16);
}

__device__ __forceinline__ void load_half1(Half4 &h, const uint8_t *u)
{
    h.r = *reinterpret_cast<const uint32_t *>(u + 16);
    h.p = *reinterpret_cast<const uint4a4 *>(u + 20);
}

template <bool Q4> struct HalfOf { typedef Half type; };
template <> struct HalfOf<true> { typedef Half4 type; };

// 16 int8 -> 16 f16 (value * d), d an f16 scale: the bytes become 1024 + (b+128)
// in f16 by bit tricks, the bias is subtracted exactly, then one packed multiply
// rounds d*b once -- the same value as (f16)((float)d * (float)b).
// (OFFSET 128: int8 bytes, sign bit flipped first; OFFSET 8: unsigned nibbles 0..15, one per byte.)
template <int OFFSET = 128>
__device__ __forceinline__ void dequant16(uint4v raw, _Float16 d, uint4v &lo, uint4v &hi)
{
    const half2v bias = {(_Float16)(1024.0f + OFFSET), (_Float16)(1024.0f + OFFSET)};
    const half2v dd = {d, d};
    uint32_t o[8];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t x = OFFSET == 128 ? raw[w] ^ 0x80808080u : raw[w];
        const uint32_t a = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u); // [0x64,b1,0x64,b0]
        const uint32_t b = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u); // [0x64,b3,0x64,b2]
        o[2 * w] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(half2v, a) - bias) * dd);
        o[2 * w + 1] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(half2v, b) - bias) * dd);
    }
    lo = (uint4v){o[0], o[1], o[2], o[3]};
    hi = (uint4v){o[4], o[5], o[6], o[7]};
}

// Dequantize one block of a unit (block 2*pr or 2*pr+1 of one key) into its 64 bytes of the
// unit's 128 bytes of f16 at `dst`.
__device__ __forceinline__ void stage_block0(const Half &h, uint8_t *dst)
{
    uint4v e0, e1;
    e0[0] = __builtin_amdgcn_alignbit(h.p[1], h.p[0], 16);
    e0[1] = __builtin_amdgcn_alignbit(h.p[2], h.p[1], 16);
    e0[2] = __builtin_amdgcn_alignbit(h.p[3], h.p[2], 16);
    e0[3] = __builtin_amdgcn_alignbit(h.q[0], h.p[3], 16);
    e1[0] = __builtin_amdgcn_alignbit(h.q[1], h.q[0], 16);
    e1[1] = __builtin_amdgcn_alignbit(h.q[2], h.q[1], 16);
    e1[2] = __builtin_amdgcn_alignbit(h.q[3], h.q[2], 16);
    e1[3] = __builtin_amdgcn_alignbit(h.r, h.q[3], 16);
    const _Float16 s0 = __builtin_bit_cast(_Float16, (uint16_t)(h.p[0] & 0xffffu));
    uint4v *d4 = reinterpret_cast<uint4v *>(dst);
    uint4v x0, x1;
    dequant16(e0, s0, x0, x1);
    d4[0] = x0;
    d4[1] = x1;
    dequant16(e1, s0, x0, x1);
    d4[2] = x0;
    d4[3] = x1;
}

__device__ __forceinline__ void stage_block1(const Half &h, uint8_t *dst)
{
    const _Float16 s1 = __builtin_bit_cast(_Float16, (uint16_t)(h.r >> 16));
    uint4v *d4 = reinterpret_cast<uint4v *>(dst);
    uint4v x0, x1;
    dequant16(h.p, s1, x0, x1);
    d4[4] = x0;
    d4[5] = x1;
    dequant16(h.q, s1, x0, x1);
    d4[6] = x0;
    d4[7] = x1;
}

__device__ __forceinline__ void stage_block0(const Half4 &h, uint8_t *dst)
{
    uint4v e;
    e[0] = __builtin_amdgcn_alignbit(h.p[1], h.p[0], 16);
    e[1] = __builtin_amdgcn_alignbit(h.p[2], h.p[1], 16);
    e[2] = __builtin_amdgcn_alignbit(h.p[3], h.p[2], 16);
    e[3] = __builtin_amdgcn_alignbit(h.r, h.p[3], 16);
    const uint4v mask = {0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu};
    const _Float16 s0 = __builtin_bit_cast(_Float16, (uint16_t)(h.p[0] & 0xffffu));
    uint4v *d4 = reinterpret_cast<uint4v *>(dst);
    uint4v x0, x1;
    dequant16<8>(e & mask, s0, x0, x1);        // elements 0..15
    d4[0] = x0;
    d4[1] = x1;
    dequant16<8>((e >> 4) & mask, s0, x0, x1); // elements 16..31
    d4[2] = x0;
    d4[3] = x1;
}

__device__ __forceinline__ void stage_block1(const Half4 &h, uint8_t *dst)
{
    const uint4v mask = {0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu};
    const _Float16 s1 = __builtin_bit_cast(_Float16, (uint16_t)(h.r >> 16));
    uint4v *d4 = reinterpret_cast<uint4v *>(dst);
    uint4v x0, x1;
    dequant16<8>(h.p & mask, s1, x0, x1);
    d4[4] = x0;
    d4[5] = x1;
    dequant16<8>((h.p >> 4) & mask, s1, x0, x1);
    d4[6] = x0;
    d4[7] = x1;
}

// Number of key slices of task block tb (see ChunkArgs::slice_tiles); *seq_block receives the number
// of keys its last token sees.
__device__ __host__ __forceinline__ int block_slices(int tb, int ntask, int group, int tokens, int pos0,
                                                     int splits, int slice_tiles, int *seq_block)
{
    const int last_task = tb * kTasks + kTasks - 1 < ntask ? tb * kTasks + kTasks - 1 : ntask - 1;
    const int tt_last = last_task / group;
    const int last_tok = ((tt_last + 1) * kQTile < tokens ? (tt_last + 1) * kQTile : tokens) - 1;
    const int seq = pos0 + last_tok + 1;
    if (seq_block)
        *seq_block = seq;
    const int tiles = (seq + kKTile - 1) / kKTile;
    const int n = (tiles + slice_tiles - 1) / slice_tiles;
    return n < 1 ? 1 : (n < splits ? n : splits);
}

// max(x[lane], x[lane ^ 32]) without going through LDS: swapping the upper half of one copy
// with the lower half of another leaves {lo, lo} and {hi, hi}.  (Written as asm: the
// compiler's builtin for this instruction returns its first result twice.)
__device__ __forceinline__ float xor32_max(float x)
{
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load (vmcnt(0)), which would expose the full latency of the next tile's
// prefetch at each phase boundary; here only LDS operations are drained.
// It is also a fence for the instruction scheduler: the slots of the tile loop only overlap as
// planned if each slot's VALU work and MFMA work stay on their own side of the barrier.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ uint32_t lds_address(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// 64 lanes x 16 bytes from base + voff (per lane) to LDS address lds_at + 16 * lane, not through
// registers.  The compiler neither knows nor waits for these loads: s_waitcnt vmcnt(n) by hand.
__device__ __forceinline__ void dma16(uint32_t lds_at, const uint8_t *base, uint32_t voff)
{
    // (both are the same in every lane; taking them from the first one tells the compiler so)
    const uint32_t at = __builtin_amdgcn_readfirstlane(lds_at);
    const uint64_t b = (uint64_t)(uintptr_t)base;
    // (the builtin returns an int: without the casts its low half would be sign-extended over the high one)
    const uint64_t bu = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32)) << 32);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(at), "v"(voff), "s"(bu)
                 : "memory");
}

// F16: K and V come from the f16 copy of the cache (a.k16, a.vt), tile by tile through
// global_load_lds, instead of being dequantized by this workgroup.
template <bool SPLIT, bool Q4 = false, bool F16 = false>
__global__ void __launch_bounds__(kPfThreads, 2) chunk_q8_kernel(const ChunkArgs a)
{
    static_assert(!(F16 && Q4), "the f16 copy has one format");
    constexpr int kBuf = F16 ? kBufBytesF : kBufBytes;  // one tile buffer
    constexpr int kVAt = F16 ? kKTileBytes : kVOff;     // V tile inside it
    constexpr int kQSteps = F16 ? 0 : kQLdsSteps;       // Q steps parked in LDS
    typedef typename HalfOf<Q4>::type Half;
    constexpr int kRowBytes = Q4 ? hipml::kRowBytesQ4 : hipml::kRowBytes;
    constexpr int kUnitBytes = Q4 ? 36 : 68;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int ln = lane & 31;  // MFMA column: token within the tile
    const int lh = lane >> 5;  // k half-group
    // Waves w and w+4 share a SIMD.  Set 0 (waves 0..3) and set 1 (waves 4..7) run the same
    // program half an iteration apart: while one set issues MFMAs (PV of tile t, scores of
    // tile t+1) the other does its VALU work (softmax, dequantization of the next tile).
    // Set 0 stages the K tiles, set 1 the V tiles.
    const int set = wave >> 2;

    // blockIdx.x -> (kv head, key slice, task block).  Consecutive workgroups go to different
    // XCDs (8 of them, each with its own L2); the workgroups that stream the same (kv head,
    // slice) are therefore placed 8 apart, so that slice's K/V rows pass through one L2.
    int kvh, split, tb, nsp = 1;
    if (!SPLIT || a.uniform) {
        const int combos = a.n_kv * (SPLIT ? a.splits : 1);
        const int bid = blockIdx.x;
        int combo;
        if (combos % 8 == 0) {
            const int per = combos / 8;
            const int xcd = bid & 7, j = bid >> 3;
            combo = xcd + 8 * (j % per);
            tb = j / per;
        } else if (8 % combos == 0) {
            const int xcd = bid & 7, j = bid >> 3;
            const int share = 8 / combos; // XCDs per combo
            combo = xcd % combos;
            tb = j * share + xcd / combos;
        } else {
            combo = bid % combos;
            tb = bid / combos;
        }
        kvh = combo % a.n_kv;
        split = combo / a.n_kv;
        nsp = SPLIT ? a.splits : 1;
        if (tb >= a.nblock)
            return; // uniform over the workgroup
    } else {
        // per-block slice counts: workgroup -> (kv head, slice index), the slice index is resolved
        // to (block, slice of the block) by walking the blocks
        kvh = blockIdx.x % a.n_kv;
        int sl = blockIdx.x / a.n_kv;
        if (sl >= a.nslice)
            return;
        tb = 0;
        for (;;) {
            nsp = block_slices(tb, a.ntask, a.group, a.tokens, a.pos0, a.splits, a.slice_tiles, nullptr);
            if (sl < nsp)
                break;
            sl -= nsp;
            tb++;
        }
        split = sl;
    }

    const int task = tb * kTasks + wave;
    const bool task_valid = task < a.ntask;
    const int tt = (task_valid ? task : a.ntask - 1) / a.group;
    const int hq = (task_valid ? task : a.ntask - 1) - tt * a.group;
    const int head = kvh * a.group + hq;
    const int t0 = tt * kQTile;

    // visible key range of this workgroup: up to the last token of its last task
    const int last_task = (tb * kTasks + kTasks - 1 < a.ntask ? tb * kTasks + kTasks - 1 : a.ntask - 1);
    const int tt_last = last_task / a.group;
    const int last_tok = ((tt_last + 1) * kQTile < a.tokens ? (tt_last + 1) * kQTile : a.tokens) - 1;
    const int seq_block = a.pos0 + last_tok + 1;
    int klo = 0, khi = seq_block;
    if (SPLIT && F16) {
        // whole tiles: the transposed V tiles of the copy start at multiples of kKTile
        const int tiles_block = (seq_block + kKTile - 1) / kKTile;
        klo = (int)((long long)tiles_block * split / nsp) * kKTile;
        khi = (int)((long long)tiles_block * (split + 1) / nsp) * kKTile;
        khi = khi < seq_block ? khi : seq_block;
    } else if (SPLIT) {
        klo = (int)((long long)seq_block * split / nsp);
        khi = (int)((long long)seq_block * (split + 1) / nsp);
    }
    const int tok = t0 + ln;
    const int my_last_key = a.pos0 + tok;               // inclusive causal bound of this lane's token
    const int task_last_key = a.pos0 + t0 + kQTile - 1; // of the task's last token
    const bool tok_valid = task_valid && tok < a.tokens;
    const int ntile = khi > klo ? (khi - klo + kKTile - 1) / kKTile : 0;

    // ---- staging role: thread -> one 68-byte unit of the K tile (set 0) or V tile (set 1) ----
    // A wave of the set covers 16 rows x 4 units.  Eight consecutive lanes take 4 rows x 2 units, so
    // that their 128-bit LDS writes (a unit's chunks are 128 bytes apart between units, rows are
    // 528 / 544 bytes apart) fall into distinct banks; the wave still reads 16 whole contiguous rows.
    const int su = threadIdx.x & 255;
    const int srow = (su >> 6) * 16 + ((su >> 1) & 7) + ((su >> 5) & 1) * 8;
    const int spr = (su & 1) | ((su >> 3) & 2);
    const uint8_t *sbase = (set ? a.vc : a.kc) + (size_t)kvh * a.stride * kRowBytes + spr * kUnitBytes;
    const int sdst = set ? kVOff + srow * kVRow + spr * 128 : srow * kKRow + spr * 128;
    // One block of the unit is in flight at a time: block 0 of tile t+1 travels during the MFMA slot
    // M2(t-1) and is dequantized in V1(t), block 1 travels during M1(t) and is dequantized in V2(t).
    // (Past the last tile the loads repeat the last key: issuing unconditionally keeps the loads'
    // registers out of a branch, where the compiler would copy them right behind the loads and wait
    // for memory to do it.)
    Half half;
    auto unit_ptr = [&](int t) {
        int key = klo + t * kKTile + srow;
        key = key < khi ? key : khi - 1;
        return sbase + (size_t)key * kRowBytes;
    };
    auto issue0 = [&](int t) {
        if constexpr (!F16)
            load_half0(half, unit_ptr(t));
    };
    auto issue1 = [&](int t) {
        if constexpr (!F16)
            load_half1(half, unit_ptr(t));
    };
    auto stage0 = [&](int t) {
        if constexpr (!F16)
            stage_block0(half, lds + (t & 1) * kBuf + sdst);
    };
    auto stage1 = [&](int t) {
        if constexpr (!F16)
            stage_block1(half, lds + (t & 1) * kBuf + sdst);
    };
    Half first1; // block 1 of the first tile: fetched together with block 0, ahead of the Q loads
    if (!F16 && ntile > 0) {
        issue0(0);
        load_half1(first1, unit_ptr(0));
    }
    // F16: tile t of the slice is tile klo / kKTile + t of the copy, one contiguous piece per K and per
    // V^T tile; the 33 (K) and 36 (V^T) KiB go as 1-KiB requests i = wave, wave + 8, ..., five per wave
    // and tile (the last ones repeat the tile's last KiB, so that every wave's count is the same and
    // the waits below are constants).  A tile past the slice's last repeats that one: it lands in the
    // buffer nobody reads any more.
    constexpr int kDmaPerTile = 5;
    const uint32_t lds_at = lds_address(lds); // (lane l's 16 bytes land at the request's address + 16 l)
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto dma_tile = [&](int t, bool v_tile) {
        if constexpr (F16) {
            const int tc = t < ntile ? t : ntile - 1;
            const size_t tile = (size_t)kvh * a.tile_stride + (klo / kKTile + tc);
            const uint8_t *src = v_tile ? a.vt + tile * kVtTileBytes : a.k16 + tile * kKTileBytes;
            const int last = (v_tile ? kVtTileBytes : kKTileBytes) / 1024 - 1;
            const uint32_t dst = lds_at + (t & 1) * kBuf + (v_tile ? kVAt : 0);
#pragma unroll
            for (int j = 0; j < kDmaPerTile; j++) {
                int i = wave_u + 8 * j;
                i = i < last ? i : last;
                dma16(dst + i * 1024, src + i * 1024, lane * 16);
            }
        }
    };
    auto dma_wait_oldest = [&]() { // all but the newest tile's requests have landed
        if constexpr (F16)
            asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
    };
    auto dma_wait_all = [&]() {
        if constexpr (F16)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // ---- Q^T operand: 16 k-steps of 8 f16 (d = ks*16 + lh*8 + j) ---------------------------
    // Steps 0..kQLdsSteps-1 are parked in this wave's corner of LDS and re-read per use: 256
    // registers do not hold O (128), all of Q (64), the scores, the tile prefetch and the operand
    // pipeline at once, and what the compiler would spill instead goes to scratch memory.
    //
    // The rows are fetched whole (one instruction = one token's 256 floats of this head, 1 KB
    // contiguous), converted and transposed through this wave's 16.5 KB corner of the tile buffers,
    // which are still unused: a lane-per-token fetch of 16-byte pieces from rows 24 KB apart took
    // several times longer to arrive.  The operand is then read back with the K tile's pattern.
    half8 qf[16];
    uint8_t *qlds = lds + kQLdsOff + wave * kQLdsSteps * 1024 + lane * 16; // (unused when no step is parked)
    {
        uint8_t *qt = lds + wave * (kQTile * kKRow);
        const float *qh = a.q + (size_t)head * kHeadDim + lane * 4;
        const size_t tok_stride = (size_t)a.n_head * kHeadDim;
#pragma unroll
        for (int b = 0; b < 2; b++) {
            float4v f[16];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int tr = t0 + b * 16 + i;
                f[i] = *reinterpret_cast<const float4v *>(qh + (size_t)(tr < a.tokens ? tr : a.tokens - 1) * tok_stride);
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                half4 h;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    h[j] = (_Float16)f[i][j];
                *reinterpret_cast<half4 *>(qt + (b * 16 + i) * kKRow + lane * 8) = h;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's own writes
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            const half8 h = *reinterpret_cast<const half8 *>(qt + ln * kKRow + ks * 32 + lh * 16);
            if (ks < kQSteps)
                *reinterpret_cast<half8 *>(qlds + ks * 1024) = h;
            else
                qf[ks] = h;
        }
    }
    __syncthreads(); // every wave has its Q: the tile buffers may now take the first tile

    float16v O[8];
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            O[t][i] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;
    float16v S;   // scores of the half that is next in line for softmax
    half8 P[2];   // its probabilities, as the PV product's B operand

    // V transpose-read geometry: 16-lane group G = lane/16 covers d rows (G&1)*16.. of the
    // 32-row tile and k half-group lh = G>>1; lane L of the group supplies key (L/4), d run (L%4)*4.
    const int gl = lane & 15;
    const int vtr_off = kVAt + (gl >> 2) * kVRow + (((lane >> 4) & 1) * 16 + (gl & 3) * 4) * 2;

    // a 32-key half of tile t that this task can see at all (wave-uniform)
    auto live = [&](int t, int hk) {
        const int k0 = klo + t * kKTile + hk * 32;
        return task_valid && k0 <= task_last_key && k0 < khi;
    };

    // ---- S^T = K . Q^T for half hk of tile t ------------------------------------------------------
    // The 16 MFMAs form one accumulation chain; their A operands are read from LDS two steps
    // ahead, and the scheduling groups below pin that interleaving (read, then MFMA) so an
    // operand's LDS latency is covered by the two MFMAs in front of it.
    auto scores = [&](int t, int hk) {
        if (!live(t, hk))
            return;
        const uint8_t *Kh = lds + (t & 1) * kBuf + hk * 32 * kKRow + ln * kKRow + lh * 16;
        float16v acc;
#pragma unroll
        for (int i = 0; i < 16; i++)
            acc[i] = 0.0f;
        half8 A[16], B[kQSteps > 0 ? kQSteps : 1];
#pragma unroll
        for (int ks = 0; ks < kQSteps; ks++)
            B[ks] = *reinterpret_cast<const half8 *>(qlds + ks * 1024);
#pragma unroll
        for (int ks = 0; ks < 16; ks++)
            A[ks] = *reinterpret_cast<const half8 *>(Kh + ks * 32);
#pragma unroll
        for (int ks = 0; ks < 16; ks++)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[ks], ks < kQSteps ? B[ks] : qf[ks], acc,
                                                         0, 0, 0);
        S = acc;
        __builtin_amdgcn_sched_group_barrier(0x100, 2 + kQSteps, 0); // operands of the first steps
#pragma unroll
        for (int ks = 0; ks < 14; ks++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // 1 MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // 1 LDS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    };

    // ---- online softmax of half hk of tile t; lane holds keys (i/4)*8 + lh*4 + i%4 ---------------
    auto softmax = [&](int t, int hk) {
        if (!live(t, hk))
            return;
        const int k0 = klo + t * kKTile + hk * 32;
        const bool need_mask = (k0 + 31 > a.pos0 + t0) || (k0 + 32 > khi);
        if (need_mask) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int kg = k0 + (i >> 2) * 8 + lh * 4 + (i & 3);
                S[i] = (kg <= my_last_key && kg < khi) ? S[i] : -INFINITY;
            }
        }
        float mt = S[0];
#pragma unroll
        for (int i = 1; i < 16; i++)
            mt = fmaxf(mt, S[i]);
        mt = xor32_max(mt) * a.scale_log2;
        // m_run is the exponent the sums are held against, not the running maximum: it follows the maximum
        // only when some token's maximum has grown by more than kPfLazy since it was set.  Deep in a long
        // prefix a token of the 32 still finds a new maximum in every third tile, and each time the 128
        // accumulator registers would be rescaled; until the exponent moves, probabilities may be as
        // large as 2^kPfLazy, which f16 holds with the same relative precision.
        if (__any(mt > m_run + kPfLazy)) {
            const float m_new = fmaxf(m_run, mt);
            const float corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= corr;
#pragma unroll
            for (int dt = 0; dt < 8; dt++)
                O[dt] *= corr;
            m_run = m_new;
        }
        const float mneg = m_run == -INFINITY ? 0.0f : -m_run;
        float ls = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float e = __builtin_amdgcn_exp2f(fmaf(S[i], a.scale_log2, mneg));
            ls += e;
            P[i >> 3][i & 7] = (_Float16)e;
        }
        l_run += ls;
        // computed here, in the VALU slot, not where the MFMA slot first reads them
        asm volatile("" : "+v"(P[0]), "+v"(P[1]), "+v"(l_run), "+v"(m_run));
    };

    // ---- O^T += V^T . P^T for half hk of tile t ---------------------------------------------------
    // 16 MFMAs into 8 accumulators; each A operand is two transpose reads, issued two MFMAs ahead.
    // F16: the first two V operands of a PV product are read at the end of the VALU slot in front of it
    // (the tile has been in LDS for a slot by then), so that the MFMA slot opens with an MFMA and not
    // with the latency of an LDS read: 4.32 against 4.37 ms at 2,048 @ 100,000.  (The kernel over the
    // cache has no registers left for that.)
    half8 preA[2];
    auto pre_pv = [&](int t, int hk) {
        if constexpr (F16) {
            if (!live(t, hk))
                return;
            const uint8_t *Vt = lds + (t & 1) * kBuf + kVAt + ln * kVtRow + (hk * 32 + lh * 8) * 2;
            preA[0] = *reinterpret_cast<const half8 *>(Vt);
            preA[1] = *reinterpret_cast<const half8 *>(Vt + 32 * kVtRow);
        }
    };
    auto pv = [&](int t, int hk) {
        if (!live(t, hk))
            return;
        half8 A[16];
        if constexpr (F16) {
            // row d of the transposed tile holds the keys in operand order: one 128-bit read per operand
            const uint8_t *Vt = lds + (t & 1) * kBuf + kVAt + ln * kVtRow + (hk * 32 + lh * 8) * 2;
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int dt = 0; dt < 8; dt++)
                    A[u * 8 + dt] = (u == 0 && dt < 2) ? preA[dt] : *reinterpret_cast<const half8 *>(Vt + dt * 32 * kVtRow + u * 32);
        } else {
            const uint8_t *Vh = lds + (t & 1) * kBuf + vtr_off + hk * 32 * kVRow;
#pragma unroll
            for (int u = 0; u < 2; u++) {
#pragma unroll
                for (int dt = 0; dt < 8; dt++) {
                    // keys of read q: (2u+q)*8 + lh*4 + {0..3}
                    const uint8_t *vp = Vh + dt * 64;
                    const short4v r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (short4v __attribute__((address_space(3))) *)(vp + ((2 * u) * 8 + lh * 4) * kVRow));
                    const short4v r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (short4v __attribute__((address_space(3))) *)(vp + ((2 * u + 1) * 8 + lh * 4) * kVRow));
                    const half4 h0 = __builtin_bit_cast(half4, r0);
                    const half4 h1 = __builtin_bit_cast(half4, r1);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        A[u * 8 + dt][j] = h0[j];
                        A[u * 8 + dt][4 + j] = h1[j];
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int dt = 0; dt < 8; dt++)
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[u * 8 + dt], P[u], O[dt], 0, 0, 0);
        constexpr int kReads = F16 ? 1 : 2; // LDS reads per operand
        if (!F16)
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * kReads, 0); // 2 operands up front
#pragma unroll
        for (int k = 0; k < 14; k++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    };

    // Tile t lives in LDS buffer t & 1.  A tile takes four slots, each closed by a barrier:
    //   V1: dequantize block 0 of this thread's unit of tile t+1, fetch its block 1, softmax of half 0
    //   M1: PV of half 0, scores of half 1                                                   (MFMA)
    //   V2: dequantize block 1, fetch block 0 of tile t+2, softmax of half 1
    //   M2: PV of half 1, scores of half 0 of tile t+1                                       (MFMA)
    // The dequantization is split so that the two VALU slots are equally long (a slot lasts as long
    // as the longer of one set's VALU work and the other set's MFMA work), and each fetch goes out
    // as soon as its registers are free, ahead of the softmax, so that it travels while this wave
    // still has VALU work and through one MFMA slot.
    // Set 1 runs one slot behind set 0 (it passes one extra barrier first, set 0 one extra at
    // the end), so in every slot one set of each SIMD issues MFMAs while the other does VALU work.
    // Hazards: set 0 writes K(t+1) in its V1(t) and V2(t); the K(t-1) it replaces was last read in
    // M1(t-1), which set 1 finished one slot before V1(t), and K(t+1) is first read in M2(t).  Set 1
    // writes V(t+1) in its V1(t) and V2(t), which are set 0's M1(t) and M2(t); the V(t-1) it replaces
    // was last read in M2(t-1), finished by both sets before that, and V(t+1) is first read in M1(t+1).
    if constexpr (F16) {
        // K(t + 1) is requested at the head of the slot M2(t - 1) and waited for at the end of M1(t) (three
        // slots to arrive in), V(t + 1) at the head of M1(t) and the end of V2(t) (two slots: the set that
        // runs ahead reads its first V operands in V1(t + 1), which is the other set's M2(t), so every wave's
        // share must have landed one barrier before that); the buffer a tile lands in was last read one
        // slot before the request, by either set.
        dma_tile(0, false);
        dma_tile(0, true);
        dma_tile(1, false);
        dma_wait_oldest();
    } else if (ntile > 0) {
        stage0(0);
        stage_block1(first1, lds + sdst);
        issue0(1);
    }
    lds_barrier();
    if (set == 1)
        lds_barrier();
    if (ntile > 0)
        scores(0, 0);
    lds_barrier();
    for (int t = 0; t < ntile; t++) {
        if (t + 1 < ntile)
            stage0(t + 1);
        issue1(t + 1);
        softmax(t, 0);
        pre_pv(t, 0);
        lds_barrier();
        dma_tile(t + 1, true);
        pv(t, 0);
        scores(t, 1);
        dma_wait_oldest();
        lds_barrier();
        if (t + 1 < ntile)
            stage1(t + 1);
        issue0(t + 2);
        softmax(t, 1);
        pre_pv(t, 1);
        dma_wait_all(); // V(t + 1), before the barrier after which the other set reads it ahead of its M1(t + 1)
        lds_barrier();
        dma_tile(t + 2, false);
        pv(t, 1);
        if (t + 1 < ntile)
            scores(t + 1, 0);
        lds_barrier();
    }
    if (set == 0)
        lds_barrier();
    if constexpr (F16)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the tile buffers are about to be reused

    // ---- epilogue --------------------------------------------------------------------------
    l_run += __shfl_xor(l_run, 32);
    if (SPLIT && nsp > 1) {
        // Partials leave through LDS: a lane holds 16-byte pieces of its token's row, 32 rows apart in
        // memory per store; turned round in this wave's corner of the (now unused) tile buffers, a
        // store instruction covers two half rows of 512 contiguous bytes.  Two passes of 128 d.
        lds_barrier(); // every wave has finished with the tiles (nsp is uniform over the workgroup)
        constexpr int kPitch = 512 + 16;
        uint8_t *mine = lds + wave * (kQTile * kPitch);
        const int l32 = lane & 31, rsel = lane >> 5;
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
#pragma unroll
            for (int dl = 0; dl < 4; dl++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int dt = hf * 4 + dl;
                    const float4v x = {O[dt][g * 4], O[dt][g * 4 + 1], O[dt][g * 4 + 2], O[dt][g * 4 + 3]};
                    *reinterpret_cast<float4v *>(mine + ln * kPitch + (dl * 32 + g * 8 + lh * 4) * 4) = x;
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's own writes
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int r2 = 0; r2 < 16; r2++) {
                const int r = r2 * 2 + rsel; // token of the tile
                const float4v x = *reinterpret_cast<const float4v *>(mine + r * kPitch + l32 * 16);
                if (task_valid && t0 + r < a.tokens) {
                    const size_t prow = ((size_t)split * a.qslots + (t0 + r)) * a.n_head + head;
                    *reinterpret_cast<float4v *>(a.part_acc + prow * kHeadDim + hf * 128 + l32 * 4) = x;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // reads done before the next pass overwrites
            __builtin_amdgcn_wave_barrier();
        }
        if (tok_valid && lh == 0) {
            const size_t row = ((size_t)split * a.qslots + tok) * a.n_head + head;
            a.part_ml[row * 2] = m_run;
            a.part_ml[row * 2 + 1] = l_run;
        }
        return;
    }
    if (!tok_valid)
        return;
    {
        const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
        const size_t orow = ((size_t)tok * a.n_head + head) * kHeadDim;
        float *po = a.out + orow;
        // (with key slices the merge kernel gates every row, also the ones written here: it runs at
        // full occupancy, where the exponentials and divisions of the gate are cheap)
        if (a.gate && !SPLIT) {
            const float *pg = a.gate + orow;
#pragma unroll
            for (int dt = 0; dt < 8; dt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4v gt = *reinterpret_cast<const float4v *>(pg + dt * 32 + g * 8 + lh * 4);
                    const float4v x = {gated(O[dt][g * 4] * inv, gt[0]), gated(O[dt][g * 4 + 1] * inv, gt[1]),
                                       gated(O[dt][g * 4 + 2] * inv, gt[2]),
                                       gated(O[dt][g * 4 + 3] * inv, gt[3])};
                    *reinterpret_cast<float4v *>(po + dt * 32 + g * 8 + lh * 4) = x;
                }
            return;
        }
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

// ---- sliced chunk prefill over the f16 copy, 64 tokens per wave ----------------------------------------
// The kernel above feeds every MFMA one 1-KiB operand from LDS, and a wave cannot ask for them faster than
// the pipe consumes them.  Here a task is 64 tokens x 1 head: each K and V^T operand read from LDS feeds two
// MFMAs (one per 32-token half), which halves the LDS operand traffic per MFMA.  That takes all 512 registers of a
// SIMD for one wave (O: 2 x 8 x 16 = 256 accumulators, Q: 128, scores of this half and of the next: 64,
// P: 16), so a workgroup is four waves, one per SIMD, and nothing hides a wave's softmax but its own MFMAs:
// the softmax of one 32-key half is cut into 16 pieces that sit, in program order, between the score MFMAs
// of the next half.  Every MFMA is written as inline assembly with its accumulator class spelled out (O in
// accumulation registers, scores in vector registers): left to itself the compiler puts every MFMA result
// of a 512-register kernel into accumulation registers, which O alone fills.
// The compiler does not know what the statements are, so it inserts no wait states for them.  What keeps
// their results safe: a score accumulator is read by vector code one PV product (32 MFMAs) after the MFMA
// that finished it; O is read by vector code (rescale, epilogue) only behind explicit s_nop padding or two
// further MFMAs; P and the operands are overwritten long after the MFMAs that read them have issued.
// Tiles, slices, partial rows and the merge are those of chunk_q8_kernel<true, false, true>.
constexpr int kT64Tasks = 4;                   // tasks (= waves) per workgroup
constexpr int kT64Tile = 64;                   // query tokens per task
constexpr int kT64Threads = 64 * kT64Tasks;
constexpr int kT64Dma = 9;                     // 1-KiB requests per wave for a K tile (33) or a V^T tile (36)
constexpr int kT64Lds = 2 * kBufBytesF;        // 141,312

// All 256 accumulation registers as a clobber list.  Every MFMA statement of the kernel below carries it, so
// the compiler can keep nothing of its own in them from one MFMA to the next (under register pressure it
// would otherwise park vector registers there, on top of O).
#define HIPML_A10(t) "a" #t "0", "a" #t "1", "a" #t "2", "a" #t "3", "a" #t "4", "a" #t "5", "a" #t "6", "a" #t "7", "a" #t "8", "a" #t "9"
#define HIPML_ACC_ALL                                                                                            \
    HIPML_A10(), HIPML_A10(1), HIPML_A10(2), HIPML_A10(3), HIPML_A10(4), HIPML_A10(5), HIPML_A10(6), HIPML_A10(7),  \
        HIPML_A10(8), HIPML_A10(9), HIPML_A10(10), HIPML_A10(11), HIPML_A10(12), HIPML_A10(13), HIPML_A10(14),      \
        HIPML_A10(15), HIPML_A10(16), HIPML_A10(17), HIPML_A10(18), HIPML_A10(19), HIPML_A10(20), HIPML_A10(21),    \
        HIPML_A10(22), HIPML_A10(23), HIPML_A10(24), "a250", "a251", "a252", "a253", "a254", "a255"
#define HIPML_MFMA_V0(acc, A, B) \
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(A), "v"(B) : HIPML_ACC_ALL)
#define HIPML_MFMA_V(acc, A, B) \
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(A), "v"(B) : HIPML_ACC_ALL)
// O^T lives in the 256 accumulation registers as state the compiler does not see: token half h, d tile dt in
// a[(8h + dt) * 16 .. + 15].  The build checks the generated code of this kernel for accumulation registers
// outside these statements (hipml_amd/build.py).
#define HIPML_MFMA_O(R, A, B) \
    asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]"                                            \
                 :                                                                                               \
                 : "v"(A), "v"(B), "n"(R), "n"((R) + 15)                                                         \
                 : HIPML_ACC_ALL)

template <int R, int N>
__device__ __forceinline__ void acc_zero()
{
    // (the clobber of the last register is what sizes the kernel's accumulation file)
    asm volatile("v_accvgpr_write_b32 a[%0], 0\n\tv_accvgpr_write_b32 a[%1], 0\n\tv_accvgpr_write_b32 a[%2], 0\n\t"
                 "v_accvgpr_write_b32 a[%3], 0"
                 :
                 : "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3)
                 : "a255");
    if constexpr (N > 4)
        acc_zero<R + 4, N - 4>();
}
// (The reads of accumulation registers below carry their own wait states: an MFMA of 8 passes needs 11 between
// its issue and a read of its result by another unit, and the compiler inserts none for statements it cannot
// read.  s_nop 10 in the same statement as the first read makes that independent of what is scheduled between
// this statement and the MFMA before it.)
template <int R, int N, bool FIRST = true>
__device__ __forceinline__ void acc_scale(float c)
{
    float t0, t1, t2, t3;
    if constexpr (FIRST)
        asm volatile("s_nop 10\n\tv_accvgpr_read_b32 %0, a[%5]\n\tv_accvgpr_read_b32 %1, a[%6]\n\t"
                     "v_accvgpr_read_b32 %2, a[%7]\n\tv_accvgpr_read_b32 %3, a[%8]\n\t"
                     "v_mul_f32 %0, %0, %4\n\tv_mul_f32 %1, %1, %4\n\tv_mul_f32 %2, %2, %4\n\tv_mul_f32 %3, %3, %4\n\t"
                     "v_accvgpr_write_b32 a[%5], %0\n\tv_accvgpr_write_b32 a[%6], %1\n\tv_accvgpr_write_b32 a[%7], %2\n\t"
                     "v_accvgpr_write_b32 a[%8], %3"
                     : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3)
                     : "v"(c), "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
    else
    asm volatile("v_accvgpr_read_b32 %0, a[%5]\n\tv_accvgpr_read_b32 %1, a[%6]\n\tv_accvgpr_read_b32 %2, a[%7]\n\t"
                 "v_accvgpr_read_b32 %3, a[%8]\n\t"
                 "v_mul_f32 %0, %0, %4\n\tv_mul_f32 %1, %1, %4\n\tv_mul_f32 %2, %2, %4\n\tv_mul_f32 %3, %3, %4\n\t"
                 "v_accvgpr_write_b32 a[%5], %0\n\tv_accvgpr_write_b32 a[%6], %1\n\tv_accvgpr_write_b32 a[%7], %2\n\t"
                 "v_accvgpr_write_b32 a[%8], %3"
                 : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3)
                 : "v"(c), "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
    if constexpr (N > 4)
        acc_scale<R + 4, N - 4, false>(c);
}
template <int R>
__device__ __forceinline__ float4v acc_read4()
{
    float4v x;
    asm volatile("s_nop 10\n\tv_accvgpr_read_b32 %0, a[%4]\n\tv_accvgpr_read_b32 %1, a[%5]\n\t"
                 "v_accvgpr_read_b32 %2, a[%6]\n\tv_accvgpr_read_b32 %3, a[%7]"
                 : "=v"(x[0]), "=v"(x[1]), "=v"(x[2]), "=v"(x[3])
                 : "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
    return x;
}

__global__ void __launch_bounds__(kT64Threads, 1) __attribute__((amdgpu_waves_per_eu(1, 1)))
chunk_f16_t64_kernel(const ChunkArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int ln = lane & 31; // MFMA column: token within a 32-token half
    const int lh = lane >> 5; // k half-group

    // blockIdx.x -> (kv head, key slice, task block), as in chunk_q8_kernel (every block has a.splits slices)
    int kvh, split, tb;
    {
        const int combos = a.n_kv * a.splits;
        const int bid = blockIdx.x;
        int combo;
        if (combos % 8 == 0) {
            const int per = combos / 8;
            const int xcd = bid & 7, j = bid >> 3;
            combo = xcd + 8 * (j % per);
            tb = j / per;
        } else if (8 % combos == 0) {
            const int xcd = bid & 7, j = bid >> 3;
            const int share = 8 / combos;
            combo = xcd % combos;
            tb = j * share + xcd / combos;
        } else {
            combo = bid % combos;
            tb = bid / combos;
        }
        kvh = combo % a.n_kv;
        split = combo / a.n_kv;
        if (tb >= a.nblock)
            return; // uniform over the workgroup
    }
    const int nsp = a.splits;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave); // (scalar: what follows from it stays in scalar registers)
    // Tasks of one KV head, in order: the whole 64-token tiles, one task per head (its halves are the tile's
    // two 32-token halves); then the rest of the tokens: more than 32 make one more such tile with a ragged
    // second half, up to 32 make tasks of 32 tokens x 2 heads (the halves are two heads of the same tokens;
    // they share the K/V operands all the same), so that 672 tokens x 6 heads are 63 tasks = 16 workgroups per
    // KV head and slice, not 66 = 17.  Half h of this wave's task: tokens th0[h] .. th0[h] + 31 of head hd[h].
    const int task = tb * kT64Tasks + wave_u;
    const bool task_valid = task < a.ntask;
    const int rem = a.tokens % kT64Tile;
    const int whole = (a.tokens / kT64Tile + (rem > 32 ? 1 : 0)) * a.group; // tasks of 64 tokens x 1 head
    auto last_token_of = [&](int k) { // of task k (the last one any of its halves holds)
        const int end = k < whole ? (k / a.group + 1) * kT64Tile : a.tokens;
        return (end < a.tokens ? end : a.tokens) - 1;
    };
    int th0[2], hd[2];
    bool half_valid[2];
    {
        const int k = task_valid ? task : a.ntask - 1;
        if (k < whole) {
            const int tt = k / a.group, hq = k - tt * a.group;
            th0[0] = tt * kT64Tile;
            th0[1] = tt * kT64Tile + 32;
            hd[0] = hd[1] = kvh * a.group + hq;
            half_valid[0] = half_valid[1] = task_valid;
        } else {
            const int j = k - whole;
            th0[0] = th0[1] = a.tokens - rem;
            hd[0] = kvh * a.group + 2 * j;
            hd[1] = kvh * a.group + (2 * j + 1 < a.group ? 2 * j + 1 : a.group - 1);
            half_valid[0] = task_valid;
            half_valid[1] = task_valid && 2 * j + 1 < a.group;
        }
    }

    const int last_task = (tb * kT64Tasks + kT64Tasks - 1 < a.ntask ? tb * kT64Tasks + kT64Tasks - 1 : a.ntask - 1);
    const int seq_block = a.pos0 + last_token_of(last_task) + 1;
    const int tiles_block = (seq_block + kKTile - 1) / kKTile;
    const int klo = (int)((long long)tiles_block * split / nsp) * kKTile;
    int khi = (int)((long long)tiles_block * (split + 1) / nsp) * kKTile;
    khi = khi < seq_block ? khi : seq_block;
    const int ntile = khi > klo ? (khi - klo + kKTile - 1) / kKTile : 0;

    // K tile t of the slice lives in K buffer t & 1, its V^T tile in V^T buffer t & 1; each arrives as
    // nine 1-KiB requests per wave (the last ones repeat the tile's last KiB; a tile past the slice's last
    // repeats that one), so that the waits below are constants.
    const uint32_t lds_at = lds_address(lds);
    // Request j of nine for tile t (the K tile or the V^T tile): KiB i = wave + 4 j of the tile.  The per-lane
    // offsets and the KiB offsets are made once (a request in the loop is then three instructions: LDS
    // address into m0, the wait state m0 asks for, the load), and the K tile's last request repeats KiB 32
    // for the waves whose ninth would lie behind the tile.
    uint32_t voff[kT64Dma];
    int soff[kT64Dma];
#pragma unroll
    for (int j = 0; j < kT64Dma; j++) {
        soff[j] = (wave_u + kT64Tasks * j) * 1024;
        voff[j] = lane * 16 + soff[j];
    }
    const int soff_k8 = (wave_u + kT64Tasks * 8 < kKTileBytes / 1024 ? wave_u + kT64Tasks * 8 : kKTileBytes / 1024 - 1) * 1024;
    const uint32_t voff_k8 = lane * 16 + soff_k8;
    auto dma_req = [&](int t, bool v_tile, int j) {
        const int tc = t < ntile ? t : ntile - 1;
        const size_t tile = (size_t)kvh * a.tile_stride + (klo / kKTile + tc);
        const uint8_t *src = v_tile ? a.vt + tile * kVtTileBytes : a.k16 + tile * kKTileBytes;
        const uint32_t dst = lds_at + (t & 1) * kBufBytesF + (v_tile ? kKTileBytes : 0);
        const bool last_k = !v_tile && j == kT64Dma - 1;
        const uint32_t at = __builtin_amdgcn_readfirstlane(dst);
        const int so = __builtin_amdgcn_readfirstlane(last_k ? soff_k8 : soff[j]);
        const uint64_t p = (uint64_t)(uintptr_t)src;
        const uint64_t pu = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)p) |
                            ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(p >> 32)) << 32);
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     :
                     : "s"(at), "s"(so), "v"(last_k ? voff_k8 : voff[j]), "s"(pu)
                     : "memory", "scc");
    };
    auto dma_tile = [&](int t, bool v_tile) {
#pragma unroll
        for (int j = 0; j < kT64Dma; j++)
            dma_req(t, v_tile, j);
    };
    if (ntile > 0) {
        dma_tile(0, false);
        dma_tile(0, true);
    }

    // ---- Q^T operand: per 32-token half, 16 k-steps of 8 f16 (d = ks*16 + lh*8 + j), all in registers.
    // Rows are fetched whole, converted and turned round in this wave's corner of the second tile buffer.
    half8 Q[2][16];
    {
        uint8_t *qt = lds + kBufBytesF + wave * (32 * kKRow);
        const size_t tok_stride = (size_t)a.n_head * kHeadDim;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const float *qh = a.q + (size_t)hd[h] * kHeadDim + lane * 4;
#pragma unroll
            for (int b = 0; b < 2; b++) {
                float4v f[16];
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int tr = th0[h] + b * 16 + i;
                    f[i] = __builtin_nontemporal_load(
                        reinterpret_cast<const float4v *>(qh + (size_t)(tr < a.tokens ? tr : a.tokens - 1) * tok_stride));
                }
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    half4 x;
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        x[j] = (_Float16)f[i][j];
                    *reinterpret_cast<half4 *>(qt + (b * 16 + i) * kKRow + lane * 8) = x;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's own writes
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int ks = 0; ks < 16; ks++)
                Q[h][ks] = *reinterpret_cast<const half8 *>(qt + ln * kKRow + ks * 32 + lh * 16);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read before the next half overwrites the corner
            __builtin_amdgcn_wave_barrier();
        }
    }
    __syncthreads(); // every wave has its Q, tile 0 has landed (no load is outstanding): the second buffer is free
    if (ntile > 0)
        dma_tile(1, false);

    acc_zero<0, 256>();
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.0f, 0.0f};
    float mneg[2] = {0.0f, 0.0f}, ls[2] = {0.0f, 0.0f};
    float16v S[2], N[2]; // scores of the half whose softmax runs now, and of the next one
    half8 P[2][2];

    // The softmax of a 32-key half is spread over the MFMAs around it.  Its maxima are taken from the finished
    // scores N while the PV product of the half before runs (max_piece, masking included); the step that follows
    // first moves the reference exponent where a maximum has outgrown it (lazily, as chunk_q8_kernel does: the
    // only place O is rescaled, behind that step's first two MFMAs) and then takes two of a lane's 32
    // exponentials after each pair of score MFMAs.
    // A wave issues in order: behind two MFMAs in a row nothing goes out until the first has left the pipe (32
    // cycles), and vector work that follows the pair for longer than the second one runs leaves the pipe idle.
    // So every MFMA is followed by its own slot of at most ~28 cycles of other work: one exponential with its
    // multiply-add and sum, or one LDS read, or one request, or a third of a maximum.
    float mt[2] = {-INFINITY, -INFINITY}, mx = 0.0f;
    auto max_part = [&](int t, int hk, int h, int part) { // scores N of half hk of tile t, token half h
        if (part == 0) {
            const int k0 = klo + t * kKTile + hk * 32;
            const int tok0 = a.pos0 + th0[h];
            if ((k0 + 31 > tok0) || (k0 + 32 > khi)) { // (uniform over the wave)
                // (the empty statement keeps this a branch: turned into selects, the 80 instructions would run
                // for every half, and only the halves on the diagonal and at the end of the slice need them)
                asm volatile("" ::: "memory");
                const int my_last = tok0 + ln;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int kg = k0 + (i >> 2) * 8 + lh * 4 + (i & 3);
                    N[h][i] = (kg <= my_last && kg < khi) ? N[h][i] : -INFINITY;
                }
            }
            mx = fmaxf(fmaxf(N[h][0], N[h][1]), N[h][2]);
            mx = fmaxf(fmaxf(mx, N[h][3]), N[h][4]);
            mx = fmaxf(fmaxf(mx, N[h][5]), N[h][6]);
            mx = fmaxf(mx, N[h][7]);
        } else if (part == 1) {
            mx = fmaxf(fmaxf(mx, N[h][8]), N[h][9]);
            mx = fmaxf(fmaxf(mx, N[h][10]), N[h][11]);
            mx = fmaxf(fmaxf(mx, N[h][12]), N[h][13]);
            mx = fmaxf(fmaxf(mx, N[h][14]), N[h][15]);
        } else {
            mt[h] = xor32_max(mx) * a.scale_log2;
        }
    };
    // Softmax of S.  A lane's 32 exponentials are taken in the order the PV product needs them: first the 16
    // of its first k-step (keys 0..15 of the half: P[h][0]), then the 16 of the second.  Exponential v of that
    // order, with its multiply-add, conversion and (every second time) the sum of a pair:
    auto exp_value = [&](int v) {
        const int h = (v >> 3) & 1, i = (v >> 4) * 8 + (v & 7);
        P[h][i >> 3][i & 7] = (_Float16)__builtin_amdgcn_exp2f(fmaf(S[h][i], a.scale_log2, mneg[h]));
        if (i & 1) {
            // the sum takes the probabilities as the PV product sees them (f16), two per instruction
            const half2v pr = {P[h][i >> 3][(i & 7) - 1], P[h][i >> 3][i & 7]};
            ls[h] = __builtin_amdgcn_fdot2(pr, half2v{(_Float16)1.0f, (_Float16)1.0f}, ls[h], false);
        }
    };
    // Behind one MFMA a wave gets four or five vector instructions through before the next MFMA is held up
    // (an exponential counts double), so the 32 exponentials are spread: the score step carries the first
    // kExpStep (slots 2..31), the PV product that follows takes the last kExpPv in its first slots; it does
    // not read them before its second half (pv below).  Slot 1 of the step (behind the second MFMA: O is at
    // rest) moves the reference exponent where a maximum has outgrown it, the only place O is rescaled.
    // (Measured at 2,048 @ 100,000: 24 | 8 4.05 ms, 22 | 10 4.07, 20 | 12 4.09, 18 | 14 4.07; 32 | 0 4.13.)
    constexpr int kExpStep = 24, kExpPv = 32 - kExpStep; // (kExpPv even, at most 14)
    auto exp_slot = [&](int p) {
        if (p == 1) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (__any(mt[h] > m_run[h] + kPfLazy)) {
                    const float m_new = fmaxf(m_run[h], mt[h]);
                    const float corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run[h] - m_new);
                    l_run[h] *= corr;
                    if (h == 0)
                        acc_scale<0, 128>(corr);
                    else
                        acc_scale<128, 128>(corr);
                    m_run[h] = m_new;
                }
                mneg[h] = m_run[h] == -INFINITY ? 0.0f : -m_run[h];
                ls[h] = 0.0f;
            }
        } else if (p >= 2) {
            const int lo = (p - 2) * kExpStep / 30, hi = (p - 1) * kExpStep / 30;
#pragma unroll
            for (int v = lo; v < hi; v++)
                exp_value(v);
        }
    };
    // Scores of half hk of tile t into N (MFMA), the exponentials of S in the slots (SOFT); each K operand
    // feeds the MFMAs of both token halves and is read from LDS two steps ahead.
    auto step = [&](auto mfma_tag, auto soft_tag, int t, int hk) {
        constexpr bool MFMA = decltype(mfma_tag)::value, SOFT = decltype(soft_tag)::value;
        const uint8_t *Kh = lds + (t & 1) * kBufBytesF + (hk * 32 + ln) * kKRow + lh * 16;
        half8 A0, A1;
        if constexpr (MFMA) {
            A0 = *reinterpret_cast<const half8 *>(Kh);
            A1 = *reinterpret_cast<const half8 *>(Kh + 32);
        }
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            half8 A2 = A0;
            if constexpr (MFMA) {
                if (ks + 2 < 16)
                    A2 = *reinterpret_cast<const half8 *>(Kh + (ks + 2) * 32);
                if (ks == 0)
                    HIPML_MFMA_V0(N[0], A0, Q[0][ks]);
                else
                    HIPML_MFMA_V(N[0], A0, Q[0][ks]);
            }
            if constexpr (SOFT)
                exp_slot(2 * ks);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MFMA) {
                if (ks == 0)
                    HIPML_MFMA_V0(N[1], A0, Q[1][ks]);
                else
                    HIPML_MFMA_V(N[1], A0, Q[1][ks]);
                A0 = A1;
                A1 = A2;
            }
            if constexpr (SOFT)
                exp_slot(2 * ks + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // O^T += V^T . P^T for half hk of tile t: each V^T operand feeds both token halves.  The slot behind the
    // first MFMA of a pair reads the operand of two steps on; the first kExpPv slots take the exponentials that
    // the second eight steps read, the second slots after them carry this wave's nine requests for tile dt (its
    // V^T tile if dv), and the first slots of the last six steps, MAXP, the maxima of the scores N of the half
    // (nt, nhk) that follows.
    auto pv = [&](auto max_tag, int t, int hk, int nt, int nhk, int dt, bool dv) {
        constexpr bool MAXP = decltype(max_tag)::value;
        const uint8_t *Vt = lds + (t & 1) * kBufBytesF + kKTileBytes + ln * kVtRow + (hk * 32 + lh * 8) * 2;
        half8 A0 = *reinterpret_cast<const half8 *>(Vt);
        half8 A1 = *reinterpret_cast<const half8 *>(Vt + 32 * kVtRow);
#define HIPML_PV_STEP(s)                                                                                        \
    {                                                                                                           \
        half8 A2 = A0;                                                                                          \
        HIPML_MFMA_O(((s) & 7) * 16, A0, P[0][(s) >> 3]);                                                       \
        if ((s) + 2 < 16)                                                                                       \
            A2 = *reinterpret_cast<const half8 *>(Vt + (((s) + 2) & 7) * 32 * kVtRow + (((s) + 2) >> 3) * 32); \
        if constexpr (2 * (s) < kExpPv)                                                                         \
            exp_value(kExpStep + 2 * (s));                                                                      \
        if constexpr (MAXP && (s) >= 10)                                                                        \
            max_part(nt, nhk, ((s) - 10) / 3, ((s) - 10) % 3);                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        HIPML_MFMA_O(128 + ((s) & 7) * 16, A0, P[1][(s) >> 3]);                                                 \
        if constexpr (2 * (s) + 1 < kExpPv)                                                                     \
            exp_value(kExpStep + 2 * (s) + 1);                                                                  \
        else if constexpr ((s) - kExpPv / 2 < kT64Dma)                                                          \
            dma_req(dt, dv, (s) - kExpPv / 2);                                                                  \
        if constexpr (2 * (s) + 2 == kExpPv) {                                                                  \
            l_run[0] += ls[0];                                                                                  \
            l_run[1] += ls[1];                                                                                  \
        }                                                                                                       \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        A0 = A1;                                                                                                \
        A1 = A2;                                                                                                \
    }
        HIPML_PV_STEP(0) HIPML_PV_STEP(1) HIPML_PV_STEP(2) HIPML_PV_STEP(3) HIPML_PV_STEP(4) HIPML_PV_STEP(5)
        HIPML_PV_STEP(6) HIPML_PV_STEP(7) HIPML_PV_STEP(8) HIPML_PV_STEP(9) HIPML_PV_STEP(10) HIPML_PV_STEP(11)
        HIPML_PV_STEP(12) HIPML_PV_STEP(13) HIPML_PV_STEP(14) HIPML_PV_STEP(15)
#undef HIPML_PV_STEP
    };
    const std::true_type yes;
    const std::false_type no;

    // Per tile t: [scores(t, 1) with the exponentials of (t, 0); PV(t, 0), requesting V^T(t + 1) into the buffer
    // of V^T(t - 1)]; K(t + 1) has landed: barrier A; [scores(t + 1, 0) with the exponentials of (t, 1); PV(t, 1),
    // requesting K(t + 2) into the buffer of K(t), which every wave finished with before barrier A]; V^T(t + 1)
    // has landed: barrier B (after it every wave has finished with V^T(t)).  Requests outstanding at barrier A,
    // oldest first: K(t + 1), V^T(t + 1); at barrier B: V^T(t + 1), K(t + 2): the wait is vmcnt(9) both times.
    if (ntile > 0) {
        step(yes, no, 0, 0);
        // these scores were finished just now (the statement owns N, so no read of them can move above it)
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(N[0]), "+v"(N[1])::"memory");
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int part = 0; part < 3; part++)
                max_part(0, 0, h, part);
        S[0] = N[0];
        S[1] = N[1];
    }
    for (int t = 0; t < ntile; t++) {
        step(yes, yes, t, 1);
        pv(yes, t, 0, t, 1, t + 1, true);
        S[0] = N[0];
        S[1] = N[1];
        asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        lds_barrier();
        if (t + 1 < ntile) {
            step(yes, yes, t + 1, 0);
            pv(yes, t, 1, t + 1, 0, t + 2, false);
        } else {
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // O may be rescaled right behind the MFMAs of PV(t, 0)
            step(no, yes, t + 1, 0);
            pv(no, t, 1, t + 1, 0, t + 2, false);
        }
        S[0] = N[0];
        S[1] = N[1];
        asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        lds_barrier();
    }
    // the tile buffers are about to be reused, and O is about to be read
    asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    lds_barrier();

    // ---- epilogue: partial rows leave through this wave's corner of LDS, as in chunk_q8_kernel ----------
    constexpr int kPitch = 512 + 16;
    uint8_t *mine = lds + wave * (32 * kPitch);
    const int l32 = lane & 31, rsel = lane >> 5;
    auto half_rows = [&](auto h_tag, auto hf_tag) {
        // 128 columns (d tiles 4 hf .. 4 hf + 3) of token half h into this wave's corner
        constexpr int h = decltype(h_tag)::value, hf = decltype(hf_tag)::value;
        constexpr int R = (h * 8 + hf * 4) * 16;
#define HIPML_ROW_PIECE(dl, g)                                                                                   \
    *reinterpret_cast<float4v *>(mine + ln * kPitch + ((dl) * 32 + (g) * 8 + lh * 4) * 4) = acc_read4<R + (dl) * 16 + (g) * 4>();
        HIPML_ROW_PIECE(0, 0) HIPML_ROW_PIECE(0, 1) HIPML_ROW_PIECE(0, 2) HIPML_ROW_PIECE(0, 3)
        HIPML_ROW_PIECE(1, 0) HIPML_ROW_PIECE(1, 1) HIPML_ROW_PIECE(1, 2) HIPML_ROW_PIECE(1, 3)
        HIPML_ROW_PIECE(2, 0) HIPML_ROW_PIECE(2, 1) HIPML_ROW_PIECE(2, 2) HIPML_ROW_PIECE(2, 3)
        HIPML_ROW_PIECE(3, 0) HIPML_ROW_PIECE(3, 1) HIPML_ROW_PIECE(3, 2) HIPML_ROW_PIECE(3, 3)
#undef HIPML_ROW_PIECE
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const float lsum = l_run[h] + __shfl_xor(l_run[h], 32);
        const int tbase = th0[h], head = hd[h];
        const bool task_valid = half_valid[h];
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            if (h == 0 && hf == 0)
                half_rows(I0(), I0());
            else if (h == 0)
                half_rows(I0(), I1());
            else if (hf == 0)
                half_rows(I1(), I0());
            else
                half_rows(I1(), I1());
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int r2 = 0; r2 < 16; r2++) {
                const int r = r2 * 2 + rsel;
                const float4v x = *reinterpret_cast<const float4v *>(mine + r * kPitch + l32 * 16);
                if (task_valid && tbase + r < a.tokens) {
                    const size_t prow = ((size_t)split * a.qslots + (tbase + r)) * a.n_head + head;
                    *reinterpret_cast<float4v *>(a.part_acc + prow * kHeadDim + hf * 128 + l32 * 4) = x;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
        }
        if (task_valid && tbase + ln < a.tokens && lh == 0) {
            const size_t row = ((size_t)split * a.qslots + (tbase + ln)) * a.n_head + head;
            a.part_ml[row * 2] = m_run[h];
            a.part_ml[row * 2 + 1] = lsum;
        }
    }
}

// ---- chunk prefill with the key split inside the workgroup -----------------------------------------
// Near position 0 a chunk has few keys per token and little to do in total (672 tokens at depth 0:
// 5.6 GFLOP, 1.5 MB of cache), but as many Q and output rows as at any depth.  The kernel above then
// has too few workgroups for the chip unless the keys are cut into slices, and slices cost partial
// rows in memory and a second launch that is longer than the attention itself.  Here the slices stay
// inside the workgroup: it takes one tile of 32 tokens and two heads of one KV head, and cuts their
// keys into four slices, one wave per (slice, head).  The two waves of a slice share its K/V tiles
// (32 keys per step, dequantized by those two waves, single-buffered: 4 x 34 KB of LDS); the four
// partial results of a head meet in LDS at the end, each wave finishing 64 of the 256 output
// columns, gate included.  672 tokens x 24 heads are 252 such workgroups, one round of the chip.
//
// A step is a VALU slot (dequantize the next K tile and this step's V tile, softmax) and an MFMA slot (PV
// of this step, scores of the next), each closed by a workgroup barrier; see the loop.
// Operand layouts, MFMA shapes and numerics are those of chunk_q8_kernel, except that the running sums
// are held against a reference exponent that follows the running maximum lazily (see softmax below).
constexpr int kWgSlices = 4;                   // key slices of a task, one wave each
constexpr int kWgStep = 32;                    // keys per step
constexpr int kWgK = kWgStep * kKRow;          // 16,896: K tile of a slice
constexpr int kWgV = kWgStep * kVRow;          // 17,408: its V tile
constexpr int kWgSlice = kWgK + kWgV;          // 34,304
constexpr int kWgQPark = 3;                   // d-steps of the Q operand read from LDS at every use: 256 registers do not hold the rest
constexpr int kWgQAt = kWgSlices * kWgSlice;   // 137,216: [head 2][step][lane] x 16 bytes
constexpr int kWgLds = kWgQAt + 2 * kWgQPark * 1024;
constexpr int kWgXAt = 4096;                   // merge: (max, sum) table below, accumulator exchange from here
constexpr int kWgXArea = 8192;                 // two 32-column tiles of one wave
constexpr int kWgOutPitch = 272;               // a token's 64 finished columns + pad
constexpr int kWgAhead = 2;     // K operands read this many MFMAs ahead of their use
constexpr int kWgAheadPv = 2; // V operands
constexpr float kWgLazy = 8.0f;                // growth of a maximum (log2 units) that moves the reference exponent

// ROPE: the query rows are rotated (NeoX pairs (k, k + 32) of the first 64 columns, position pos0 + token)
// between their load and their conversion to f16, with the expressions of the RoPE kernels and
// without contraction, so the operands are the bits those kernels would have left in memory.
template <bool Q4, bool ROPE>
__global__ void __launch_bounds__(kPfThreads, 1) chunk_wg_kernel(const ChunkArgs a)
{
    typedef typename HalfOf<Q4>::type Half;
    constexpr int kRowBytes = Q4 ? hipml::kRowBytesQ4 : hipml::kRowBytes;
    constexpr int kUnitBytes = Q4 ? 36 : 68;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    static_assert(kWgLds <= 160 * 1024 && kWgXAt + 12 * kWgXArea <= kWgLds && kWgXAt + 8 * kQTile * kWgOutPitch <= kWgLds, "merge areas");

    // (the same in every lane: taking it from the first one lets everything derived from it live in scalar registers)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int ln = lane & 31;
    const int lh = lane >> 5;
    const int sl = wave >> 1;                     // key slice
    const int hp = wave & 1;                      // head of the pair

    // blockIdx.x -> (token tile, kv head, head pair), the token tiles with the most keys first
    const int pairs = (a.group + 1) >> 1;
    const int per_tt = a.n_kv * pairs;
    const int ntt = (a.tokens + kQTile - 1) / kQTile;
    const int tt = ntt - 1 - (int)blockIdx.x / per_tt;
    const int rem = (int)blockIdx.x % per_tt;
    const int kvh = rem % a.n_kv;
    const int hq = (rem / a.n_kv) * 2 + hp;
    const bool task_valid = hq < a.group;        // (an odd group leaves the last pair one head)
    const int head = kvh * a.group + (task_valid ? hq : a.group - 1);
    const int t0 = tt * kQTile;
    const int last_tok = ((tt + 1) * kQTile < a.tokens ? (tt + 1) * kQTile : a.tokens) - 1;
    const int khi = a.pos0 + last_tok + 1;                          // keys the tile's last token sees
    const int nstep = ((khi + kWgStep - 1) / kWgStep + kWgSlices - 1) / kWgSlices; // per slice, same for all
    const int kbeg = sl * nstep * kWgStep;                          // this slice's first key
    const int tok = t0 + ln;
    const int my_last_key = a.pos0 + tok;
    const bool tok_valid = task_valid && tok < a.tokens;

    uint8_t *Kt = lds + sl * kWgSlice;
    uint8_t *Vt = Kt + kWgK;

    // ---- staging role: lane -> one unit (two blocks) of the slice's K tile and one of its V tile ----
    // (the (row, unit) pattern of chunk_q8_kernel over the slice's 128 lanes: conflict-free 128-bit writes)
    const int su = hp * 64 + lane;
    const int srow = (su >> 6) * 16 + ((su >> 1) & 7) + ((su >> 5) & 1) * 8;
    const int spr = (su & 1) | ((su >> 3) & 2);
    // (uniform base + 32-bit lane offset: a KV head's rows span less than 4 GB)
    const uint8_t *kbase = a.kc + (size_t)kvh * a.stride * kRowBytes;
    const uint8_t *vbase = a.vc + (size_t)kvh * a.stride * kRowBytes;
    // (a row past the visible keys repeats the last one: unconditional loads keep their registers out of
    // branches; such keys are masked)
    auto unit_at = [&](int s) {
        int key = kbeg + s * kWgStep + srow;
        key = key < khi ? key : khi - 1;
        return (uint32_t)key * (uint32_t)kRowBytes + (uint32_t)(spr * kUnitBytes);
    };
    // One unit is in flight at a time, alternately the K and the V unit: a unit is requested when the
    // one before it has been dequantized and travels through the MFMA slot that follows.
    Half r0, r1;
    auto issue_k = [&](int s) {
        const uint8_t *u = kbase + unit_at(s);
        load_half0(r0, u);
        load_half1(r1, u);
    };
    auto issue_v = [&](int s) {
        const uint8_t *u = vbase + unit_at(s);
        load_half0(r0, u);
        load_half1(r1, u);
    };
    auto stage_k = [&]() {
        uint8_t *d = Kt + srow * kKRow + spr * 128;
        stage_block0(r0, d);
        stage_block1(r1, d);
    };
    auto stage_v = [&]() {
        uint8_t *d = Vt + srow * kVRow + spr * 128;
        stage_block0(r0, d);
        stage_block1(r1, d);
    };

    // ---- Q^T operand of this wave's head: the head's four waves fetch eight token rows each (one
    // instruction = one token's 256 floats), convert them and write them as f16 rows into the V tile of
    // slice `hp`, which is unused until the first V tile is staged; every wave then reads all 16 steps.
    half8 qf[16];
    uint8_t *qpark = lds + kWgQAt + hp * kWgQPark * 1024 + lane * 16;
    {
        uint8_t *qa = lds + hp * kWgSlice + kWgK;
        const float *qh = a.q + (size_t)head * kHeadDim + lane * 4;
        const size_t tok_stride = (size_t)a.n_head * kHeadDim;
        float4v f[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int tr = t0 + sl * 8 + i;
            // (read once, by this workgroup: non-temporal, as the gate rows and the output rows below)
            f[i] = __builtin_nontemporal_load(reinterpret_cast<const float4v *>(qh + (size_t)(tr < a.tokens ? tr : a.tokens - 1) * tok_stride));
        }
        issue_k(0); // (behind the query rows: they come from further away)
        // (cos, sin) of pairs 4 l8 .. 4 l8 + 3; lanes 0..15 hold columns 0..63, the others load a row they do not use
        float4v cs0[ROPE ? 8 : 1], cs1[ROPE ? 8 : 1];
        if constexpr (ROPE) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int tr = t0 + sl * 8 + i;
                const float4v *e = reinterpret_cast<const float4v *>(
                    a.rope_tab + ((size_t)(a.pos0 + (tr < a.tokens ? tr : a.tokens - 1)) * 32 + 4 * (lane & 7)) * 2);
                cs0[i] = e[0];
                cs1[i] = e[1];
            }
        }
        stage_k();
        issue_k(1);
        if constexpr (ROPE) {
            // y1 = x1 cos - x2 sin (lanes 0..7 hold x1), y2 = x1 sin + x2 cos (lanes 8..15 hold x2): each
            // product rounded by itself, then one addition, as the RoPE kernels compute them
#pragma clang fp contract(off)
            const bool lo = lane < 8, rot = lane < 16;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float c[4] = {cs0[i][0], cs0[i][2], cs1[i][0], cs1[i][2]};
                const float sn[4] = {cs0[i][1], cs0[i][3], cs1[i][1], cs1[i][3]};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float x = f[i][j];
                    // lane l ^ 8 of the same 16 lanes: a rotation of the row by 8
                    const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, false));
                    const float own = x * c[j];
                    const float cross = other * sn[j];
                    const float y = own + (lo ? -cross : cross);
                    f[i][j] = rot ? y : x;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            half4 h;
#pragma unroll
            for (int j = 0; j < 4; j++)
                h[j] = (_Float16)f[i][j];
            *reinterpret_cast<half4 *>(qa + (sl * 8 + i) * kKRow + lane * 8) = h;
        }
        lds_barrier(); // Q rows and K(0) are in LDS
#pragma unroll
        for (int ks = 0; ks < 16; ks++) {
            // (steps below kWgQPark stay in registers for the first scores only; their parked copies are
            // read from the second scores on, two barriers after they are written)
            qf[ks] = *reinterpret_cast<const half8 *>(qa + ln * kKRow + ks * 32 + lh * 16);
            if (ks < kWgQPark && (ks & 3) == sl) // the head's four waves read the same values: each parks its share
                *reinterpret_cast<half8 *>(qpark + ks * 1024) = qf[ks];
        }
    }

    float16v O[8];
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            O[t][i] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;
    float16v S;
    half8 P[2];

    const int gl = lane & 15;
    const int vtr_off = (gl >> 2) * kVRow + (((lane >> 4) & 1) * 16 + (gl & 3) * 4) * 2;

    auto live = [&](int s) { return task_valid && kbeg + s * kWgStep < khi; }; // wave-uniform

    auto scores = [&](int s, auto first) { // first: the scores of step 0, every Q step still in registers
        constexpr bool kFirst = decltype(first)::value;
        if (!live(s))
            return;
        const uint8_t *Kh = Kt + ln * kKRow + lh * 16;
        float16v acc;
#pragma unroll
        for (int i = 0; i < 16; i++)
            acc[i] = 0.0f;
        half8 A[16], B[kWgQPark > 0 ? kWgQPark : 1];
        if constexpr (!kFirst) {
#pragma unroll
            for (int ks = 0; ks < kWgQPark; ks++)
                B[ks] = *reinterpret_cast<const half8 *>(qpark + ks * 1024);
        }
#pragma unroll
        for (int ks = 0; ks < 16; ks++)
            A[ks] = *reinterpret_cast<const half8 *>(Kh + ks * 32);
#pragma unroll
        for (int ks = 0; ks < 16; ks++)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[ks], !kFirst && ks < kWgQPark ? B[ks] : qf[ks], acc, 0, 0, 0);
        S = acc;
        // K operands are read kWgAhead MFMAs ahead (an LDS read under the load of eight waves takes longer
        // than two MFMAs); the parked Q steps head the chain and are all read up front
        __builtin_amdgcn_sched_group_barrier(0x100, kWgAhead + (kFirst ? 0 : kWgQPark), 0);
#pragma unroll
        for (int ks = 0; ks < 16 - kWgAhead; ks++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kWgAhead, 0);
    };

    // lane holds keys (i/4)*8 + lh*4 + i%4 of the step for token ln
    auto softmax = [&](int s) {
        if (!live(s))
            return;
        const int k0 = kbeg + s * kWgStep;
        const bool need_mask = (k0 + 31 > a.pos0 + t0) || (k0 + 32 > khi);
        if (need_mask) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int kg = k0 + (i >> 2) * 8 + lh * 4 + (i & 3);
                S[i] = (kg <= my_last_key && kg < khi) ? S[i] : -INFINITY;
            }
        }
        float mt = S[0];
#pragma unroll
        for (int i = 1; i < 16; i++)
            mt = fmaxf(mt, S[i]);
        mt = xor32_max(mt) * a.scale_log2;
        // m_run is the exponent the sums are held against, not the running maximum: it follows the
        // maximum only when some token's maximum has grown by more than kWgLazy since it was set, so
        // the 128 accumulator registers are rescaled on few steps.  Until then probabilities may be as
        // large as 2^kWgLazy, which f16 holds with the same relative precision.
        if (__any(mt > m_run + kWgLazy)) {
            const float m_new = fmaxf(m_run, mt);
            const float corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= corr;
#pragma unroll
            for (int dt = 0; dt < 8; dt++)
                O[dt] *= corr;
            m_run = m_new;
        }
        const float mneg = m_run == -INFINITY ? 0.0f : -m_run;
        float ls = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float e = __builtin_amdgcn_exp2f(fmaf(S[i], a.scale_log2, mneg));
            ls += e;
            P[i >> 3][i & 7] = (_Float16)e;
        }
        l_run += ls;
        asm volatile("" : "+v"(P[0]), "+v"(P[1]), "+v"(l_run), "+v"(m_run));
    };

    auto pv = [&](int s) {
        if (!live(s))
            return;
        half8 A[16];
        const uint8_t *Vh = Vt + vtr_off;
#pragma unroll
        for (int u = 0; u < 2; u++) {
#pragma unroll
            for (int dt = 0; dt < 8; dt++) {
                const uint8_t *vp = Vh + dt * 64;
                const short4v r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3))) *)(vp + ((2 * u) * 8 + lh * 4) * kVRow));
                const short4v r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3))) *)(vp + ((2 * u + 1) * 8 + lh * 4) * kVRow));
                const half4 h0 = __builtin_bit_cast(half4, r0);
                const half4 h1 = __builtin_bit_cast(half4, r1);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    A[u * 8 + dt][j] = h0[j];
                    A[u * 8 + dt][4 + j] = h1[j];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int dt = 0; dt < 8; dt++)
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[u * 8 + dt], P[u], O[dt], 0, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * kWgAheadPv, 0);
#pragma unroll
        for (int k = 0; k < 16 - kWgAheadPv; k++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kWgAheadPv, 0);
    };

    // Two slots per step, each closed by a barrier:
    //   V: dequantize K(s+1) into the K tile, request V(s), softmax of step s, dequantize V(s) into the
    //      V tile, request K(s+2)                                                             (VALU)
    //   M: PV of step s, scores of step s+1                                                   (MFMA)
    // K(s) is last read in M(s-1) and V(s-1) as well, so both tiles are free in V(s).  One K or V unit is
    // in flight per lane: K travels through an M slot, V through the softmax.
    // Waves 4..7 (slices 2 and 3) run one slot behind waves 0..3 (slices 0 and 1): they pass one barrier
    // more before their first scores and waves 0..3 one more after their last step, so the two waves of a
    // SIMD are in opposite slots.  A slice's tiles are touched by its own two waves only, which are in the
    // same set, so the two barriers per step still separate every write from the reads around it; the Q
    // rows in the V areas of slices 0 and 1 have been read by every wave before waves 0..3 pass their
    // first barrier.  (A wave's step is a chain, so the gain is small: 25.6 against 26.0 us at 672 @ 0.)
    if (wave >= 4)
        lds_barrier();
    scores(0, std::true_type());
    lds_barrier(); // K(0) may be replaced, and every wave has read its Q: the V tiles may be written
    for (int s = 0; s < nstep; s++) {
        const bool more = s + 1 < nstep;
        if (more)
            stage_k();      // K(s + 1)
        issue_v(s);
        softmax(s);
        stage_v();          // V(s)
        issue_k(s + 2);
        lds_barrier();
        pv(s);
        if (more)
            scores(s + 1, std::false_type());
        lds_barrier();
    }
    if (wave < 4)
        lds_barrier(); // (waves 4..7 are in their last M slot)

    // ---- the four slices of a head meet -------------------------------------------------------------
    // Wave `sl` finishes columns 64 sl .. 64 sl + 63 (accumulators 2 sl and 2 sl + 1) of its head.  The
    // gate values of the rows it will write are requested first.
    const int orow = lane >> 4, opiece = lane & 15; // output pass r2: token r2 * 4 + orow, 16-byte piece
    float4v gt[8];
    if (a.gate) {
#pragma unroll
        for (int r2 = 0; r2 < 8; r2++) {
            const int tr = t0 + r2 * 4 + orow;
            gt[r2] = __builtin_nontemporal_load(reinterpret_cast<const float4v *>(
                a.gate + ((size_t)(tr < a.tokens ? tr : a.tokens - 1) * a.n_head + head) * kHeadDim + sl * 64 + opiece * 4));
        }
    }
    l_run += __shfl_xor(l_run, 32);
    float2 *mlx = reinterpret_cast<float2 *>(lds); // [head 2][slice 4][token 32]
    if (lh == 0)
        mlx[(hp * kWgSlices + sl) * kQTile + ln] = make_float2(m_run, l_run);
    float den = 0.0f, w_mine = 0.0f;
    float wj[kWgSlices]; // weight of each slice's sums for this lane's token
    auto weights = [&]() { // (after the first barrier below: the table travels with the first accumulators)
        float m = -INFINITY;
        float2 v[kWgSlices];
#pragma unroll
        for (int j = 0; j < kWgSlices; j++) {
            v[j] = mlx[(hp * kWgSlices + j) * kQTile + ln];
            if (v[j].y > 0.0f)
                m = fmaxf(m, v[j].x);
        }
#pragma unroll
        for (int j = 0; j < kWgSlices; j++) {
            const bool on = v[j].y > 0.0f;
            const float w = on ? __builtin_amdgcn_exp2f(v[j].x - m) : 0.0f;
            den = fmaf(on ? v[j].y : 0.0f, w, den);
            w_mine = j == sl ? w : w_mine;
            wj[j] = w;
        }
    };
    // Two passes, columns 0..127 and 128..255: every wave hands the accumulators it does not finish to
    // the wave that does (the layout is the same in every wave, so lane l writes and reads slot l).
    uint8_t *xbase = lds + kWgXAt;
#pragma unroll
    for (int p = 0; p < 2; p++) {
#pragma unroll
        for (int q2 = 0; q2 < 2; q2++) {
            const int qd = 2 * p + q2;
            if (sl != qd) {
                const int from = sl < qd ? sl : sl - 1;
                float4v *dst = reinterpret_cast<float4v *>(xbase + ((hp * 2 + q2) * 3 + from) * kWgXArea) + lane;
#pragma unroll
                for (int dtl = 0; dtl < 2; dtl++)
#pragma unroll
                    for (int g = 0; g < 4; g++)
                        dst[(dtl * 4 + g) * 64] = (float4v){O[2 * qd + dtl][g * 4], O[2 * qd + dtl][g * 4 + 1],
                                                            O[2 * qd + dtl][g * 4 + 2], O[2 * qd + dtl][g * 4 + 3]};
            }
        }
        lds_barrier();
        if (p == 0)
            weights();
#pragma unroll
        for (int q2 = 0; q2 < 2; q2++) {
            const int qd = 2 * p + q2;
            if (sl == qd) {
                // (the accumulators arrive as they are; each is weighted here, where it is added)
#pragma unroll
                for (int dtl = 0; dtl < 2; dtl++)
                    O[2 * qd + dtl] *= w_mine;
#pragma unroll
                for (int from = 0; from < 3; from++) {
                    const float4v *src =
                        reinterpret_cast<const float4v *>(xbase + ((hp * 2 + q2) * 3 + from) * kWgXArea) + lane;
                    const float w = wj[from < qd ? from : from + 1];
#pragma unroll
                    for (int dtl = 0; dtl < 2; dtl++)
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            const float4v x = src[(dtl * 4 + g) * 64];
#pragma unroll
                            for (int j = 0; j < 4; j++)
                                O[2 * qd + dtl][g * 4 + j] = fmaf(x[j], w, O[2 * qd + dtl][g * 4 + j]);
                        }
                }
            }
        }
        lds_barrier();
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    float16v R[2];
#pragma unroll
    for (int qd = 0; qd < 4; qd++)
        if (sl == qd) {
            R[0] = O[2 * qd];
            R[1] = O[2 * qd + 1];
        }
    // Turned round in this wave's corner of LDS, a store instruction covers four tokens' 256 contiguous bytes.
    uint8_t *mine = xbase + wave * (kQTile * kWgOutPitch);
#pragma unroll
    for (int dtl = 0; dtl < 2; dtl++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4v x = {R[dtl][g * 4] * inv, R[dtl][g * 4 + 1] * inv, R[dtl][g * 4 + 2] * inv,
                               R[dtl][g * 4 + 3] * inv};
            *reinterpret_cast<float4v *>(mine + ln * kWgOutPitch + (dtl * 32 + g * 8 + lh * 4) * 4) = x;
        }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's own writes
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r2 = 0; r2 < 8; r2++) {
        const int r = r2 * 4 + orow;
        float4v x = *reinterpret_cast<const float4v *>(mine + r * kWgOutPitch + opiece * 16);
        if (task_valid && t0 + r < a.tokens) {
            const size_t o = ((size_t)(t0 + r) * a.n_head + head) * kHeadDim + sl * 64 + opiece * 4;
            if (a.gate)
                x = (float4v){gated(x[0], gt[r2][0]), gated(x[1], gt[r2][1]), gated(x[2], gt[r2][2]),
                              gated(x[3], gt[r2][3])};
            if (a.out16)
                *reinterpret_cast<half4 *>(a.out16 + o) = __builtin_convertvector(x, half4);
            else // (non-temporal: 16.5 MB of dirty lines for 672 tokens would otherwise be written back when the
                 // kernel ends, 2.8 us of a 28.6 us launch)
                __builtin_nontemporal_store(x, reinterpret_cast<float4v *>(a.out + o));
        }
    }
}

// Fold the key slices: one workgroup per (token, 4 heads); thread = (head, float4 of d).  A (token,
// head) whose task block has a single slice was written by the attention kernel itself.
// out16 != nullptr: the finished rows go there as f16 (round to nearest even), the operand form of
// the output projection, and `out` only carries the single-slice rows in from the attention kernel.
__global__ void __launch_bounds__(256) chunk_combine_kernel(
    const float *__restrict__ part_acc, const float *__restrict__ part_ml, float *out,
    const float *__restrict__ gate, int n_head, int qslots, int splits, int group, int ntask, int tokens,
    int pos0, int slice_tiles, int uniform, _Float16 *__restrict__ out16)
{
    const int tok = blockIdx.x;
    const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int d4 = (threadIdx.x & 63) * 4;
    if (head >= n_head)
        return;
    const size_t o = ((size_t)tok * n_head + head) * kHeadDim + d4;
    int nsp = splits;
    if (!uniform) {
        const int task = (tok / kQTile) * group + head % group;
        nsp = block_slices(task / kTasks, ntask, group, tokens, pos0, splits, slice_tiles, nullptr);
        if (nsp == 1) {
            if (gate || out16) {
                float4v x = *reinterpret_cast<const float4v *>(out + o);
                if (gate) {
                    const float4v gt = *reinterpret_cast<const float4v *>(gate + o);
                    x = (float4v){gated(x[0], gt[0]), gated(x[1], gt[1]), gated(x[2], gt[2]), gated(x[3], gt[3])};
                }
                if (out16)
                    *reinterpret_cast<half4 *>(out16 + o) = __builtin_convertvector(x, half4);
                else
                    *reinterpret_cast<float4v *>(out + o) = x;
            }
            return;
        }
    }
    float4v num = {0, 0, 0, 0};
    float den = 0.0f;
    const float4v z = {0, 0, 0, 0};
    float4v gt = {0, 0, 0, 0};
    if (gate)
        gt = *reinterpret_cast<const float4v *>(gate + o);
    if (nsp <= 4) {
        // every slice's (max, sum) and accumulator row asked for before the first is used
        float2 ml[4];
        float4v x[4];
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const size_t row = ((size_t)(s < nsp ? s : 0) * qslots + tok) * n_head + head;
            ml[s] = *reinterpret_cast<const float2 *>(part_ml + row * 2);
            x[s] = *reinterpret_cast<const float4v *>(part_acc + row * kHeadDim + d4);
        }
        float m = -INFINITY;
#pragma unroll
        for (int s = 0; s < 4; s++)
            if (s < nsp && ml[s].y > 0.0f)
                m = fmaxf(m, ml[s].x);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const bool on = s < nsp && ml[s].y > 0.0f;
            const float w = on ? __builtin_amdgcn_exp2f(ml[s].x - m) : 0.0f;
            num += on ? x[s] * w : z;
            den = fmaf(on ? ml[s].y : 0.0f, w, den);
        }
    } else if (nsp <= 16) {
        // up to 16 slices: every (max, sum) pair first, then the accumulator rows four at a time, each
        // group asked for before its first row is used
        float2 ml[16];
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const size_t row = ((size_t)(s < nsp ? s : 0) * qslots + tok) * n_head + head;
            ml[s] = *reinterpret_cast<const float2 *>(part_ml + row * 2);
        }
        float m = -INFINITY;
#pragma unroll
        for (int s = 0; s < 16; s++)
            if (s < nsp && ml[s].y > 0.0f)
                m = fmaxf(m, ml[s].x);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (g * 4 < nsp) { // uniform over the workgroup's threads of this head
                float4v x[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int sl = g * 4 + i;
                    const size_t row = ((size_t)(sl < nsp ? sl : 0) * qslots + tok) * n_head + head;
                    x[i] = *reinterpret_cast<const float4v *>(part_acc + row * kHeadDim + d4);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int sl = g * 4 + i;
                    const bool on = sl < nsp && ml[sl].y > 0.0f;
                    const float w = on ? __builtin_amdgcn_exp2f(ml[sl].x - m) : 0.0f;
                    num += on ? x[i] * w : z;
                    den = fmaf(on ? ml[sl].y : 0.0f, w, den);
                }
            }
        }
    } else {
        float m = -INFINITY;
        for (int s = 0; s < nsp; s++) {
            const size_t row = ((size_t)s * qslots + tok) * n_head + head;
            const float2 ml = *reinterpret_cast<const float2 *>(part_ml + row * 2);
            if (ml.y > 0.0f)
                m = fmaxf(m, ml.x);
        }
        for (int s = 0; s < nsp; s++) {
            const size_t row = ((size_t)s * qslots + tok) * n_head + head;
            const float2 ml = *reinterpret_cast<const float2 *>(part_ml + row * 2);
            const float4v x = *reinterpret_cast<const float4v *>(part_acc + row * kHeadDim + d4);
            const float w = ml.y > 0.0f ? __builtin_amdgcn_exp2f(ml.x - m) : 0.0f;
            num += ml.y > 0.0f ? x * w : z;
            den = fmaf(ml.y > 0.0f ? ml.y : 0.0f, w, den);
        }
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    float4v r = num * inv;
    if (!(den > 0.0f))
        r = (float4v){0, 0, 0, 0};
    if (gate)
        r = (float4v){gated(r[0], gt[0]), gated(r[1], gt[1]), gated(r[2], gt[2]), gated(r[3], gt[3])};
    if (out16)
        *reinterpret_cast<half4 *>(out16 + o) = __builtin_convertvector(r, half4);
    else
        *reinterpret_cast<float4v *>(out + o) = r;
}

// f16 copy of finished f32 rows (the unsplit path with an f16 destination), 4 values per thread.
__global__ void __launch_bounds__(256) rows_f16_kernel(const float4v *__restrict__ x, half4 *__restrict__ y, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4)
        y[i] = __builtin_convertvector(x[i], half4);
}

// The f16 copy of 64-key tiles of a cache: what a chunk workgroup would stage for itself, made once.
// grid (tiles, n_kv, 2); tile = tile0 + blockIdx.x; rows at or past seq_end repeat row seq_end - 1 (the
// attention kernels mask them; a later call that brings the rows overwrites the tile).
// The K rows leave as they lie in LDS; the V tile leaves through the transposing reads of the PV
// product, so row d of the copy holds, for every 16 keys, the eight values of k-group 0 and the eight
// of k-group 1 in operand order (key (j/4)*8 + g*4 + j%4 of the sixteen at position g*8 + j).
template <bool Q4>
__global__ void __launch_bounds__(256) kv_f16_tiles_kernel(const uint8_t *__restrict__ kc,
                                                           const uint8_t *__restrict__ vc, uint8_t *__restrict__ k16,
                                                           uint8_t *__restrict__ vt, int stride, int tile0,
                                                           int seq_end, int tile_stride)
{
    // grid (tiles, n_kv, 2): blockIdx.z = 0 makes the K tile, 1 the V^T tile (35 KB of LDS either way: four
    // workgroups per CU, which this pass needs more than anything else: it is all latency)
    typedef typename HalfOf<Q4>::type Half;
    constexpr int kRowBytes = Q4 ? hipml::kRowBytesQ4 : hipml::kRowBytes;
    constexpr int kUnitBytes = Q4 ? 36 : 68;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tile = tile0 + blockIdx.x;
    const int kvh = blockIdx.y;
    const bool v_tile = blockIdx.z != 0;
    const int su = threadIdx.x;
    const int lane = su & 63, wave = su >> 6;
    // thread -> (row, unit) as in the chunk kernel's staging: conflict-free 128-bit LDS writes
    const int srow = (su >> 6) * 16 + ((su >> 1) & 7) + ((su >> 5) & 1) * 8;
    const int spr = (su & 1) | ((su >> 3) & 2);
    int key = tile * kKTile + srow;
    key = key < seq_end ? key : seq_end - 1;
    const size_t src = ((size_t)kvh * stride + key) * kRowBytes + spr * kUnitBytes;
    const uint8_t *from_cache = (v_tile ? vc : kc) + src;
    Half h0, h1;
    load_half0(h0, from_cache);
    load_half1(h1, from_cache);
    uint8_t *sd = lds + srow * (v_tile ? kVRow : kKRow) + spr * 128;
    stage_block0(h0, sd);
    stage_block1(h1, sd);
    __syncthreads();
    const size_t at = (size_t)kvh * tile_stride + tile;
    if (!v_tile) {
        const uint4v *from = reinterpret_cast<const uint4v *>(lds);
        uint4v *to = reinterpret_cast<uint4v *>(k16 + at * kKTileBytes);
        for (int i = su; i < kKTileBytes / 16; i += 256)
            to[i] = from[i];
    } else {
        const int ln = lane & 31, lh = lane >> 5, gl = lane & 15;
        const int vtr_off = (gl >> 2) * kVRow + (((lane >> 4) & 1) * 16 + (gl & 3) * 4) * 2;
        uint8_t *to = vt + at * kVtTileBytes;
#pragma unroll
        for (int o8 = 0; o8 < 8; o8++) {
            const int o = wave * 8 + o8; // operand (half hk, step u, d tile dt) of the tile's 32
            const int hk = o >> 4, u = (o >> 3) & 1, dt = o & 7;
            const uint8_t *vp = lds + vtr_off + hk * 32 * kVRow + dt * 64;
            const short4v r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (short4v __attribute__((address_space(3))) *)(vp + ((2 * u) * 8 + lh * 4) * kVRow));
            const short4v r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (short4v __attribute__((address_space(3))) *)(vp + ((2 * u + 1) * 8 + lh * 4) * kVRow));
            const uint32_t *w0 = reinterpret_cast<const uint32_t *>(&r0), *w1 = reinterpret_cast<const uint32_t *>(&r1);
            const uint4v piece = {w0[0], w0[1], w1[0], w1[1]};
            *reinterpret_cast<uint4v *>(to + (dt * 32 + ln) * kVtRow + (hk * 32 + u * 16 + lh * 8) * 2) = piece;
        }
    }
}

size_t kv_f16_bytes(int stride, int n_kv)
{
    const size_t tiles = ((size_t)stride + kKTile - 1) / kKTile;
    return (size_t)n_kv * tiles * kBufBytesF;
}

// Tiles tile0 .. of a copy with tile_stride tiles per KV head, from cache rows below seq_end.
static int launch_kv_f16_tiles(hipStream_t st, const uint8_t *kc, const uint8_t *vc, void *copy, int n_kv, int stride,
                               int tile_stride, int start, int seq_end, int q4)
{
    uint8_t *k16 = static_cast<uint8_t *>(copy);
    uint8_t *vt = k16 + (size_t)n_kv * tile_stride * kKTileBytes;
    const int tile0 = start / kKTile, tile1 = (seq_end + kKTile - 1) / kKTile;
    const dim3 grid((unsigned)(tile1 - tile0), (unsigned)n_kv, 2);
    if (q4)
        HIPML_LAUNCH(kv_f16_tiles_kernel<true>, grid, dim3(256, 1, 1), kTilesLds, st, kc, vc, k16, vt, stride,
                           tile0, seq_end, tile_stride);
    else
        HIPML_LAUNCH(kv_f16_tiles_kernel<false>, grid, dim3(256, 1, 1), kTilesLds, st, kc, vc, k16, vt, stride,
                           tile0, seq_end, tile_stride);
    return launched("kv_f16_rows");
}

int launch_kv_f16_rows(hipStream_t st, const uint8_t *kc, const uint8_t *vc, void *copy, int n_kv, int stride,
                       int start, int rows, int q4)
{
    if (rows < 1)
        return 0;
    return launch_kv_f16_tiles(st, kc, vc, copy, n_kv, stride, (stride + kKTile - 1) / kKTile, start, start + rows, q4);
}

int prefill_init()
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_q8_kernel<false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kPfLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_q8_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kPfLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_q8_kernel<false, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kPfLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_q8_kernel<true, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kPfLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_q8_kernel<false, false, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kPfLdsF);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_q8_kernel<true, false, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kPfLdsF);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_f16_t64_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kT64Lds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&kv_f16_tiles_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kTilesLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&kv_f16_tiles_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kTilesLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_wg_kernel<false, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kWgLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_wg_kernel<true, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kWgLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_wg_kernel<false, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kWgLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chunk_wg_kernel<true, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kWgLds);
    if (e != hipSuccess)
        return fail((int)e, "hipFuncSetAttribute(prefill LDS) failed: %d (%s)", (int)e,
                    hipGetErrorString(e));
    return 0;
}

// Deep in a prefix a sliced chunk over the cache runs faster as two steps: the live rows of the cache are first
// written out as f16 tiles (what hipml_kv_f16_rows makes) into the tail of the caller's partial-row scratch, and
// the attention then runs over those with the 64-token kernel and fewer slices.  That needs a scratch sized for
// more slices than the attention uses: `splits` (the count the scratch was sized for) must cover `*use` slices
// of partial rows plus the tiles, which start at byte *tiles_at of part_acc.  hipml_attn_chunk_splits returns
// such a count where the detour pays (the pass over the cache costs 1.3 us per 1,000 rows, the kernel of 32
// tokens per wave with its own dequantization 15 % of the attention; measured gain, 2,048 tokens at depth
// 2,048 / 8,192 / 16,384 / 100,000: 13 / 10 / 11 / 13 %, 1,024 tokens at 2,048 / 8,192: 3 / 4 %, 768 tokens at
// 3,072 / 6,144: 0.5 / 3 %); with any smaller count the chunk runs as before.
// Where the detour pays: chunks of 768 tokens or more behind a prefix at least as long, and chunks of 640 or
// more (the 672 tokens of the usual prefill chunk) behind a prefix of eight times their length (672 tokens at
// depth 672 / 2,048 / 8,192 / 32,768 / 100,000: -3 / -3 / +5 / +7 / +6 %).
bool chunk_tiles_pay(int pos0, int tokens)
{
    return (tokens >= 768 && pos0 >= tokens) || (tokens >= 640 && pos0 >= 8 * tokens);
}

bool chunk_tiles_plan(int pos0, int tokens, int n_head, int n_kv, int splits, int *use, size_t *tiles_at)
{
    if (!chunk_tiles_pay(pos0, tokens) || splits < 3)
        return false;
    const int s = hipml_attn_chunk_slices(pos0, tokens, n_kv);
    if (s < 2)
        return false;
    const size_t per_slice = (size_t)((tokens + 31) / 32 * 32) * n_head * kHeadDim * sizeof(float);
    const size_t tiles = (size_t)n_kv * ((pos0 + tokens + kKTile - 1) / kKTile) * kBufBytesF;
    if ((size_t)splits * per_slice < (size_t)s * per_slice + tiles)
        return false;
    *use = s;
    *tiles_at = (size_t)s * per_slice;
    return true;
}

int chunk_tiles_splits(int pos0, int tokens, int n_head, int n_kv, int slices)
{
    const size_t per_slice = (size_t)((tokens + 31) / 32 * 32) * n_head * kHeadDim * sizeof(float);
    const size_t tiles = (size_t)n_kv * ((pos0 + tokens + kKTile - 1) / kKTile) * kBufBytesF;
    return slices + (int)((tiles + per_slice - 1) / per_slice);
}

int launch_chunk_q8(hipStream_t st, const float *q, const uint8_t *kc, const uint8_t *vc,
                    float *out, int n_head, int n_kv, int pos0, int tokens, int stride,
                    float *part_acc, float *part_ml, int splits, const float *gate, int q4, void *out16,
                    const void *kv_f16, const float *rope_tab)
{
    {
        int use;
        size_t tiles_at;
        if (kv_f16 == nullptr && rope_tab == nullptr &&
            chunk_tiles_plan(pos0, tokens, n_head, n_kv, splits, &use, &tiles_at)) {
            const int live_tiles = (pos0 + tokens + kKTile - 1) / kKTile;
            uint8_t *tiles = reinterpret_cast<uint8_t *>(part_acc) + tiles_at;
            if (int rc = launch_kv_f16_tiles(st, kc, vc, tiles, n_kv, stride, live_tiles, 0, pos0 + tokens, q4))
                return rc;
            return launch_chunk_q8(st, q, kc, vc, out, n_head, n_kv, pos0, tokens, live_tiles * kKTile, part_acc,
                                   part_ml, use, gate, 0, out16, tiles, nullptr);
        }
        // A count that was meant to hold the tiles but does not (hipml_attn_chunk_splits assumes 6 heads per KV
        // head; fewer make the partial rows, and with them the room per slice, smaller): the extra slices are
        // not slices to run.  The kernel that dequantizes for itself gets the count it would have been given.
        if (kv_f16 == nullptr && rope_tab == nullptr && splits >= 3 && chunk_tiles_pay(pos0, tokens) &&
            n_head / n_kv < 6) {
            const int s = hipml_attn_chunk_slices(pos0, tokens, n_kv);
            if (s >= 2 && s < splits && splits == chunk_tiles_splits(pos0, tokens, 6 * n_kv, n_kv, s))
                splits = s;
        }
    }
    // rope_tab != nullptr (splits == 0 only): q holds unrotated rows, the kernel rotates them as it loads them
    ChunkArgs a;
    // kv_f16 != nullptr: K and V are read from the f16 copy of the cache (kc, vc unused)
    a.tile_stride = (stride + kKTile - 1) / kKTile;
    a.k16 = static_cast<const uint8_t *>(kv_f16);
    a.vt = a.k16 + (size_t)n_kv * a.tile_stride * kKTileBytes;
    a.gate = gate;
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
    a.splits = splits < 2 ? 1 : splits;
    a.qslots = (tokens + 31) / 32 * 32;
    a.ntask = (tokens + kQTile - 1) / kQTile * a.group;
    a.nblock = (a.ntask + kTasks - 1) / kTasks;
    a.scale_log2 = kLog2e / 16.0f; // 1/sqrt(256), as the reference's chunk launcher fixes it
    a.out16 = nullptr;
    if (splits == 0 && kv_f16 == nullptr) {
        // the key slices stay inside the workgroup: no partial rows, gate and f16 rows in the same launch
        a.out16 = static_cast<_Float16 *>(out16);
        const unsigned wgs = (unsigned)((tokens + kQTile - 1) / kQTile * n_kv * ((a.group + 1) / 2));
        a.rope_tab = rope_tab;
        if (q4 && rope_tab)
            HIPML_LAUNCH((chunk_wg_kernel<true, true>), dim3(wgs, 1, 1), dim3(kPfThreads, 1, 1), kWgLds, st, a);
        else if (q4)
            HIPML_LAUNCH((chunk_wg_kernel<true, false>), dim3(wgs, 1, 1), dim3(kPfThreads, 1, 1), kWgLds, st, a);
        else if (rope_tab)
            HIPML_LAUNCH((chunk_wg_kernel<false, true>), dim3(wgs, 1, 1), dim3(kPfThreads, 1, 1), kWgLds, st, a);
        else
            HIPML_LAUNCH((chunk_wg_kernel<false, false>), dim3(wgs, 1, 1), dim3(kPfThreads, 1, 1), kWgLds, st, a);
        return launched(q4 ? "attn_chunk_q4_wg" : "attn_chunk_q8_wg");
    }
    // slices per block: the last block (most keys) gets `splits`, a block with fewer key tiles gets
    // proportionally fewer, so a chunk near position 0 does not write and re-read `splits` partial
    // copies of rows that see only a few tiles
    const int tiles_last = (pos0 + tokens + kKTile - 1) / kKTile;
    a.slice_tiles = (tiles_last + a.splits - 1) / a.splits;
    a.nslice = 0;
    for (int tb = 0; tb < a.nblock; tb++)
        a.nslice += block_slices(tb, a.ntask, a.group, tokens, pos0, a.splits, a.slice_tiles, nullptr);
    a.uniform = a.nslice == a.nblock * a.splits;
    const dim3 block(kPfThreads, 1, 1);
    unsigned grid;
    if (a.splits > 1 && !a.uniform) {
        grid = (unsigned)(n_kv * a.nslice);
    } else {
        // grid.x covers every (combo, task block); the XCD-aware decode in the kernel may leave a
        // few trailing workgroups without work when 8 is not a multiple of `combos`.
        const int combos = n_kv * a.splits;
        if (combos % 8 == 0)
            grid = (unsigned)(combos * a.nblock);
        else if (8 % combos == 0)
            grid = (unsigned)(8 * ((a.nblock + 8 / combos - 1) / (8 / combos)));
        else
            grid = (unsigned)(combos * a.nblock);
    }
    if (splits < 2) {
        if (kv_f16)
            HIPML_LAUNCH((chunk_q8_kernel<false, false, true>), dim3(grid, 1, 1), block, kPfLdsF, st, a);
        else if (q4)
            HIPML_LAUNCH((chunk_q8_kernel<false, true>), dim3(grid, 1, 1), block, kPfLds, st, a);
        else
            HIPML_LAUNCH(chunk_q8_kernel<false>, dim3(grid, 1, 1), block, kPfLds, st, a);
        int rc = launched(kv_f16 ? "attn_chunk_f16" : q4 ? "attn_chunk_q4" : "attn_chunk_q8");
        if (rc || out16 == nullptr)
            return rc;
        const size_t n4 = (size_t)tokens * n_head * kHeadDim / 4;
        HIPML_LAUNCH(rows_f16_kernel, dim3((unsigned)((n4 + 255) / 256), 1, 1), dim3(256, 1, 1), 0, st,
                           reinterpret_cast<const float4v *>(out), static_cast<half4 *>(out16), n4);
        return launched("attn_chunk_rows_f16");
    }
    // 64 tokens per wave: its own task blocks (4 tasks of 64 tokens), every one with `splits` slices.  Both
    // kernels run one workgroup per CU, so the hardware starts them in rounds of 256; where the other cut of
    // the tokens needs a round more, the kernel of 32 tokens per wave keeps the chunk.
    ChunkArgs b = a;
    {
        const int rem = tokens % kT64Tile; // (up to 32 left-over tokens: tasks of 32 tokens x 2 heads, see the kernel)
        b.ntask = (tokens / kT64Tile + (rem > 32 ? 1 : 0)) * a.group + (rem > 0 && rem <= 32 ? (a.group + 1) / 2 : 0);
    }
    b.nblock = (b.ntask + kT64Tasks - 1) / kT64Tasks;
    unsigned g64 = (unsigned)(n_kv * a.splits * b.nblock);
    if ((n_kv * a.splits) % 8 != 0 && 8 % (n_kv * a.splits) == 0)
        g64 = (unsigned)(8 * ((b.nblock + 8 / (n_kv * a.splits) - 1) / (8 / (n_kv * a.splits))));
    if (kv_f16 && a.uniform && (g64 + 255) / 256 <= (grid + 255) / 256) {
        HIPML_LAUNCH(chunk_f16_t64_kernel, dim3(g64, 1, 1), dim3(kT64Threads, 1, 1), kT64Lds, st, b);
    } else if (kv_f16)
        HIPML_LAUNCH((chunk_q8_kernel<true, false, true>), dim3(grid, 1, 1), block, kPfLdsF, st, a);
    else if (q4)
        HIPML_LAUNCH((chunk_q8_kernel<true, true>), dim3(grid, 1, 1), block, kPfLds, st, a);
    else
        HIPML_LAUNCH(chunk_q8_kernel<true>, dim3(grid, 1, 1), block, kPfLds, st, a);
    int rc = launched(kv_f16 ? "attn_chunk_f16_split" : q4 ? "attn_chunk_q4_split" : "attn_chunk_q8_split");
    if (rc)
        return rc;
    HIPML_LAUNCH(chunk_combine_kernel, dim3((unsigned)tokens, (unsigned)((n_head + 3) / 4), 1),
                       dim3(256, 1, 1), 0, st, part_acc, part_ml, out, gate, n_head, a.qslots, a.splits, a.group,
                       a.ntask, tokens, pos0, a.slice_tiles, a.uniform, static_cast<_Float16 *>(out16));
    return launched("attn_chunk_combine");
}

} // namespace hipml
